// BF16 weight GEMM for 9 to 64 rows (gfx950): the projections of a decode or verify step with more rows than the
// GEMV takes. Like the GEMV it is bound by the weight stream - every weight byte is read from HBM once with 128-bit
// nontemporal loads - but the arithmetic runs on the matrix cores: with sixteen rows a weight piece of 1 KiB is one
// v_mfma_f32_16x16x32_bf16, so the vector units, which bound the GEMV from five rows up, do nothing here.
//
// The reference has no kernel for this range: its engine calls the vendor GEMM above 8 rows (crates/glm53f-forward/
// src/gemm.rs:228-234, :293-325). What this replaces there is that call, for 9..64 rows.
//
// Numerics: exact bf16 products, f32 accumulation on the matrix core over K in steps of 32 inside a wave's K range,
// the ranges of a workgroup's waves added in wave order; bf16 outputs rounded to nearest even. A row's result does
// not depend on the rows beside it or on their number. No bit-level contract (the reference has none above 8 rows: its own test holds
// the vendor GEMM to the GEMV within f32 rounding).
//
// Shape of the work. A workgroup owns T tiles of sixteen outputs; its KS waves split the K range; a wave walks its
// range in chunks of CK. Both operands reach the matrix core's fragment layout (lane l: row l % 16, k = 8 (l / 16)
// .. + 7 of a step of 32) through LDS, because the layout's natural load - sixteen rows of 64 bytes per instruction
// - asks the texture path for 64 cache lines per KiB: a kernel that loads fragments directly, activations from the
// L2 in the same way, reaches 2.9 TB/s of weights on 4096 -> 24,640 with sixteen rows, this one 6.4 TB/s. Here
//   - a load instruction covers whole runs of a row (CK = 256: two rows of 512 consecutive bytes, lanes 0..31 one
//     row, 32..63 the next; CK = 128: four rows of 256 bytes), CK / 32 of them a tile of sixteen rows x CK; the
//     wave writes the tile to its own LDS rows (2 CK + 16 bytes apart: a fragment read's sixteen rows then fall on
//     all 64 banks once) and reads it back as CK / 32 fragments. No workgroup barrier: a wave's LDS instructions
//     run in order, and the region is its own;
//   - the activations' tiles (NT of sixteen rows) go the same way once per chunk and stay in registers for the T
//     weight tiles, so their traffic from the L2 is NT / T of the weight stream;
//   - two sets of loads alternate over the items of a chunk (the NT activation tiles, then the T weight tiles):
//     the next item is requested before the current one is waited for.
// The launch takes T so that the grid is at most one workgroup per CU where the registers allow (measured: one
// round of 193 workgroups of four waves at T = 8 runs 4096 -> 24,640 in 31.3 us, 385 at T = 4 in 33.6, and 257 at
// T = 6 - one more than the CUs, so a second round of one - in 40.7).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "glm53f_fwd_gemv.h"

namespace fwd_gemm {
namespace {

constexpr int kInvalid = 1;                       // hipErrorInvalidValue
constexpr int kCus = 256;

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t f2bf2(float lo, float hi) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf2));
}

template <int CK> struct Staged {
    static constexpr int N8 = CK / 32;            // loads of an item = fragments of an item
    static constexpr int LANES = CK / 8;          // lanes that cover one row's CK elements with 16 bytes each
    static constexpr int ROW = 2 * CK + 16;       // bytes between a staged tile's rows
    static constexpr int BYTES = 16 * ROW;        // a wave's staging region
};

// CK: k per chunk. NT: tiles of sixteen rows (rows <= 16 NT). T: tiles of sixteen outputs per workgroup. KS: waves
// of a workgroup, each with k / KS of the K range (a multiple of CK).
template <int CK, int NT, int T, int KS>
__global__ void __launch_bounds__(64 * KS) stream_kernel(const uint16_t* __restrict__ x, long long ldx, long long x_gs,
                                                         const uint16_t* __restrict__ w, long long ldw, long long w_gs,
                                                         int rows, int n, int k, void* __restrict__ out, int out_f32,
                                                         long long ldo, long long o_gs) {
    using S = Staged<CK>;
    constexpr int N8 = S::N8, RPL = 64 / S::LANES, NI = NT + T;
    constexpr int PART = KS * T * NT * 1024;      // the partial tiles reuse the staging regions
    constexpr int LDS_BYTES = KS * S::BYTES > PART ? KS * S::BYTES : PART;
    __shared__ __align__(16) unsigned char lds[LDS_BYTES];
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int g = blockIdx.z, tiles = n / 16, tile0 = blockIdx.x * T;
    const int row0 = blockIdx.y * (16 * NT);      // gridDim.y > 1: the rows in groups of 16 NT, a workgroup each
    rows = min(rows - row0, 16 * NT);
    const int kc = k / KS, lo = wave * kc, chunks = kc / CK;
    const int lrow = lane / S::LANES, lcol = 8 * (lane % S::LANES);
    unsigned char* stage = lds + wave * S::BYTES;
    unsigned char* put = stage + lrow * S::ROW + 2 * lcol;                        // + RPL j rows
    const unsigned char* get = stage + (lane & 15) * S::ROW + 16 * (lane >> 4);   // + 64 s

    // items 0 .. NT - 1 of a chunk: the activations' tiles (a row past the end repeats the last one: its column
    // is not stored); item NT + i: weight tile i of this workgroup (a tile past the last repeats it, not stored)
    const uint16_t* xsrc = x + g * x_gs + (long long)row0 * ldx + lo + lcol;
    const uint16_t* wsrc = w + g * w_gs + (long long)lrow * ldw + lo + lcol;
    auto request = [&](u32x4 (&set)[N8], int item, int c) {
        if (item < NT) {
#pragma unroll
            for (int j = 0; j < N8; ++j)
                set[j] = *reinterpret_cast<const u32x4*>(xsrc + (long long)min(16 * item + RPL * j + lrow, rows - 1) * ldx + CK * c);
        } else {
            const uint16_t* src = wsrc + (long long)(16 * min(tile0 + item - NT, tiles - 1)) * ldw + CK * c;
#pragma unroll
            for (int j = 0; j < N8; ++j)
                set[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + (long long)(RPL * j) * ldw));
        }
    };
    auto fragments = [&](const u32x4 (&set)[N8], u32x4 (&frag)[N8]) {
#pragma unroll
        for (int j = 0; j < N8; ++j) *reinterpret_cast<u32x4*>(put + RPL * j * S::ROW) = set[j];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int s = 0; s < N8; ++s) frag[s] = *reinterpret_cast<const u32x4*>(get + 64 * s);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    f32x4 acc[T][NT];
#pragma unroll
    for (int i = 0; i < T; ++i)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[i][nt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    u32x4 xf[NT][N8];

    // One chunk: `first` holds (or has in flight) the chunk's item 0, the sets alternate from there; the item
    // after the chunk's last (the next chunk's item 0; after the last chunk a repeat, not used) goes to the set
    // that the next call names `first`.
    auto chunk = [&](u32x4 (&first)[N8], u32x4 (&second)[N8], int c) {
#pragma unroll
        for (int item = 0; item < NI; ++item) {
            u32x4 (&cur)[N8] = (item & 1) ? second : first;
            u32x4 (&nxt)[N8] = (item & 1) ? first : second;
            if (item + 1 < NI) request(nxt, item + 1, c);
            else request(nxt, 0, min(c + 1, chunks - 1));
            if (item < NT) {
                fragments(cur, xf[item]);
            } else {
                u32x4 wf[N8];
                fragments(cur, wf);
#pragma unroll
                for (int s = 0; s < N8; ++s)
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        f32x4& a = acc[item - NT][nt];
                        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wf[s]),
                                                                    __builtin_bit_cast(bf16x8, xf[nt][s]), a, 0, 0, 0);
                    }
            }
        }
    };
    u32x4 sa[N8], sb[N8];
    request(sa, 0, 0);
    if constexpr (NI % 2 == 0) {                  // an even number of items: every chunk starts on the same set
        for (int c = 0; c < chunks; ++c) chunk(sa, sb, c);
    } else {
        int c = 0;
        for (; c + 1 < chunks; c += 2) {
            chunk(sa, sb, c);
            chunk(sb, sa, c + 1);
        }
        if (c < chunks) chunk(sa, sb, c);
    }

    // acc[i][nt][e] = C[output 16 (tile0 + i) + 4 (lane / 16) + e][row 16 nt + lane % 16]: the waves' partial tiles,
    // added in wave order (the staging regions are free once every wave has left the loop)
    float* part = reinterpret_cast<float*>(lds);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < T; ++i)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            *reinterpret_cast<f32x4*>(&part[(((wave * T + i) * NT + nt) * 64 + lane) * 4]) = acc[i][nt];
    __syncthreads();
    for (int e = t; e < T * NT * 64; e += 64 * KS) {
        const int tn = e >> 6, l = e & 63, i = tn / NT, nt = tn % NT;
        f32x4 s = *reinterpret_cast<const f32x4*>(&part[(tn * 64 + l) * 4]);
#pragma unroll
        for (int kk = 1; kk < KS; ++kk) {
            const f32x4 p = *reinterpret_cast<const f32x4*>(&part[((kk * T * NT + tn) * 64 + l) * 4]);
            s = f32x4{s[0] + p[0], s[1] + p[1], s[2] + p[2], s[3] + p[3]};
        }
        const int row = 16 * nt + (l & 15), o = 16 * (tile0 + i) + 4 * (l >> 4);
        if (row >= rows || tile0 + i >= tiles) continue;
        if (out_f32) {
            float* dst = static_cast<float*>(out) + g * o_gs + (long long)(row0 + row) * ldo + o;
            dst[0] = s[0]; dst[1] = s[1]; dst[2] = s[2]; dst[3] = s[3];
        } else {
            uint32_t* dst = reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(out) + g * o_gs + (long long)(row0 + row) * ldo + o);
            dst[0] = f2bf2(s[0], s[1]);
            dst[1] = f2bf2(s[2], s[3]);
        }
    }
}

struct Args {
    const uint16_t* x; long long ldx, x_gs;
    const uint16_t* w; long long ldw, w_gs;
    int groups, rows, n, k;
    void* out; int out_f32; long long ldo, o_gs;
    hipStream_t stream;
};

template <int CK, int NT, int T, int KS>
int32_t launch(const Args& a) {
    const dim3 grid((unsigned)((a.n / 16 + T - 1) / T), (unsigned)((a.rows + 16 * NT - 1) / (16 * NT)), (unsigned)a.groups);
    stream_kernel<CK, NT, T, KS><<<grid, 64 * KS, 0, a.stream>>>(a.x, a.ldx, a.x_gs, a.w, a.ldw, a.w_gs, a.rows, a.n, a.k,
                                                                 a.out, a.out_f32, a.ldo, a.o_gs);
    return (int32_t)hipGetLastError();
}

// T: the power of two (at most TMAX) that brings the grid nearest to one workgroup per CU from above.
template <int CK, int NT, int KS, int TMAX>
int32_t launch_tiles(const Args& a) {
    const long long tiles = (long long)(a.n / 16) * a.groups;
    if constexpr (TMAX >= 8) if (tiles > 4 * kCus) return launch<CK, NT, 8, KS>(a);
    if constexpr (TMAX >= 4) if (tiles > 2 * kCus) return launch<CK, NT, 4, KS>(a);
    if constexpr (TMAX >= 2) if (tiles > kCus) return launch<CK, NT, 2, KS>(a);
    return launch<CK, NT, 1, KS>(a);
}

// The K split depends on n and k alone, so a row's bits do not change with the number of rows beside it: eight waves
// where the grid is at most one workgroup per CU even at one tile each (more loads in flight per CU), four otherwise,
// one where the K range is too short to split into chunks. The chunk is 256 k where the wave's range is a multiple
// of it and, with eight waves, where sixteen rows leave the registers for it; with four waves the workgroup may
// run alone on its CU (eight weight tiles x four row tiles: 426 registers, the accumulators in the AGPRs), which
// pays because the activations' L2 traffic falls with the tiles per workgroup: 4096 -> 24,640 with 64 rows
// 38 us at eight tiles against 45 at four.
template <int NT, int TMAX>
int32_t launch_split(const Args& a) {
    const long long tiles = (long long)(a.n / 16) * a.groups;
    if (tiles <= kCus && a.k % (8 * 128) == 0) {
        // A weight so small that a workgroup per tile and per sixteen rows still leaves CUs free (the gates' first
        // projection: 16 tiles) is bound by a wave's chain of items, not by bytes: the row tiles go to workgroups of
        // their own, which re-read the weight from the L2 (4096 -> 256 with 64 rows: 11 -> 6 us).
        if (a.k % (8 * 256) == 0 && (NT == 1 || tiles * NT <= kCus)) return launch<256, 1, 1, 8>(a);
        return launch<128, NT, 1, 8>(a);
    }
    if (a.k % (4 * 128) == 0) {
        if (a.k % (4 * 256) == 0) return launch_tiles<256, NT, 4, 8>(a);
        return launch_tiles<128, NT, 4, TMAX>(a);
    }
    return launch_tiles<128, NT, 1, TMAX>(a);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace
}  // namespace fwd_gemm

extern "C" int32_t glm53f_fwd_gemm_bf16_skinny(const uint16_t* x, int64_t ldx, int64_t x_gstride, const uint16_t* w,
                                               int64_t ldw, int64_t w_gstride, int32_t groups, int32_t rows, int32_t n,
                                               int32_t k, void* out, int32_t out_f32, int64_t ldo, int64_t o_gstride,
                                               ihipStream_t* stream) {
    using namespace fwd_gemm;
    if (groups < 1 || groups > 65535 || rows < 1 || rows > 64 || n < 16 || n % 16 || k < 128 || k % 128) return kInvalid;
    if (!x || !w || !out || !aligned16(x) || !aligned16(w) || ldx % 8 || ldw % 8 || x_gstride % 8 || w_gstride % 8 ||
        ldx < k || ldw < k || ldo < n)
        return kInvalid;
    // bf16 outputs are stored two at a time (32 bits), f32 outputs one at a time
    if (!out_f32 && ((reinterpret_cast<uintptr_t>(out) & 3u) || ldo % 2 || o_gstride % 2)) return kInvalid;
    if (out_f32 && (reinterpret_cast<uintptr_t>(out) & 3u)) return kInvalid;
    const Args a{x, ldx, x_gstride, w, ldw, w_gstride, groups, rows, n, k, out, out_f32, ldo, o_gstride, stream};
    switch ((rows + 15) / 16) {                   // (the last argument bounds T where the chunk is 128 k)
        case 1: return launch_split<1, 8>(a);
        case 2: return launch_split<2, 4>(a);
        default: return launch_split<4, 4>(a);    // 33 to 48 rows too: a third tile's seven items per chunk need more
                                                  // registers than a fourth tile of repeated rows costs
    }
}
