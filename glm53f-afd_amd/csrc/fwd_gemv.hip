// BF16 weight GEMV for 1 to 8 rows (gfx950): HBM-bound, every weight byte streamed once with 128-bit nontemporal
// loads. Numerical contract: the reference's host model, crates/glm53f-forward/src/reference.rs:27-71 (kernel
// counterpart kernels/gemv_bf16.cu:29-106 with 32-lane warps): 32 partial sums per output and K split, each an
// fma chain over k = lo + 8 l + 256 i + j; an xor butterfly over 16, 8, 4, 2, 1; splits added in order.
//
// Here half a wave (32 lanes) plays the model's 32 partials of OUTS outputs at once (1 or 2: more outputs share
// the activations a lane reads, fewer give more workgroups for a small n). The activations of the workgroup's K
// range sit in LDS as f32 (widened once when they are staged), so a lane reads them as 128-bit pieces next to the
// weight pieces it streams; a workgroup of 8 half-waves owns 8 OUTS outputs.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "glm53f_fwd_gemv.h"

namespace fwd_gemv {
namespace {

constexpr int kInvalid = 1;                       // hipErrorInvalidValue
constexpr int THREADS = 256;
constexpr int STEP = 256;                         // values of K per step of a half-wave: 32 lanes x 8
constexpr int LDS_BYTES = 64 * 1024;              // staged activations: rows x range piece x 4 bytes at most

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 hwbf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float lo16(uint32_t v) { return __uint_as_float(v << 16); }
__device__ __forceinline__ float hi16(uint32_t v) { return __uint_as_float(v & 0xffff0000u); }
__device__ __forceinline__ uint16_t f2bf(float x) { return __builtin_bit_cast(uint16_t, (__bf16)x); }

// x[lane ^ M] inside a row of 16 lanes by DPP (quad permutes, a rotation by 8, two masked shifts by 4).
template <int M>
__device__ __forceinline__ float lane_xor16(float x) {
    const int xi = __float_as_int(x);
    if constexpr (M == 1) return __int_as_float(__builtin_amdgcn_update_dpp(0, xi, 0xB1, 0xf, 0xf, true));
    if constexpr (M == 2) return __int_as_float(__builtin_amdgcn_update_dpp(0, xi, 0x4E, 0xf, 0xf, true));
    if constexpr (M == 8) return __int_as_float(__builtin_amdgcn_update_dpp(0, xi, 0x128, 0xf, 0xf, true));
    if constexpr (M == 4) {
        const int lo = __builtin_amdgcn_update_dpp(0, xi, 0x104, 0xf, 0x5, false);
        return __int_as_float(__builtin_amdgcn_update_dpp(lo, xi, 0x114, 0xf, 0xa, false));
    }
    return x;
}

// The model's warp_sum over the 32 lanes of a half-wave (crates/glm53f-layers/src/math.rs:76-88): every lane ends
// with the same bits.
__device__ __forceinline__ float half_wave_sum(float v) {
    v = v + __shfl_xor(v, 16, 64);
    v = v + lane_xor16<8>(v);
    v = v + lane_xor16<4>(v);
    v = v + lane_xor16<2>(v);
    v = v + lane_xor16<1>(v);
    return v;
}

template <bool F32>
__device__ __forceinline__ void store_out(void* out, long long idx, float v) {
    if constexpr (F32) static_cast<float*>(out)[idx] = v;
    else static_cast<uint16_t*>(out)[idx] = f2bf(v);
}

// grid (ceil(n / (8 OUTS)), ksplit, groups). kp: the piece of a split's K range staged at a time (a multiple of
// 256, rows * kp * 4 bytes of LDS). UNROLL: steps whose weight pieces are requested together.
// inside > 1 (then gridDim.y is 1): the workgroup walks all `inside` splits of its outputs itself, one after the
// other, and adds their sums in split order as the model does - no partial sums in memory, no counter, no fence.
// The split exists to give a small n workgroups enough; with few splits the walk is shorter than the hand-over
// through memory (4096 -> 256 with four splits: 13 us as four workgroups per block of outputs, 2 MB of weights).
template <int M, int OUTS, bool F32>
__global__ void __launch_bounds__(THREADS) gemv_kernel(const uint16_t* __restrict__ x, long long ldx, long long x_gs,
                                                       const uint16_t* __restrict__ w, long long ldw, long long w_gs,
                                                       int n, int kc, int kp, int inside, float* __restrict__ partials,
                                                       unsigned* __restrict__ sync, void* __restrict__ out,
                                                       long long ldo, long long o_gs) {
    constexpr int BLOCK_OUTS = (THREADS / 32) * OUTS;
    constexpr int UNROLL = OUTS == 1 ? 8 : 4;
    extern __shared__ __align__(16) unsigned char smem[];
    float* xs = reinterpret_cast<float*>(smem);                       // [M][kp]
    const int t = threadIdx.x, hw = t >> 5, l = t & 31;
    const int g = blockIdx.z, nsplit = gridDim.y;
    const int o0 = blockIdx.x * BLOCK_OUTS + hw * OUTS;               // n % 8 == 0: o0 < n means o0 + OUTS <= n
    const bool live = o0 < n;
    void* og = F32 ? static_cast<void*>(static_cast<float*>(out) + g * o_gs)
                   : static_cast<void*>(static_cast<uint16_t*>(out) + g * o_gs);

    float total[OUTS][M];                         // inside > 1: the splits' sums so far
    for (int walk = 0; walk < inside; ++walk) {
    const int split = inside > 1 ? walk : (int)blockIdx.y;
    const int lo = split * kc;
    const uint16_t* xg = x + g * x_gs + lo;
    const uint16_t* w0 = w + g * w_gs + (long long)(live ? o0 : 0) * ldw + lo;

    float acc[OUTS][M];
#pragma unroll
    for (int r = 0; r < OUTS; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = 0.0f;

    for (int p0 = 0; p0 < kc; p0 += kp) {
        const int pw = min(kp, kc - p0);                              // this piece's width, a multiple of 8
        // lane l takes k = p0 + 8 l + 256 i of the piece while that is inside it. The weight pieces of UNROLL steps
        // are requested together, the next set before the current one is worked on, the first before the
        // activations are staged.
        auto request = [&](u32x4 (&wv)[UNROLL][OUTS], int k0) {
#pragma unroll
            for (int u = 0; u < UNROLL; ++u)
#pragma unroll
                for (int r = 0; r < OUTS; ++r)   // unconditional (a step past the piece re-reads its last one)
                    wv[u][r] = __builtin_nontemporal_load(
                        reinterpret_cast<const u32x4*>(w0 + r * ldw + p0 + min(k0 + STEP * u, pw - 8)));
        };
        auto work = [&](const u32x4 (&wv)[UNROLL][OUTS], int k0) {
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                if (k0 + STEP * u >= pw) break;
                float wf[OUTS][8];
#pragma unroll
                for (int r = 0; r < OUTS; ++r)
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        wf[r][2 * d] = lo16(wv[u][r][d]);
                        wf[r][2 * d + 1] = hi16(wv[u][r][d]);
                    }
#pragma unroll
                for (int m = 0; m < M; ++m) {
                    const f32x4* xp = reinterpret_cast<const f32x4*>(xs + m * kp + k0 + STEP * u);
                    const f32x4 xa = xp[0], xb = xp[1];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float xv = j < 4 ? xa[j] : xb[j - 4];
#pragma unroll
                        for (int r = 0; r < OUTS; ++r) acc[r][m] = __builtin_fmaf(xv, wf[r][j], acc[r][m]);
                    }
                }
            }
        };
        u32x4 wa[UNROLL][OUTS], wb[UNROLL][OUTS];
        int k0 = 8 * l;
        request(wa, k0);
        if (p0 > 0 || walk > 0) __syncthreads();
        for (int e = t; e < M * (pw / 8); e += THREADS) {
            const int m = e / (pw / 8), c = e - m * (pw / 8);
            const u32x4 v = *reinterpret_cast<const u32x4*>(xg + m * ldx + p0 + 8 * c);
            f32x4* dst = reinterpret_cast<f32x4*>(xs + m * kp + 8 * c);
            dst[0] = f32x4{lo16(v[0]), hi16(v[0]), lo16(v[1]), hi16(v[1])};
            dst[1] = f32x4{lo16(v[2]), hi16(v[2]), lo16(v[3]), hi16(v[3])};
        }
        __syncthreads();
        if (!live) continue;
        while (k0 < pw) {                         // in pairs, so that the two register sets are compile-time choices
            request(wb, k0 + STEP * UNROLL);        // (unconditional: past the piece's end a request repeats its last step)
            work(wa, k0);
            k0 += STEP * UNROLL;
            if (k0 >= pw) break;
            request(wa, k0 + STEP * UNROLL);
            work(wb, k0);
            k0 += STEP * UNROLL;
        }
    }

    if (live) {
#pragma unroll
        for (int r = 0; r < OUTS; ++r)
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const float v = half_wave_sum(acc[r][m]);
                if (inside > 1) {                 // (every lane of the half-wave holds the same bits)
                    total[r][m] = walk == 0 ? v : total[r][m] + v;
                    if (walk == inside - 1 && l == ((r * M + m) & 31)) store_out<F32>(og, (long long)m * ldo + o0 + r, total[r][m]);
                } else if (l == ((r * M + m) & 31)) {
                    if (nsplit > 1) partials[(((long long)g * nsplit + split) * M + m) * n + o0 + r] = v;
                    else store_out<F32>(og, (long long)m * ldo + o0 + r, v);
                }
            }
    }
    }
    if (nsplit == 1) return;

    // The last workgroup of this block of outputs to finish adds the splits in split order. Counters: one per 8
    // outputs as the caller sized them; this workgroup uses the one of its first 8.
    // (the flag lives where the activations were staged: every lane is past its last read of them at the barrier
    // below, and the staging may fill all the LDS a launch can ask for without an attribute)
    int& last = *reinterpret_cast<int*>(smem);
    __threadfence();
    __syncthreads();
    unsigned* counter = sync + (long long)g * (n / 8) + OUTS * blockIdx.x;
    if (t == 0) last = atomicAdd(counter, 1u) == (unsigned)(nsplit - 1);
    __syncthreads();
    if (!last) return;
    __threadfence();
    if (t == 0) *counter = 0;                     // every split of this block has signalled
    const long long split_stride = (long long)M * n;
    for (int e = t; e < BLOCK_OUTS * M; e += THREADS) {
        const int m = e / BLOCK_OUTS, o = blockIdx.x * BLOCK_OUTS + e % BLOCK_OUTS;
        if (o >= n) continue;
        const long long base = ((long long)g * nsplit * M + m) * n + o;
        float s = __hip_atomic_load(partials + base, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int kk = 1; kk < nsplit; ++kk)
            s = s + __hip_atomic_load(partials + base + kk * split_stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        store_out<F32>(og, (long long)m * ldo + o, s);
    }
}

// The same contract for five to eight rows when the wide kernel below would leave CUs without a workgroup (the output
// projection: n = 4096). The two halves of a wave take the same two outputs and split the rows between them (their
// loads of a weight piece name the same address: one fetch), so a lane carries a quarter of the accumulators of two
// outputs x eight rows, the rows' activations are read from LDS once for two outputs, and there are waves enough to
// keep two workgroups on every CU. The weight stream does not stop at the pieces of the K range: a group of four
// steps is always in flight while the other is worked on, and the next piece's activations are requested before
// the current piece is worked on. Each accumulator still sees its products in the model's order.
constexpr int SPLIT_OUTS = 2, SPLIT_UNROLL = 4;
constexpr int SPLIT_BLOCK_OUTS = (THREADS / 64) * SPLIT_OUTS;        // 8: one counter per workgroup
constexpr int SPLIT_KP = 2 * STEP * SPLIT_UNROLL;                    // 2048: a piece is two groups of steps

template <int M, bool F32>
__global__ void __launch_bounds__(THREADS) gemv_split_rows_kernel(const uint16_t* __restrict__ x, long long ldx,
                                                                  long long x_gs, const uint16_t* __restrict__ w,
                                                                  long long ldw, long long w_gs, int n, int kc,
                                                                  int inside, float* __restrict__ partials,
                                                                  unsigned* __restrict__ sync, void* __restrict__ out,
                                                                  long long ldo, long long o_gs) {
    constexpr int MR = (M + 1) / 2;                                   // rows of a lane: row0 .. row0 + MR - 1, below M
    constexpr int kp = SPLIT_KP, GROUP = STEP * SPLIT_UNROLL;
    static_assert(M * kp * 4 <= LDS_BYTES, "a piece's activations fit the LDS of a launch without an attribute");
    __shared__ __align__(16) float xs[M * kp];
    const int t = threadIdx.x, l = t & 31;
    const int row0 = ((t >> 5) & 1) * MR;
    const int g = blockIdx.z, nsplit = gridDim.y;
    const int o0 = blockIdx.x * SPLIT_BLOCK_OUTS + (t >> 6) * SPLIT_OUTS;   // n % 8 == 0: all eight exist
    void* og = F32 ? static_cast<void*>(static_cast<float*>(out) + g * o_gs)
                   : static_cast<void*>(static_cast<uint16_t*>(out) + g * o_gs);

    float total[SPLIT_OUTS][MR];                  // inside > 1 (as in gemv_kernel): the splits' sums so far
    for (int walk = 0; walk < inside; ++walk) {
    const int split = inside > 1 ? walk : (int)blockIdx.y;
    const int lo = split * kc;
    const uint16_t* xg = x + g * x_gs + lo;
    const uint16_t* w0 = w + g * w_gs + (long long)o0 * ldw + lo;

    float acc[SPLIT_OUTS][MR];
#pragma unroll
    for (int r = 0; r < SPLIT_OUTS; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[r][m] = 0.0f;

    // lane l takes k = 8 l + 256 i while that is below kc; kq: the first k of a group of steps
    auto request = [&](u32x4 (&wv)[SPLIT_UNROLL][SPLIT_OUTS], int kq) {
#pragma unroll
        for (int u = 0; u < SPLIT_UNROLL; ++u)
#pragma unroll
            for (int r = 0; r < SPLIT_OUTS; ++r)   // unconditional (a step past the range re-reads its last piece)
                wv[u][r] = __builtin_nontemporal_load(
                    reinterpret_cast<const u32x4*>(w0 + r * ldw + min(kq + 8 * l + STEP * u, kc - 8)));
    };
    // p0: the first k of the staged piece
    auto work = [&](const u32x4 (&wv)[SPLIT_UNROLL][SPLIT_OUTS], int kq, int p0) {
#pragma unroll
        for (int u = 0; u < SPLIT_UNROLL; ++u) {
            const int k = kq + 8 * l + STEP * u;
            if (k >= kc) break;
            float wf[SPLIT_OUTS][8];
#pragma unroll
            for (int r = 0; r < SPLIT_OUTS; ++r)
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    wf[r][2 * d] = lo16(wv[u][r][d]);
                    wf[r][2 * d + 1] = hi16(wv[u][r][d]);
                }
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                if (2 * MR != M && m == MR - 1 && row0 != 0) break;   // an odd M: the second half is one row short
                // a step's 256 values sit as the 32 lanes' first four, then their second four: the lanes of a half
                // read consecutive 16-byte pieces (lane-major, 32 bytes apart, they would meet in the banks)
                const f32x4* xp = reinterpret_cast<const f32x4*>(xs + (row0 + m) * kp + (k - p0) - 4 * l);
                const f32x4 xa = xp[0], xb = xp[32];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float xv = j < 4 ? xa[j] : xb[j - 4];
#pragma unroll
                    for (int r = 0; r < SPLIT_OUTS; ++r) acc[r][m] = __builtin_fmaf(xv, wf[r][j], acc[r][m]);
                }
            }
        }
    };
    // A piece's activations: lane t takes the eight values at k = p0 + 8 t of every row (kp = 8 x 256 lanes).
    u32x4 xq[M];
    auto request_x = [&](int p0) {
        const int k = min(p0 + 8 * t, kc - 8);
#pragma unroll
        for (int m = 0; m < M; ++m) xq[m] = *reinterpret_cast<const u32x4*>(xg + m * ldx + k);
    };
    auto stage_x = [&]() {
#pragma unroll
        for (int m = 0; m < M; ++m) {
            f32x4* dst = reinterpret_cast<f32x4*>(xs + m * kp + 8 * t - 4 * (t & 31));
            dst[0] = f32x4{lo16(xq[m][0]), hi16(xq[m][0]), lo16(xq[m][1]), hi16(xq[m][1])};
            dst[32] = f32x4{lo16(xq[m][2]), hi16(xq[m][2]), lo16(xq[m][3]), hi16(xq[m][3])};
        }
    };

    u32x4 wa[SPLIT_UNROLL][SPLIT_OUTS], wb[SPLIT_UNROLL][SPLIT_OUTS];
    request(wa, 0);
    request_x(0);
    for (int p0 = 0; p0 < kc; p0 += kp) {
        if (p0 > 0 || walk > 0) __syncthreads();  // every lane is past its reads of the piece before
        stage_x();
        __syncthreads();
        request(wb, p0 + GROUP);
        if (p0 + kp < kc) request_x(p0 + kp);
        work(wa, p0, p0);
        request(wa, p0 + kp);
        if (p0 + GROUP < kc) work(wb, p0 + GROUP, p0);
    }

#pragma unroll
    for (int r = 0; r < SPLIT_OUTS; ++r)
#pragma unroll
        for (int mi = 0; mi < MR; ++mi) {
            const float v = half_wave_sum(acc[r][mi]);
            const int m = row0 + mi;
            if (inside > 1) {
                total[r][mi] = walk == 0 ? v : total[r][mi] + v;
                if (walk == inside - 1 && m < M && l == ((r * MR + mi) & 31)) store_out<F32>(og, (long long)m * ldo + o0 + r, total[r][mi]);
            } else if (m < M && l == ((r * MR + mi) & 31)) {
                if (nsplit > 1) partials[(((long long)g * nsplit + split) * M + m) * n + o0 + r] = v;
                else store_out<F32>(og, (long long)m * ldo + o0 + r, v);
            }
        }
    }
    if (nsplit == 1) return;

    int& last = *reinterpret_cast<int*>(xs);      // as above: the last workgroup of these eight outputs adds the splits
    __threadfence();
    __syncthreads();
    unsigned* counter = sync + (long long)g * (n / 8) + blockIdx.x;
    if (t == 0) last = atomicAdd(counter, 1u) == (unsigned)(nsplit - 1);
    __syncthreads();
    if (!last) return;
    __threadfence();
    if (t == 0) *counter = 0;
    const long long split_stride = (long long)M * n;
    for (int e = t; e < SPLIT_BLOCK_OUTS * M; e += THREADS) {
        const int m = e / SPLIT_BLOCK_OUTS, o = blockIdx.x * SPLIT_BLOCK_OUTS + e % SPLIT_BLOCK_OUTS;
        const long long base = ((long long)g * nsplit * M + m) * n + o;
        float s = __hip_atomic_load(partials + base, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int kk = 1; kk < nsplit; ++kk)
            s = s + __hip_atomic_load(partials + base + kk * split_stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        store_out<F32>(og, (long long)m * ldo + o, s);
    }
}

// The same contract for three rows and more, where a lane's arithmetic (rows x 8 fused multiply-adds per weight
// word pair) and its reads of the activations weigh as much as the weight stream: half a wave owns eight outputs
// and walks the K steps in the outer loop, so that the rows' activations of a step are read from LDS once for all
// eight (each accumulator still sees its products in the order of the model). 256 lanes per workgroup, 64 outputs:
// every workgroup widens the rows' activations into its own LDS, and with 32 outputs per workgroup that staging
// cost 5 to 10 % of the launch. Taken when that still gives every CU a workgroup (64-lane workgroups for a smaller
// n measured slower than the kernel above).
constexpr int WIDE_THREADS = 256, WIDE_OUTS = 8;
constexpr int WIDE_BLOCK_OUTS = (WIDE_THREADS / 32) * WIDE_OUTS;   // 64 outputs share one staging of the activations

template <int M, bool F32>
__global__ void __launch_bounds__(WIDE_THREADS) gemv_wide_kernel(const uint16_t* __restrict__ x, long long ldx,
                                                                 long long x_gs, const uint16_t* __restrict__ w,
                                                                 long long ldw, long long w_gs, int n, int kc, int kp,
                                                                 float* __restrict__ partials,
                                                                 unsigned* __restrict__ sync, void* __restrict__ out,
                                                                 long long ldo, long long o_gs) {
    constexpr int BLOCK_OUTS = WIDE_BLOCK_OUTS;
    extern __shared__ __align__(16) unsigned char smem[];
    float* xs = reinterpret_cast<float*>(smem);                       // [M][kp]
    const int t = threadIdx.x, hw = t >> 5, l = t & 31;
    const int g = blockIdx.z, split = blockIdx.y, nsplit = gridDim.y;
    const int o0 = blockIdx.x * BLOCK_OUTS + hw * WIDE_OUTS;
    const bool live = o0 < n;
    const int lo = split * kc;
    const uint16_t* xg = x + g * x_gs + lo;
    const uint16_t* w0 = w + g * w_gs + (long long)(live ? o0 : 0) * ldw + lo;

    float acc[WIDE_OUTS][M];
#pragma unroll
    for (int r = 0; r < WIDE_OUTS; ++r)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[r][m] = 0.0f;

    for (int p0 = 0; p0 < kc; p0 += kp) {
        const int pw = min(kp, kc - p0);
        auto request = [&](u32x4 (&wv)[WIDE_OUTS], int k0) {         // unconditional, as above
#pragma unroll
            for (int r = 0; r < WIDE_OUTS; ++r)
                wv[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(w0 + r * ldw + p0 + min(k0, pw - 8)));
        };
        auto work = [&](const u32x4 (&wv)[WIDE_OUTS], int k0) {
            float xr[M][8];
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const f32x4* xp = reinterpret_cast<const f32x4*>(xs + m * kp + k0);
                const f32x4 xa = xp[0], xb = xp[1];
#pragma unroll
                for (int j = 0; j < 4; ++j) { xr[m][j] = xa[j]; xr[m][4 + j] = xb[j]; }
            }
#pragma unroll
            for (int r = 0; r < WIDE_OUTS; ++r) {
                float wf[8];
#pragma unroll
                for (int d = 0; d < 4; ++d) { wf[2 * d] = lo16(wv[r][d]); wf[2 * d + 1] = hi16(wv[r][d]); }
#pragma unroll
                for (int m = 0; m < M; ++m)
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[r][m] = __builtin_fmaf(xr[m][j], wf[j], acc[r][m]);
            }
        };
        u32x4 wa[WIDE_OUTS], wb[WIDE_OUTS];
        int k0 = 8 * l;
        request(wa, k0);
        if (p0 > 0) __syncthreads();
        for (int e = t; e < M * (pw / 8); e += WIDE_THREADS) {
            const int m = e / (pw / 8), c = e - m * (pw / 8);
            const u32x4 v = *reinterpret_cast<const u32x4*>(xg + m * ldx + p0 + 8 * c);
            f32x4* dst = reinterpret_cast<f32x4*>(xs + m * kp + 8 * c);
            dst[0] = f32x4{lo16(v[0]), hi16(v[0]), lo16(v[1]), hi16(v[1])};
            dst[1] = f32x4{lo16(v[2]), hi16(v[2]), lo16(v[3]), hi16(v[3])};
        }
        __syncthreads();
        if (!live) continue;
        while (k0 < pw) {
            request(wb, k0 + STEP);
            work(wa, k0);
            k0 += STEP;
            if (k0 >= pw) break;
            request(wa, k0 + STEP);
            work(wb, k0);
            k0 += STEP;
        }
    }

    void* og = F32 ? static_cast<void*>(static_cast<float*>(out) + g * o_gs)
                   : static_cast<void*>(static_cast<uint16_t*>(out) + g * o_gs);
    if (live) {
#pragma unroll
        for (int r = 0; r < WIDE_OUTS; ++r)
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const float v = half_wave_sum(acc[r][m]);
                if (l == ((r * M + m) & 31)) {
                    if (nsplit > 1) partials[(((long long)g * nsplit + split) * M + m) * n + o0 + r] = v;
                    else store_out<F32>(og, (long long)m * ldo + o0 + r, v);
                }
            }
    }
    if (nsplit == 1) return;

    int& last = *reinterpret_cast<int*>(smem);    // as above: the last workgroup of these outputs adds the splits
    __threadfence();
    __syncthreads();
    unsigned* counter = sync + (long long)g * (n / 8) + (BLOCK_OUTS / 8) * blockIdx.x;
    if (t == 0) last = atomicAdd(counter, 1u) == (unsigned)(nsplit - 1);
    __syncthreads();
    if (!last) return;
    __threadfence();
    if (t == 0) *counter = 0;
    const long long split_stride = (long long)M * n;
    for (int e = t; e < BLOCK_OUTS * M; e += WIDE_THREADS) {
        const int m = e / BLOCK_OUTS, o = blockIdx.x * BLOCK_OUTS + e % BLOCK_OUTS;
        if (o >= n) continue;
        const long long base = ((long long)g * nsplit * M + m) * n + o;
        float s = __hip_atomic_load(partials + base, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int kk = 1; kk < nsplit; ++kk)
            s = s + __hip_atomic_load(partials + base + kk * split_stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        store_out<F32>(og, (long long)m * ldo + o, s);
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Whether a launch with `ksplit` splits and these shapes walks the splits inside its workgroups (gemv_kernel): up to
// four splits, in the kernels that serve a small n. Such a launch touches neither the partial sums nor the counters.
constexpr int kMaxSplitsInside = 4;
#ifndef KDA_SPLIT_ROWS_FROM
#define KDA_SPLIT_ROWS_FROM 3
#endif
inline bool splits_inside(int rows, int groups, int n, int ksplit) {
    if (ksplit < 2 || ksplit > kMaxSplitsInside) return false;
    const long long blocks8 = (long long)(n / 8) * ksplit * groups;
    return !(rows >= 3 && blocks8 >= 4 * 512);    // (the wide kernel keeps its splits in the grid)
}

template <int M, int OUTS, bool F32>
int32_t launch_mo(const uint16_t* x, long long ldx, long long x_gs, const uint16_t* w, long long ldw, long long w_gs,
                  int groups, int n, int k, int ksplit, float* partials, unsigned* sync, void* out, long long ldo,
                  long long o_gs, hipStream_t stream) {
    const int kc = k / ksplit;
    // the widest piece of the K range whose activations fit 32 KiB (64 KiB for one row: no second piece up to
    // k = 16,384), a multiple of 256. (This kernel serves one to four rows: launch_m.)
    static_assert(M <= 4, "five rows and more take gemv_wide_kernel or gemv_split_rows_kernel");
    int kp = (M == 1 ? LDS_BYTES : LDS_BYTES / 2) / (4 * M) / STEP * STEP;
    if (kp > kc) kp = kc;
    const size_t lds = (size_t)M * kp * 4;
    const int block_outs = (THREADS / 32) * OUTS;
    const int inside = splits_inside(M, groups, n, ksplit) ? ksplit : 1;
    const dim3 grid((unsigned)((n + block_outs - 1) / block_outs), (unsigned)(inside > 1 ? 1 : ksplit), (unsigned)groups);
    gemv_kernel<M, OUTS, F32><<<grid, THREADS, lds, stream>>>(x, ldx, x_gs, w, ldw, w_gs, n, kc, kp, inside, partials,
                                                              sync, out, ldo, o_gs);
    return (int32_t)hipGetLastError();
}

// Outputs per half-wave: two when that still leaves the chip four workgroups per CU (they share the activations a
// lane reads), else one. (Four measured slower: 250 registers, two waves per SIMD.)
template <int M, bool F32>
int32_t launch_m(const uint16_t* x, long long ldx, long long x_gs, const uint16_t* w, long long ldw, long long w_gs,
                 int groups, int n, int k, int ksplit, float* partials, unsigned* sync, void* out, long long ldo,
                 long long o_gs, hipStream_t stream) {
    const long long blocks8 = (long long)(n / 8) * ksplit * groups;   // workgroups with one output per half-wave
    if (M >= 3 && blocks8 >= 4 * 512) {                                // 64 outputs per workgroup: one per CU and more
        const int kc = k / ksplit;
        // pieces of the K range whose activations fit 32 KiB; from five rows up 64 KiB, which halves the number of
        // pieces and with them the waits for a piece's staging (two workgroups still fit a CU's LDS)
        int kp = (M > 4 ? LDS_BYTES : LDS_BYTES / 2) / (4 * M) / STEP * STEP;
        if (kp > kc) kp = kc;
        const dim3 grid((unsigned)((n + WIDE_BLOCK_OUTS - 1) / WIDE_BLOCK_OUTS), (unsigned)ksplit, (unsigned)groups);
        gemv_wide_kernel<M, F32><<<grid, WIDE_THREADS, (size_t)M * kp * 4, stream>>>(x, ldx, x_gs, w, ldw, w_gs, n, kc, kp,
                                                                                     partials, sync, out, ldo, o_gs);
        return (int32_t)hipGetLastError();
    }
    if constexpr (M >= KDA_SPLIT_ROWS_FROM) {
        const int inside = splits_inside(M, groups, n, ksplit) ? ksplit : 1;
        const dim3 grid((unsigned)(n / SPLIT_BLOCK_OUTS), (unsigned)(inside > 1 ? 1 : ksplit), (unsigned)groups);
        gemv_split_rows_kernel<M, F32><<<grid, THREADS, 0, stream>>>(x, ldx, x_gs, w, ldw, w_gs, n, k / ksplit, inside,
                                                                     partials, sync, out, ldo, o_gs);
        return (int32_t)hipGetLastError();
    } else {
        if (n % 16 == 0 && blocks8 >= 2 * 1024)
            return launch_mo<M, 2, F32>(x, ldx, x_gs, w, ldw, w_gs, groups, n, k, ksplit, partials, sync, out, ldo, o_gs, stream);
        return launch_mo<M, 1, F32>(x, ldx, x_gs, w, ldw, w_gs, groups, n, k, ksplit, partials, sync, out, ldo, o_gs, stream);
    }
}

template <bool F32>
int32_t launch(const uint16_t* x, long long ldx, long long x_gs, const uint16_t* w, long long ldw, long long w_gs,
               int groups, int rows, int n, int k, int ksplit, float* partials, unsigned* sync, void* out, long long ldo,
               long long o_gs, hipStream_t stream) {
    switch (rows) {
        case 1: return launch_m<1, F32>(x, ldx, x_gs, w, ldw, w_gs, groups, n, k, ksplit, partials, sync, out, ldo, o_gs, stream);
        case 2: return launch_m<2, F32>(x, ldx, x_gs, w, ldw, w_gs, groups, n, k, ksplit, partials, sync, out, ldo, o_gs, stream);
        case 3: return launch_m<3, F32>(x, ldx, x_gs, w, ldw, w_gs, groups, n, k, ksplit, partials, sync, out, ldo, o_gs, stream);
        case 4: return launch_m<4, F32>(x, ldx, x_gs, w, ldw, w_gs, groups, n, k, ksplit, partials, sync, out, ldo, o_gs, stream);
        case 5: return launch_m<5, F32>(x, ldx, x_gs, w, ldw, w_gs, groups, n, k, ksplit, partials, sync, out, ldo, o_gs, stream);
        case 6: return launch_m<6, F32>(x, ldx, x_gs, w, ldw, w_gs, groups, n, k, ksplit, partials, sync, out, ldo, o_gs, stream);
        case 7: return launch_m<7, F32>(x, ldx, x_gs, w, ldw, w_gs, groups, n, k, ksplit, partials, sync, out, ldo, o_gs, stream);
        case 8: return launch_m<8, F32>(x, ldx, x_gs, w, ldw, w_gs, groups, n, k, ksplit, partials, sync, out, ldo, o_gs, stream);
        default: return kInvalid;
    }
}

// ---- the split-K scratch of glm53f_fwd_gemv_bf16_static: the partial sums of the splits, then the counters.
// One copy per GPU, held until the process ends; every call on a GPU shares it.
constexpr size_t kStaticPartialFloats = 262144;   // 1 MiB of f32 partial sums
constexpr size_t kStaticCounters = 4096;          // 16 KiB of counters
static __device__ __align__(256) unsigned char scratch[kStaticPartialFloats * 4 + kStaticCounters * 4];

// The array's name is a host-side stand-in, not a device address: each GPU holds its own copy at its own address,
// looked up once per device (with that device current) and kept.
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
unsigned char* scratch_on[kMaxDevices] = {};

int scratch_of_current_device(unsigned char** ptr) {
    int dev = -1;
    const hipError_t rc = hipGetDevice(&dev);
    if (rc != hipSuccess) return (int)rc;
    if (dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_on[dev] == nullptr) {
        void* p = nullptr;
        const hipError_t sym = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (sym != hipSuccess) return (int)sym;
        if (p == nullptr) return (int)hipErrorInvalidSymbol;
        scratch_on[dev] = static_cast<unsigned char*>(p);
    }
    *ptr = scratch_on[dev];
    return 0;
}

// The counters a launch is about to use start at zero whatever an earlier call left behind (a fill kernel, not a
// memset: a caller may be recording the stream into a graph).
__global__ void __launch_bounds__(THREADS) clear_counters_kernel(unsigned* counters, int count) {
    const int i = blockIdx.x * THREADS + threadIdx.x;
    if (i < count) counters[i] = 0u;
}

}  // namespace
}  // namespace fwd_gemv

extern "C" int32_t glm53f_fwd_gemv_ksplit(int32_t groups, int32_t n, int32_t k) {
    if (groups < 1 || n < 8 || k < 8) return 1;
    const long long blocks = (long long)(n / 8) * groups;
    if (blocks >= 512) return 1;
    int best = 1;
    for (int d = 2; k / d >= 1024; ++d) {
        if (k % (256 * d) != 0) continue;
        best = d;
        if (blocks * d >= 512) break;
    }
    return best;
}

namespace fwd_gemv {
namespace {
// The reference's checks in the reference's order (gemv_bf16.cu:158-164); `scratch_given` stands for the two
// scratch pointers of a split call.
bool arguments_ok(const uint16_t* x, int64_t ldx, int64_t x_gstride, const uint16_t* w, int64_t ldw, int64_t w_gstride,
                  int32_t groups, int32_t rows, int32_t n, int32_t k, int32_t ksplit, bool scratch_given, const void* out,
                  int64_t ldo) {
    if (groups < 1 || groups > 65535 || rows < 1 || rows > 8 || n < 8 || n % 8 || k < 8 || k % 8 || ksplit < 1 ||
        ksplit > 65535 || k % ksplit || (k / ksplit) % 8)
        return false;
    if (!x || !w || !aligned16(x) || !aligned16(w) || !out || ldx % 8 || ldw % 8 || x_gstride % 8 || w_gstride % 8 ||
        ldx < k || ldw < k || ldo < n)
        return false;
    return ksplit == 1 || scratch_given;
}
}  // namespace
}  // namespace fwd_gemv

extern "C" int32_t glm53f_fwd_gemv_bf16(const uint16_t* x, int64_t ldx, int64_t x_gstride, const uint16_t* w,
                                        int64_t ldw, int64_t w_gstride, int32_t groups, int32_t rows, int32_t n,
                                        int32_t k, int32_t ksplit, float* partials, uint32_t* sync, void* out,
                                        int32_t out_f32, int64_t ldo, int64_t o_gstride, ihipStream_t* stream) {
    using namespace fwd_gemv;
    if (!arguments_ok(x, ldx, x_gstride, w, ldw, w_gstride, groups, rows, n, k, ksplit, partials && sync, out, ldo))
        return kInvalid;
    return out_f32 ? launch<true>(x, ldx, x_gstride, w, ldw, w_gstride, groups, rows, n, k, ksplit, partials, sync, out,
                                  ldo, o_gstride, stream)
                   : launch<false>(x, ldx, x_gstride, w, ldw, w_gstride, groups, rows, n, k, ksplit, partials, sync,
                                   out, ldo, o_gstride, stream);
}

// The same GEMV with the split-K scratch in the library's own per-GPU array: no allocation anywhere on the path.
// Every argument is checked before anything is enqueued: a rejected call leaves the stream (and a graph under
// capture) and the shared array untouched.
extern "C" int32_t glm53f_fwd_gemv_bf16_static(const uint16_t* x, int64_t ldx, int64_t x_gstride, const uint16_t* w,
                                               int64_t ldw, int64_t w_gstride, int32_t groups, int32_t rows, int32_t n,
                                               int32_t k, int32_t ksplit, void* out, int32_t out_f32, int64_t ldo,
                                               int64_t o_gstride, ihipStream_t* stream) {
    using namespace fwd_gemv;
    if (!arguments_ok(x, ldx, x_gstride, w, ldw, w_gstride, groups, rows, n, k, ksplit, true, out, ldo)) return kInvalid;
    float* partials = nullptr;
    unsigned* counters = nullptr;
    if (ksplit > 1) {
        // beyond the array: rejected, never truncated (whether or not this shape's kernel goes through the array:
        // the limit is the entry point's, not a kernel's)
        const unsigned long long floats = (unsigned long long)groups * (unsigned long long)ksplit * rows * n;
        const unsigned long long count = (unsigned long long)groups * (unsigned long long)(n / 8);
        if (floats > kStaticPartialFloats || count > kStaticCounters) return kInvalid;
    }
    if (ksplit > 1 && !splits_inside(rows, groups, n, ksplit)) {
        const unsigned long long count = (unsigned long long)groups * (unsigned long long)(n / 8);
        unsigned char* base = nullptr;
        const int rc = scratch_of_current_device(&base);
        if (rc != 0) return rc;
        partials = reinterpret_cast<float*>(base);
        counters = reinterpret_cast<unsigned*>(base + kStaticPartialFloats * 4);
        // The counters start at zero whatever an earlier call left behind (a kernel's last workgroup resets its
        // counter, so this only matters after a call that did not run to its end).
        clear_counters_kernel<<<(unsigned)((count + THREADS - 1) / THREADS), THREADS, 0, stream>>>(counters, (int)count);
        const int32_t lrc = (int32_t)hipGetLastError();
        if (lrc != 0) return lrc;
    }
    return out_f32 ? launch<true>(x, ldx, x_gstride, w, ldw, w_gstride, groups, rows, n, k, ksplit, partials, counters,
                                  out, ldo, o_gstride, stream)
                   : launch<false>(x, ldx, x_gstride, w, ldw, w_gstride, groups, rows, n, k, ksplit, partials, counters,
                                   out, ldo, o_gstride, stream);
}
