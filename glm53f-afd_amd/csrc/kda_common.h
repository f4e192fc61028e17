// Shared device helpers of the KDA kernels (gfx950, wave64).
#ifndef GLM53F_KDA_COMMON_H
#define GLM53F_KDA_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "glm53f_kda.h"

namespace kda {

constexpr int DK = 128, DV = 128, TAPS = 4, WINDOW = 3;
constexpr int kInvalid = 1;  // hipErrorInvalidValue

typedef uint16_t bf16_t;
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));   // a 128-bit piece that stays in registers

__device__ __forceinline__ float bf2f(bf16_t b) { return __uint_as_float((uint32_t)b << 16); }

typedef __bf16 hwbf16x2_t __attribute__((ext_vector_type(2)));
typedef float hwf32x2_t __attribute__((ext_vector_type(2)));

// Round to nearest even with gfx950's v_cvt_pk_bf16_f32: for every finite or infinite input the bits of the
// reference's bf16::from_f32 (src/bf16.rs:6-13); a NaN stays a (quiet) NaN.
__device__ __forceinline__ bf16_t f2bf(float x) { return __builtin_bit_cast(bf16_t, (__bf16)x); }

// Two values in one instruction: lo in bits 0..15, hi in bits 16..31.
__device__ __forceinline__ uint32_t f2bf2(float lo, float hi) {
    const hwf32x2_t f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, hwbf16x2_t));
}

__device__ __forceinline__ float bfround(float x) { return bf2f(f2bf(x)); }

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

// A wave-uniform pointer forced into scalar registers and made opaque to loop strength reduction: addressing
// through it is "scalar base + 32-bit lane offset", and no per-lane 64-bit pointer is carried across a loop.
template <typename T>
__device__ __forceinline__ T* uniform_ptr(T* p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    // Through a global-address-space pointer, so that accesses stay global_* instructions (a pointer made
    // from an integer would otherwise be generic and use flat_* ones, which wait on both memory counters).
    typedef __attribute__((address_space(1))) T* global_ptr_t;
    return (T*)reinterpret_cast<global_ptr_t>(((uint64_t)hi << 32) | lo);
}

// Request b's global rows: [row0, row0 + rows). Without cu_rows: one request of rows1 rows.
struct RowRange {
    long long row0;
    int rows;
};

__device__ __forceinline__ RowRange request_rows(const int32_t* cu_rows, int b, int rows1) {
    if (cu_rows == nullptr) return {0, rows1};
    const int r0 = cu_rows[b];
    return {(long long)r0, cu_rows[b + 1] - r0};
}

// How a state element type maps onto a workgroup of 256 lanes (4 waves). Every lane moves 128 bits per
// access: KPL consecutive keys of one value row. LPR lanes share a value row, a wave covers RPW rows per
// step and the workgroup 4 * RPW; STEPS steps cover the 128 value rows, 64 state values per lane.
template <typename S>
struct StateGeo;
template <>
struct StateGeo<float> {
    static constexpr int KPL = 4;
};
template <>
struct StateGeo<bf16_t> {
    static constexpr int KPL = 8;
};

template <typename S>
struct StateMap {
    static constexpr int KPL = StateGeo<S>::KPL;
    static constexpr int NP = KPL / 4;         // partial sums per lane (groups of 4 consecutive keys)
    static constexpr int LPR = DK / KPL;       // lanes per value row
    static constexpr int RPW = 64 / LPR;       // value rows per wave per step
    static constexpr int RPS = 4 * RPW;        // value rows per workgroup per step
    static constexpr int STEPS = DV / RPS;
    static constexpr bool kRound = sizeof(S) == 2;

    // Value row of step j for this lane, and its first key.
    static __device__ __forceinline__ int row(int j, int wave, int lane) { return j * RPS + wave * RPW + lane / LPR; }
    static __device__ __forceinline__ int key0(int lane) { return (lane % LPR) * KPL; }
};

// 128-bit raw state access.
// The states are streamed: every byte is read once and written once per launch, and a decode sweep's working set
// (gigabytes) is far beyond the caches. Nontemporal accesses keep them from displacing anything and measured a
// quarter faster than plain ones on the decode step (14.6 against 19.0 us for sixteen 2 MiB states).
__device__ __forceinline__ uint4 ld128(const void* p) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void st128(void* p, uint4 v) {
    const u32x4_t x = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(x, reinterpret_cast<u32x4_t*>(p));
}

template <typename S>
__device__ __forceinline__ void unpack(const uint4 raw, float (&s)[StateGeo<S>::KPL]);
template <>
__device__ __forceinline__ void unpack<float>(const uint4 raw, float (&s)[4]) {
    s[0] = __uint_as_float(raw.x);
    s[1] = __uint_as_float(raw.y);
    s[2] = __uint_as_float(raw.z);
    s[3] = __uint_as_float(raw.w);
}
template <>
__device__ __forceinline__ void unpack<bf16_t>(const uint4 raw, float (&s)[8]) {
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        s[2 * i] = __uint_as_float(w[i] << 16);
        s[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}

// Pack for the store. A bf16 state is already bf16-exact here (rounded after every row, or just loaded),
// so the conversion rounds nothing.
template <typename S>
__device__ __forceinline__ uint4 pack(const float (&s)[StateGeo<S>::KPL]);
template <>
__device__ __forceinline__ uint4 pack<float>(const float (&s)[4]) {
    return make_uint4(__float_as_uint(s[0]), __float_as_uint(s[1]), __float_as_uint(s[2]), __float_as_uint(s[3]));
}
template <>
__device__ __forceinline__ uint4 pack<bf16_t>(const float (&s)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = f2bf2(s[2 * i], s[2 * i + 1]);
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// x[lane ^ M] for M = 1, 2, 4, 8 inside a row of 16 lanes, as data-parallel-primitive moves (no LDS):
// quad permutes for 1 and 2, a rotation by 8 for 8, and for 4 a shift left into banks 0 and 2 and a shift
// right into banks 1 and 3 (a bank is 4 lanes).
template <int M>
__device__ __forceinline__ float lane_xor16(float x) {
    const int xi = __float_as_int(x);
    if constexpr (M == 1) return __int_as_float(__builtin_amdgcn_update_dpp(0, xi, 0xB1, 0xf, 0xf, true));
    if constexpr (M == 2) return __int_as_float(__builtin_amdgcn_update_dpp(0, xi, 0x4E, 0xf, 0xf, true));
    if constexpr (M == 8) return __int_as_float(__builtin_amdgcn_update_dpp(0, xi, 0x128, 0xf, 0xf, true));
    if constexpr (M == 4) {
        const int lo = __builtin_amdgcn_update_dpp(0, xi, 0x104, 0xf, 0x5, false);     // row_shl:4 -> banks 0, 2
        return __int_as_float(__builtin_amdgcn_update_dpp(lo, xi, 0x114, 0xf, 0xa, false));  // row_shr:4 -> 1, 3
    }
    return x;
}

// The sum over one value row's 128 keys of per-lane partial sums, in the order of the reference's CPU
// model (cpu.rs:214-239): partial l (l = 0..31) covers keys 4l..4l+3, then an xor butterfly over l with
// offsets 16, 8, 4, 2, 1. With NP partials per lane the low bits of l live inside the lane, so the
// butterfly's first steps cross lanes and its last adds the lane's own partials. Every lane of the row
// ends with the same bits (an addition commutes, so both partners of a step compute the same sum).
template <int NP, int LPR>
__device__ __forceinline__ float row_sum(float (&x)[NP]) {
    if constexpr (LPR == 32) {
#pragma unroll
        for (int p = 0; p < NP; ++p) x[p] = x[p] + __shfl_xor(x[p], 16, 64);
    }
#pragma unroll
    for (int p = 0; p < NP; ++p) x[p] = x[p] + lane_xor16<8>(x[p]);
    // After the step above lanes l and l ^ 8 hold the same bits, so the value of lane l ^ 4 is also what the lane four
    // further round the row holds: one rotation, which folds into the add.
#pragma unroll
    for (int p = 0; p < NP; ++p)
        x[p] = x[p] + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x[p]), 0x124, 0xf, 0xf, true));
#pragma unroll
    for (int p = 0; p < NP; ++p) x[p] = x[p] + lane_xor16<2>(x[p]);
#pragma unroll
    for (int p = 0; p < NP; ++p) x[p] = x[p] + lane_xor16<1>(x[p]);
    if (NP == 2) return x[0] + x[1];
    return x[0];
}

// One delta-rule step on this lane's KPL keys of one value row: the arithmetic, operation for operation,
// of the reference's `update` (cpu.rs:324-344, kda.cu:38-53). No fused multiply-add (the file is compiled
// with contraction off).
template <typename S>
__device__ __forceinline__ void update_row(float (&s)[StateGeo<S>::KPL], const float (&kk)[StateGeo<S>::KPL],
                                           const float (&gg)[StateGeo<S>::KPL], float v, float beta) {
    using M = StateMap<S>;
    float part[M::NP];
#pragma unroll
    for (int p = 0; p < M::NP; ++p) {
        float kv = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = 4 * p + i;
            s[c] = s[c] * gg[c];
            kv = kv + s[c] * kk[c];
        }
        part[p] = kv;
    }
    const float kv = row_sum<M::NP, M::LPR>(part);
    const float delta = (v - kv) * beta;
#pragma unroll
    for (int c = 0; c < M::KPL; ++c) s[c] = s[c] + kk[c] * delta;
}

// The read-out of one value row (cpu.rs:347-353), not rounded.
template <typename S>
__device__ __forceinline__ float read_row(const float (&s)[StateGeo<S>::KPL], const float (&qq)[StateGeo<S>::KPL]) {
    using M = StateMap<S>;
    float part[M::NP];
#pragma unroll
    for (int p = 0; p < M::NP; ++p) {
        float o = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) o = o + s[4 * p + i] * qq[4 * p + i];
        part[p] = o;
    }
    return row_sum<M::NP, M::LPR>(part);
}

// dot128 (cpu.rs:229-239) of an LDS vector with itself, by the 32 lanes of a half wave (lane32 = 0..31).
__device__ __forceinline__ float sumsq128(const float* x, int lane32, float (&v4)[4]) {
    float part[1] = {0.0f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v4[i] = x[lane32 * 4 + i];
        part[0] = part[0] + v4[i] * v4[i];
    }
    return row_sum<1, 32>(part);
}

}  // namespace kda

#endif  // GLM53F_KDA_COMMON_H
