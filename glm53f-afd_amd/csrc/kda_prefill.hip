// KDA chunked prefill on gfx950: the delta rule over a prompt segment in the chunked (WY/UT) form, with every
// GEMM-shaped step on the matrix cores and every operand carried at f32-class precision.
//
// The algebra is the reference's chunk form (crates/glm53f-kda/src/chunked.rs:67-198; kernel counterpart
// kda_prefill.cu:95-538 with 16-row chunks on CUDA cores). Here a chunk is 64 rows in four sub-chunks of 16.
// With G the cumulative log decay inside the chunk, per key channel:
//   L[i][j] = beta_i sum_d k_i k_j e^{G_i - G_j} (j < i),  M[i][j] = sum_d q_i k_j e^{G_i - G_j} (j <= i),
//   T' = (I + L)^-1 diag(beta),  Kd = k e^G,  Qg = q e^G,  Kg = k e^{G_last - G};
//   from the state S entering the chunk: P = V - Kd S,  V' = T' P,  Y = Qg S + M V',  S <- e^{G_last} S + Kg^T V'.
// e^{G_i - G_j} is factored around a reference row so that both factors are GEMM operands: inside a sub-chunk
// around its first row (one factor reaches e^{+87}), between sub-chunks around a row in between (exponents <= 0).
//
// Precision. The tiles of L and M run on the f32 MFMA (v_mfma_f32_16x16x4_f32) with f32 operands. Everything else
// runs on v_mfma_f32_16x16x32_f16 with each operand held as a PAIR of fp16 values, hi = fp16(x s) and
// lo = fp16(x s - hi), s a fixed power of two per operand that puts its values well inside the fp16 range. A
// product is three instructions (hi hi, hi lo, lo hi; lo lo is below f32 rounding), which carries 22 significant
// bits while lo is a normal fp16 number and an absolute 2^-25 / s below that (fp16 subnormals are kept by the
// conversions and by the matrix core). Scales: k-side operands (Kd, Kg, L) 2^14 (they are bounded by 1), q-side
// (Qg, M) 2^17 (bounded by 128^-1/2), T and T' 2, and what carries the magnitude of the values (S, P, V') 4: those
// must stay below 16,376 in magnitude, beyond which they become infinite where the f32 recurrence stays finite.
//
// Kernels per pass: intra_kernel (one workgroup per two chunks of a head and request: prologue, L, M, T', Kd, Qg,
// Kg, V into the workspace), inter_kernel (one workgroup per head, value-column block, request: the state in MFMA
// accumulators across the chunks of the pass); then, once per call, norm_kernel (gated RMSNorm in place, and the
// conv windows' advance).

#include <mutex>

#include "kda_common.h"

namespace kda {
namespace {

constexpr int CH = 64, SUB = 16, THREADS = 256;
constexpr int NV = 32;                    // value columns per inter workgroup
constexpr int VBLOCKS = DV / NV;          // inter workgroups per head
constexpr int NT = NV / 16;               // 16-column tiles of a workgroup's value block

typedef _Float16 f16_t;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));   // a register-friendly 128-bit piece

// Workspace of one (request, head, chunk), bytes. An MFMA operand is two planes, hi then lo, each panelled by 32
// along its contraction index ([panel][row][32]) so that the 16 rows x 32 of one operand fragment are 1 KiB of
// consecutive bytes.
constexpr int PLANE16 = 16384, PLANE8 = 8192;   // from an operand's hi plane to its lo plane
constexpr int WS_KD = 0;                  // fp16 x 2 [4 key panels][64 rows][32 keys]: -k e^G, scale 2^14
constexpr int WS_QG = 32768;              // fp16 x 2 [4 key panels][64 rows][32 keys]: q e^G, scale 2^17
constexpr int WS_KGT = 65536;             // fp16 x 2 [2 row panels][128 keys][32 rows]: k e^{G_last - G}, scale 2^14
constexpr int WS_M = 98304;               // fp16 x 2 [2 column panels][64 rows][32 columns]: M, scale 2^17
constexpr int WS_TP = 114688;             // fp16 x 2 [2 column panels][64 rows][32 columns]: T', scale 2
constexpr int WS_VT = 131072;             // bf16 [128 values][64 rows]: v, exact
constexpr int WS_E = 147456;              // f32 [128 keys]: e^{G_last}
constexpr int WS_VMAX = 147968;           // f32 [4 sub-chunks]: the largest |v| of each sub-chunk's rows (all 128 values)
constexpr int WS_CARRY = 147984;          // int [4 value blocks], in a pass's first chunk only: the serial pass before it
                                          //   leaves here the exponent term of the next chunk's scale (chunk_scale)
constexpr int WS_BYTES = 148096;             // (a multiple of 128: every slot starts on a cache line)
constexpr float SC_K = 16384.0f;          // Kd, Kg, L
constexpr float SC_Q = 131072.0f;         // Qg, M
constexpr float SC_T = 2.0f;              // T, T', and the solve's right-hand sides
static_assert(SC_K == 16384.0f && SC_Q == 131072.0f, "inter_kernel writes these as the exponents 14 and 17");
// Element index of (row, k) in a panelled matrix with `rows` rows.
__device__ __forceinline__ int panel_index(int rows, int row, int k) { return ((k >> 5) * rows + row) * 32 + (k & 31); }
// LDS row strides in 16-bit elements: 128- and 64-wide operand rows padded by 16 bytes, so that the sixteen
// rows one MFMA fragment read touches fall into distinct banks.
constexpr int LD128 = 136, LD64 = 72;

__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float fast_sigmoid(float x) { return fast_rcp(1.0f + fast_exp(-x)); }

__device__ __forceinline__ uint16_t f2h(float x) { return __builtin_bit_cast(uint16_t, (f16_t)x); }
__device__ __forceinline__ float h2f(uint16_t x) { return (float)__builtin_bit_cast(f16_t, x); }

// One operand fragment of a 16x16x32 MFMA from an LDS array [row][k] (k contiguous): lane l takes row
// row0 + l % 16, k0 + 8 * (l / 16) .. + 7. The same read serves the A operand (rows = M) and the B operand
// held transposed (rows = N).
__device__ __forceinline__ uint4 frag(const uint16_t* base, int ld, int row0, int k0, int lane) {
    return *reinterpret_cast<const uint4*>(base + (row0 + (lane & 15)) * ld + k0 + 8 * (lane >> 4));
}

__device__ __forceinline__ f32x4 mfma_f16(uint4 a, uint4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// LDS map of intra_kernel, bytes. 76.5 KB: two workgroups share a CU.
constexpr int LDD = SUB + 4;                      // f32 row stride of a diagonal block of L (16-byte multiple)
constexpr int LDT = 40, LDZ = 24;                 // 16-bit row strides of TT and Z (16-byte multiples)
constexpr int NFAC = 14;                          // per-channel factors between sub-chunks (see factor_index)
constexpr int I_CW = 0;                           // u32 [q | k | v][128 channels][4 taps]: the head's conv weights
constexpr int I_DTB = I_CW + 3 * DK * TAPS * 4;   // f32 [128]: the head's dt_bias, times -rate log2(e)
constexpr int I_TOT = I_DTB + DK * 4;             // f32 [4][128]: log2-decay totals of the sub-chunks
constexpr int I_BETA = I_TOT + 4 * DK * 4;        // f32 [64]
constexpr int I_VT = I_BETA + CH * 4;             // bf16 [128 values][LD64]: v, transposed, until it is copied out;
constexpr int I_LD = I_VT;                        //   then f32 [4][16][LDD]: the diagonal blocks of L
constexpr int I_TT = I_LD + 4 * SUB * LDD * 4;    //   and fp16 x 2 [64][LDT]: row 16 a + i holds [T_aa diag(beta) | T_aa][i][0..32)
constexpr int TT_PLANE = CH * LDT;                //   (elements from the hi plane to the lo plane)
constexpr int I_LN = I_VT + DV * LD64 * 2;        // fp16 x 2 [64][LD64]: -L below the block diagonal, zero elsewhere
constexpr int LN_PLANE = CH * LD64;
constexpr int I_KCE = I_LN + 2 * CH * LD64 * 2;   // fp16 x 2 [3][16][LD128]: 2^14 k e^{G_end - G} of sub-chunks 0..2, row major;
constexpr int KC_PLANE = 3 * SUB * LD128;         //   (elements from the hi plane to the lo plane)
constexpr int I_RT = I_KCE;                       //   later fp16 x 2 [64 columns][LD64]: the solve's right-hand sides,
constexpr int RT_PLANE = CH * LD64;               //   transposed,
constexpr int I_Z = I_RT + 2 * CH * LD64 * 2;     //   and fp16 x 2 [4 column tiles][16][LDZ]: a tile of Z on its way back
constexpr int Z_PLANE = 4 * SUB * LDZ;
constexpr int I_FAC = I_KCE + 2 * KC_PLANE * 2;    // f32 [NFAC][128]
constexpr int INTRA_LDS = I_FAC + NFAC * DK * 4;
constexpr int INTRA_CPW = 2;                      // consecutive chunks of a head per intra workgroup
static_assert(I_TT + 2 * CH * LDT * 2 <= I_LN, "the diagonal blocks and TT fit where v was");
static_assert(I_Z + 2 * Z_PLANE * 2 <= I_FAC, "the right-hand sides and Z fit the region of the column operands");
static_assert(2 * INTRA_LDS <= 160 * 1024, "two intra workgroups per CU");

// Factors e^{sum of whole sub-chunks' log decay}, per key channel: 0..3 = e^{G before sub-chunk a};
// 4..7 = e^{G_last - G at the end of sub-chunk a}; 8 + a (a - 1) / 2 + b = e^{G at the start of a - G at the end of b}
// for b < a (1 when they are neighbours).
__device__ __forceinline__ int factor_index(int a, int b) { return 8 + a * (a - 1) / 2 + b; }

// DPP moves inside a row of 16 lanes: the value n lanes below (0 where there is none), and lane n's value.
template <int N>
__device__ __forceinline__ float row_shr(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x110 + N, 0xf, 0xf, false));
}
// The same moves on raw words, in the form that needs no prepared destination (bound_ctrl: lanes without a source
// read zero): the value n lanes below, and n lanes above.
template <int N>
__device__ __forceinline__ uint32_t row_shr_u(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x110 + N, 0xf, 0xf, true);
}
template <int N>
__device__ __forceinline__ uint32_t row_shl_u(uint32_t x) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x100 + N, 0xf, 0xf, true);
}
// The value n lanes below where there is one; the other lanes (the first n of the row) keep `keep`.
template <int N>
__device__ __forceinline__ uint32_t row_shr_keep(uint32_t keep, uint32_t x) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)keep, (int)x, 0x110 + N, 0xf, 0xf, false);
}
template <int N>
__device__ __forceinline__ float row_lane(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x150 + N, 0xf, 0xf, true));
}

// a.lo * b.lo + a.hi * b.hi + c over bf16 pairs (v_dot2c_f32_bf16; within one f32 ulp of the fused form).
typedef __bf16 hwbf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(hwbf16x2, a), __builtin_bit_cast(hwbf16x2, b), c, false);
}

// The same without an addend, in the three-operand encoding: a sum that starts here needs no zeroed accumulator.
// (The one inline assembly of this file, and register operands only. An assembly *load* has no place here: the
// compiler does not know that its destination is still in flight, moves or reuses the register, and the data lands
// on whatever lives there by then - an address, once, which faults the GPU.)
__device__ __forceinline__ float dot2_bf16_first(uint32_t a, uint32_t b) {
    float r;
    asm("v_dot2_f32_bf16 %0, %1, %2, 0" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

// Eight consecutive bf16 of an input row from p. With VEC p is 16-byte aligned. Nontemporal: a row is read by one
// workgroup (and the one after it, for its first three rows), and what should stay in the caches behind the L2 is
// the workspace this pass writes for the next one (with plain loads here the inter pass measured 4 us longer).
template <bool VEC>
__device__ __forceinline__ u32x4 load8(const bf16_t* p) {
    if constexpr (VEC) {
        return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    } else {
        u32x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (uint32_t)p[2 * e] | ((uint32_t)p[2 * e + 1] << 16);
        return v;
    }
}
__device__ __forceinline__ float bf_at(const u32x4 v, int e) {   // element e of eight packed bf16
    return (e & 1) ? __uint_as_float(v[e >> 1] & 0xffff0000u) : __uint_as_float(v[e >> 1] << 16);
}
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
// Two values to fp16 in one instruction (v_cvt_pk_f16_f32, round to nearest even): lo in bits 0..15.
__device__ __forceinline__ uint32_t pack_h2(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}
// x as an fp16 pair: hi = x rounded to nearest, lo = the rounding error rounded. Two values per word, the first in
// bits 0..15.
// The rounding error a - hi is formed as fma(-hi, 1, a) with a one the optimizer cannot see through: it then takes
// the mixed-precision fused multiply-add, which reads the fp16 half in place (two instructions per pair fewer than
// widening both halves and subtracting); the difference is exact either way.
__device__ __forceinline__ void split_h2(float a, float b, uint32_t& hi, uint32_t& lo) {
    hi = pack_h2(a, b);
    const f16x2 h = __builtin_bit_cast(f16x2, hi);
    float one = 1.0f;
    asm("" : "+s"(one));
    lo = pack_h2(__builtin_fmaf(-(float)h[0], one, a), __builtin_fmaf(-(float)h[1], one, b));
}
__device__ __forceinline__ void split_h4(const f32x4 v, uint2& hi, uint2& lo) {
    split_h2(v[0], v[1], hi.x, lo.x);
    split_h2(v[2], v[3], hi.y, lo.y);
}
__device__ __forceinline__ void split_h8(const float (&v)[8], u32x4& hi, u32x4& lo) {
    uint32_t h[4], l[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) split_h2(v[2 * e], v[2 * e + 1], h[e], l[e]);
    hi = u32x4{h[0], h[1], h[2], h[3]};
    lo = u32x4{l[0], l[1], l[2], l[3]};
}
// a b with both operands as hi/lo pairs, added to c: the lo lo term is left out.
__device__ __forceinline__ f32x4 mfma_hl(uint4 ah, uint4 al, uint4 bh, uint4 bl, f32x4 c) {
    c = mfma_f16(ah, bh, c);
    c = mfma_f16(ah, bl, c);
    return mfma_f16(al, bh, c);
}
__device__ __forceinline__ f32x4 scaled(const f32x4 v, float s) { return f32x4{v[0] * s, v[1] * s, v[2] * s, v[3] * s}; }

// A 16 x 16 transpose on the matrix core. Every lane gives four 16-bit values of its row (lane l: row l % 16, the
// values at positions 4 (l / 16) .. + 3 of the row's sixteen); the product with the identity comes back in the
// accumulator layout, in which lane l holds position l % 16 of rows 4 (l / 16) .. + 3: four consecutive rows of one
// column, which is what a store into a [column][row] matrix wants. Exact: every sum has one nonzero term.
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4 transpose16(uint32_t v01, uint32_t v23, uint2 identity) {       // fp16 values
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, make_uint2(v01, v23)),
                                                 __builtin_bit_cast(f16x4, identity), zero, 0, 0, 0);
}
__device__ __forceinline__ f32x4 transpose16_bf(uint32_t v01, uint32_t v23, uint2 identity) {    // bf16 values
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, make_uint2(v01, v23)),
                                                     __builtin_bit_cast(s16x4, identity), zero, 0, 0, 0);
}
// rows 4 (l / 16) .. + 3 of column l % 16 of the identity, whose one is the 16-bit pattern `one`
__device__ __forceinline__ uint2 transpose_identity(int lane, uint32_t one) {
    const int n = lane & 15, k0 = 4 * (lane >> 4);
    return make_uint2((k0 == n ? one : 0u) | (k0 + 1 == n ? one << 16 : 0u),
                      (k0 + 2 == n ? one : 0u) | (k0 + 3 == n ? one << 16 : 0u));
}

// Pass 1: the chunks of one head of one request, everything that does not need the state, into their workspace
// slots. Wave w owns sub-chunk w of a chunk (rows 16 w .. 16 w + 15); in the elementwise phases lane l holds row
// l % 16 and 32 channels of it: with g = l / 16, the four pieces of eight channels 32 p + 8 g .. + 7, p = 0..3 (the
// four lanes of a row then read 64 consecutive bytes with every load, and write 64 with every store of Kd and Qg).
// That is the operand layout of the matrix cores for products that contract over channels, so the tiles of L and M
// take their row side straight from registers (the diagonal ones both sides); what contracts over rows later (v,
// Kg) is written transposed through the matrix core.
template <bool VEC>
__global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) intra_kernel(
        int H, const int32_t* __restrict__ cu_rows, int rows1, int sub0, int chunks,
        const bf16_t* __restrict__ P, long long p_stride, long long b_off, const bf16_t* __restrict__ A,
        long long a_stride, const bf16_t* __restrict__ conv, const long long* __restrict__ conv_off,
        const bf16_t* __restrict__ cw, const float* __restrict__ a_log, const float* __restrict__ dt_bias, float lower,
        unsigned char* __restrict__ ws) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int c_first = blockIdx.x * INTRA_CPW, h = blockIdx.y, b = blockIdx.z;
    const RowRange rr = request_rows(cu_rows, b, rows1);
    if (rr.rows - (sub0 + c_first * CH) <= 0) return;
    int t = threadIdx.x;
    const long long C = 3LL * H * DK;
    const bf16_t* cs = conv + (conv_off != nullptr ? conv_off[b] : 0);

    u32x4* cw_s = reinterpret_cast<u32x4*>(smem + I_CW);            // [3 * 128] channels, four taps each
    float* dtb_s = reinterpret_cast<float*>(smem + I_DTB);
    float* tot = reinterpret_cast<float*>(smem + I_TOT);
    float* beta_s = reinterpret_cast<float*>(smem + I_BETA);
    uint16_t* VT = reinterpret_cast<uint16_t*>(smem + I_VT);
    uint16_t* Ln = reinterpret_cast<uint16_t*>(smem + I_LN);
    float* Ld = reinterpret_cast<float*>(smem + I_LD);
    uint16_t* KcE = reinterpret_cast<uint16_t*>(smem + I_KCE);
    float* fac = reinterpret_cast<float*>(smem + I_FAC);
    float* first = reinterpret_cast<float*>(smem + I_KCE);          // [4][128]: until the column operands go there

    // the head's conv weights and dt_bias, once.
    // A conv weight is stored as the bf16 pair (w, 0) for an even channel and (0, w) for an odd one: the input rows
    // hold two channels per 32-bit word, and v_dot2c_f32_bf16 of such a word with the pair is w x + acc for the one
    // channel, with no unpacking.
    for (int e = t; e < 3 * DK; e += THREADS) {
        const uint2 w4 = *reinterpret_cast<const uint2*>(cw + ((size_t)(e >> 7) * H * DK + (size_t)h * DK + (e & (DK - 1))) * TAPS);
        const uint32_t w[4] = {w4.x & 0xffffu, w4.x >> 16, w4.y & 0xffffu, w4.y >> 16};
        const int sh = (e & 1) ? 16 : 0;
        cw_s[e] = u32x4{w[0] << sh, w[1] << sh, w[2] << sh, w[3] << sh};
    }
    // The gates work in base 2: sigmoid(r (a + dtb)) = 1 / (1 + 2^(c a + c dtb)) with c = -r log2(e), and the log
    // decays are kept in log2 units (G log2(e)), so that every e^G below is one v_exp_f32.
    const float gate_c = -fast_exp(a_log[h]) * 1.4426950408889634f;
    const float lower2 = lower * 1.4426950408889634f;
    if (t < DK) dtb_s[t] = gate_c * dt_bias[h * DK + t];
    __syncthreads();

    // Every lane's own row of q | k | v (twelve 128-bit pieces: its 32 channels of each) is requested a chunk
    // ahead: for the first chunk here, for the others while the chunk before is in its last phases. A row past the
    // end is replaced by the last real row (it only feeds rows past the end).
    u32x4 own[12];
    auto load_own = [&](int first_row) {
        const int rel = min(first_row + (int)(t & 15) + SUB * (int)(t >> 6), rr.rows - 1);
        const bf16_t* src = P + (rr.row0 + rel) * p_stride + h * DK + 8 * ((t >> 4) & 3);
#pragma unroll
        for (int it = 0; it < 12; ++it) own[it] = load8<VEC>(src + (long long)(it >> 2) * H * DK + 32 * (it & 3));
    };
    load_own(sub0 + c_first * CH);
#pragma unroll 1
    for (int c = c_first; c < min(chunks, c_first + INTRA_CPW); ++c) {
    // t, and what derives from it, are re-made for every chunk from a value the optimizer cannot see through:
    // otherwise the per-lane addresses of the body are hoisted out of the chunk loop and spill.
    asm volatile("" : "+v"(t));
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6), lane = t & 63;
    // Two workgroups share a CU, a wave of each on every SIMD, and the SIMD issues for the older wave first: left
    // alone, the workgroup that arrived first runs its chunks at full speed (23 us), the other fills the gaps (44 us)
    // and then finishes alone with nothing to hide its waits behind. So the waves' priority alternates from chunk to
    // chunk, the other way round in the second workgroup of a CU (workgroups fill the 256 CUs in the order of their
    // index), which keeps the two level and their phases apart: 66.4 -> 60.5 us per pass of 1024 rows. (Raising the
    // priority of the short phases between barriers on top of this took 3 us of that back.)
    __builtin_amdgcn_s_setprio(0);
    if ((((c - c_first) ^ (((blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) >> 8)) & 1) != 0)
        __builtin_amdgcn_s_setprio(1);
    const int i = lane & 15, g = lane >> 4;       // this lane's row of the sub-chunk and its set of 32 channels
    // what the lane holds after a transpose16: position cl_t (of the sixteen values the four lanes of a row put in:
    // lane group cl_t / 4, its value cl_t % 4) of rows rl_t .. rl_t + 3 of the sub-chunk
    const int cl_t = lane & 15, rl_t = 4 * (lane >> 4);
    const uint2 ident = transpose_identity(lane, 0x3c00u);          // fp16 1.0
    const uint2 ident_bf = transpose_identity(lane, 0x3f80u);       // bf16 1.0
    const int r0 = sub0 + c * CH;                 // the chunk's first row inside the request
    const int n = min(CH, rr.rows - r0);          // its real rows
    if (n <= 0) break;
    const int R = SUB * wave + i;                 // this lane's row inside the chunk
    unsigned char* wsc = ws + (((long long)b * H + h) * chunks + c) * (long long)WS_BYTES;
    // the row of forget-gate inputs, requested now and used after the conv (a row past the end reads the last real
    // row and counts as g = 0)
    u32x4 av[4];
    {
        const bf16_t* arow = A + (rr.row0 + r0 + min(R, n - 1)) * a_stride + h * DK + 8 * g;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            av[p] = load8<VEC>(arow + 32 * p);
        }
    }
    // the beta logit of row t (lanes of wave 0), requested now as well: its use sits right before a barrier
    const bf16_t b_raw = P[(rr.row0 + r0 + min((int)(t & (CH - 1)), n - 1)) * p_stride + b_off + h];

    // ---- conv + SiLU with one bf16 rounding (q, k stay in registers; v goes to VT as it is, bf16), and the sums of
    // squares for the L2 norms. Rows past the request's end are not masked: their beta is zero, which removes them
    // from L, T' and the state update, and their outputs are never stored.
    uint32_t qr[16], kr[16];                      // bf16 pairs: the conv outputs are bf16 values
    float ssq = 0.0f, ssk = 0.0f;
    float vmx = 0.0f;                             // the largest |v| among this lane's values (before the bf16 rounding)
    {
        // The conv's tap 3 is the lane's own row; the three rows before it are the own rows of the lanes below, a
        // DPP shift away. Lanes 0..2 of a sub-chunk also need the three rows before the sub-chunk (the conv window,
        // for the request's first rows): lane j < 3 loads row 16 w - 3 + j as its `halo`, zero in the other lanes.
        u32x4 halo[12];
        {
#pragma unroll
            for (int it = 0; it < 12; ++it) halo[it] = u32x4{0u, 0u, 0u, 0u};
            if (i < WINDOW) {
                const int hrel = min(r0 + SUB * wave - WINDOW + i, rr.rows - 1);
                const bf16_t* hsrc = (hrel < 0 ? cs + (long long)(hrel + WINDOW) * C : P + (rr.row0 + hrel) * p_stride) +
                                     h * DK + 8 * g;
#pragma unroll
                for (int it = 0; it < 12; ++it) halo[it] = load8<VEC>(hsrc + (long long)(it >> 2) * H * DK + 32 * (it & 3));
            }
        }
        uint32_t vb2[2];
#pragma unroll
        for (int it = 0; it < 12; ++it) {
            const int seg = it >> 2, p = it & 3;
#pragma unroll
            for (int d = 0; d < 4; ++d) {         // a 32-bit word holds two channels
                // taps 0..2 are the rows above: the own rows of the lanes below; the first lanes of the row, which
                // have no such lane, keep the halo row that belongs there (lane j's halo is row 16 w - 3 + j)
                const uint32_t x3 = own[it][d], hl = halo[it][d];
                const uint32_t x1 = row_shr_keep<2>(row_shl_u<1>(hl), x3);
                const uint32_t x2 = row_shr_keep<1>(row_shl_u<2>(hl), x3);
                const uint32_t x0 = row_shr_keep<3>(hl, x3);
                float s2[2];
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    const u32x4 w = cw_s[seg * DK + 32 * p + 8 * g + 2 * d + k];
                    float acc = dot2_bf16_first(x0, w[0]);
                    acc = dot2_bf16(x1, w[1], acc);
                    acc = dot2_bf16(x2, w[2], acc);
                    acc = dot2_bf16(x3, w[3], acc);
                    // SiLU as the quotient acc / (1 + e^-acc), the reference's form: the hardware reciprocal's
                    // product is corrected by one residual step (two fused operations), which makes it the
                    // correctly rounded quotient in all but a few cases per million. The plain product
                    // acc * rcp(1 + e^-acc) put one conv output in 150,000 on the other side of its bf16 rounding
                    // than the host's quotient (the chain kernel, with a true division: one in 700,000; so does
                    // this), and every such value in a row that decay has not yet forgotten moves the head's state
                    // by 2^-9 of a value: 5e-4 of the state where decay is slow.
                    {
                        // (Below -88.7 the exponential is infinite and the quotient -0, as on the host: the
                        // residual takes the largest finite number in its place, or it would be 0 x inf.)
                        const float dd = 1.0f + fast_exp(-acc);
                        const float y = fast_rcp(dd);
                        const float q0 = acc * y;
                        s2[k] = __builtin_fmaf(__builtin_fmaf(-q0, fminf(dd, 3.4028234663852886e38f), acc), y, q0);
                    }
                }
                const uint32_t pair = f2bf2(s2[0], s2[1]);        // the one bf16 rounding
                if (seg == 0) { qr[4 * p + d] = pair; ssq = dot2_bf16(pair, pair, ssq); }
                if (seg == 1) { kr[4 * p + d] = pair; ssk = dot2_bf16(pair, pair, ssk); }
                if (seg == 2) {
                    // v, transposed into VT four rows at a time: two words are four values of the row
                    vmx = fmaxf(vmx, fmaxf(fabsf(s2[0]), fabsf(s2[1])));
                    vb2[d & 1] = pair;
                    if (d & 1) {
                        const f32x4 x = transpose16_bf(vb2[0], vb2[1], ident_bf);
                        *reinterpret_cast<uint2*>(VT + (32 * p + 8 * (cl_t >> 2) + 4 * (d >> 1) + (cl_t & 3)) * LD64 +
                                                  SUB * wave + rl_t) = make_uint2(f2bf2(x[0], x[1]), f2bf2(x[2], x[3]));
                    }
                }
            }
        }
    }
    // L2 norms: the four lanes of a row hold 32 channels each. The q side of everything below carries a factor 8
    // (Qg and M are stored with scale 2^17 where the k side has 2^14).
    ssq += __shfl_xor(ssq, 16, 64);
    ssq += __shfl_xor(ssq, 32, 64);
    ssk += __shfl_xor(ssk, 16, 64);
    ssk += __shfl_xor(ssk, 32, 64);
    const float qinv = __builtin_amdgcn_rsqf(ssq + 1e-6f) * (0.08838834764831845f * (SC_Q / SC_K));   // 128^-0.5
    const float kinv = __builtin_amdgcn_rsqf(ssk + 1e-6f);
    // ---- gates: the cumulative log decay of the lane's row inside its sub-chunk, per channel
    float G[32];
    {
        const float lower_r = R < n ? lower2 : 0.0f;       // a row past the end counts as g = 0
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const f32x4 d0 = *reinterpret_cast<const f32x4*>(dtb_s + 32 * p + 8 * g);
            const f32x4 d1 = *reinterpret_cast<const f32x4*>(dtb_s + 32 * p + 8 * g + 4);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float dtb = e < 4 ? d0[e] : d1[e - 4];
                float x = lower_r * fast_rcp(1.0f + __builtin_amdgcn_exp2f(__builtin_fmaf(gate_c, bf_at(av[p], e), dtb)));
                x += row_shr<1>(x);               // inclusive scan over the sixteen rows
                x += row_shr<2>(x);
                x += row_shr<4>(x);
                x += row_shr<8>(x);
                G[8 * p + e] = x;
            }
        }
        if (i == SUB - 1) {
#pragma unroll
            for (int p = 0; p < 8; ++p)
                *reinterpret_cast<f32x4*>(tot + wave * DK + 32 * (p >> 1) + 8 * g + 4 * (p & 1)) = f32x4{G[4 * p], G[4 * p + 1], G[4 * p + 2], G[4 * p + 3]};
        }
        if (i == 0) {                             // G_0: the first row's own gate
#pragma unroll
            for (int p = 0; p < 8; ++p)
                *reinterpret_cast<f32x4*>(first + wave * DK + 32 * (p >> 1) + 8 * g + 4 * (p & 1)) = f32x4{G[4 * p], G[4 * p + 1], G[4 * p + 2], G[4 * p + 3]};
        }
    }
    if (t < CH) {
        beta_s[t] = t < n ? bfround(fast_sigmoid(bf2f(b_raw))) : 0.0f;
    }
    {
        // the largest |v| of the wave's sixteen rows, for the serial pass (chunk_scale), which takes the largest of a
        // chunk's four; the margin covers the rounding of v to bf16, which can lengthen a value by 2^-8 of itself
        vmx = fmaxf(vmx, lane_xor16<1>(vmx));
        vmx = fmaxf(vmx, lane_xor16<2>(vmx));
        vmx = fmaxf(vmx, lane_xor16<4>(vmx));
        vmx = fmaxf(vmx, lane_xor16<8>(vmx));
        const int vi = __float_as_int(vmx);
        vmx = fmaxf(fmaxf(__int_as_float(__builtin_amdgcn_readlane(vi, 0)), __int_as_float(__builtin_amdgcn_readlane(vi, 16))),
                    fmaxf(__int_as_float(__builtin_amdgcn_readlane(vi, 32)), __int_as_float(__builtin_amdgcn_readlane(vi, 48))));
        if (lane == 0) reinterpret_cast<float*>(wsc + WS_VMAX)[wave] = vmx * 1.0078125f;
    }
    __syncthreads();
    // v leaves for the workspace ([value][row], as the inter pass adds it to its accumulators): its place in LDS
    // is taken by the diagonal blocks after the next barrier
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int e = t + THREADS * j, v = e >> 2, piece = e & 3;       // 128 values x 4 pieces of 16 rows
        const uint4 lo = *reinterpret_cast<const uint4*>(VT + v * LD64 + 16 * piece);
        const uint4 hi = *reinterpret_cast<const uint4*>(VT + v * LD64 + 16 * piece + 8);
        uint4* dst = reinterpret_cast<uint4*>(wsc + WS_VT + (v * CH + 16 * piece) * 2);
        dst[0] = lo;
        dst[1] = hi;
    }
    // the factors between sub-chunks, one channel per lane; e^{G_last} goes to the workspace. The row side of the
    // tiles is kept relative to its sub-chunk's first row (k e^{G_i - G_0}), so the factors that meet it carry
    // e^{G_0} of their sub-chunk (u) on top of the decay between the sub-chunks. The factors that only make stored
    // operands (0..7) carry those operands' scale.
    {
        const int d = t & (DK - 1);
        const float t0 = tot[d], t1 = tot[DK + d], t2 = tot[2 * DK + d], t3 = tot[3 * DK + d];
        const float u0 = first[d], u1 = first[DK + d], u2 = first[2 * DK + d], u3 = first[3 * DK + d];
        if (t < DK) {
            fac[0 * DK + d] = SC_K * __builtin_amdgcn_exp2f(u0);
            fac[1 * DK + d] = SC_K * __builtin_amdgcn_exp2f(t0 + u1);
            fac[2 * DK + d] = SC_K * __builtin_amdgcn_exp2f(t0 + t1 + u2);
            fac[3 * DK + d] = SC_K * __builtin_amdgcn_exp2f(t0 + t1 + t2 + u3);
            reinterpret_cast<float*>(wsc + WS_E)[d] = __builtin_amdgcn_exp2f(t0 + t1 + t2 + t3);
            fac[4 * DK + d] = SC_K * __builtin_amdgcn_exp2f(t1 + t2 + t3);
            fac[5 * DK + d] = SC_K * __builtin_amdgcn_exp2f(t2 + t3);
        } else {
            fac[6 * DK + d] = SC_K * __builtin_amdgcn_exp2f(t3);
            fac[7 * DK + d] = SC_K;
            fac[factor_index(1, 0) * DK + d] = SC_K * __builtin_amdgcn_exp2f(u1);
            fac[factor_index(2, 0) * DK + d] = SC_K * __builtin_amdgcn_exp2f(t1 + u2);
            fac[factor_index(2, 1) * DK + d] = SC_K * __builtin_amdgcn_exp2f(u2);
            fac[factor_index(3, 0) * DK + d] = SC_K * __builtin_amdgcn_exp2f(t1 + t2 + u3);
            fac[factor_index(3, 1) * DK + d] = SC_K * __builtin_amdgcn_exp2f(t2 + u3);
            fac[factor_index(3, 2) * DK + d] = SC_K * __builtin_amdgcn_exp2f(u3);
        }
    }

    __syncthreads();                              // the factors are in place, v has left

    // ---- operands. Per element: ep = e^{G_i - G_0} and its reciprocal (G_0: the sub-chunk's first row, so that
    // fifteen rows of decay bound the exponent); e^{G_15 - G_i} is the last row's ep over the own one.
    // The tiles of L and M run on the f32 matrix instruction, four channels per step (one per lane group): the
    // diagonal ones take k ep, q ep (rows) and k / ep (columns) straight from registers; the same k ep, q ep are the
    // row side of the other tiles and of Kd and Qg, times factors that carry e^{G_0}.
    // The tiles are computed transposed (column side first in the MFMA), so an accumulator holds columns rl..rl+3 of
    // row cl of a tile: four consecutive elements of a row of L or M, one store per plane.
    const int rl = 4 * (lane >> 4), cl = lane & 15;
    uint16_t* Mg = reinterpret_cast<uint16_t*>(wsc + WS_M);
    // Store a finished tile at block (rb, cb). L = beta_i * acc: a diagonal block (strictly lower) in f32 for the
    // inversion, a block below the diagonal negated as an fp16 pair, an MFMA operand of the block solve. M (lower
    // with the diagonal; acc holds 8 M) goes to the workspace.
    auto put_L = [&](f32x4 acc, int rb, int cb, float unit) {
        const int gi = SUB * rb + cl, gj = SUB * cb + rl;
        const float bi = beta_s[gi];
        if (rb == cb) {
            f32x4 v;
#pragma unroll
            for (int r = 0; r < 4; ++r) v[r] = rl + r < cl ? bi * acc[r] : 0.0f;
            *reinterpret_cast<f32x4*>(Ld + gi * LDD + rl) = v;
            *reinterpret_cast<uint2*>(Ln + gi * LD64 + gj) = make_uint2(0u, 0u);
            *reinterpret_cast<uint2*>(Ln + LN_PLANE + gi * LD64 + gj) = make_uint2(0u, 0u);
        } else {
            uint2 hi, lo;
            split_h4(scaled(acc, -SC_K * unit * bi), hi, lo);
            *reinterpret_cast<uint2*>(Ln + gi * LD64 + gj) = hi;
            *reinterpret_cast<uint2*>(Ln + LN_PLANE + gi * LD64 + gj) = lo;
        }
    };
    auto put_M = [&](f32x4 acc, int rb, int cb, float unit) {
        const int gi = SUB * rb + cl, gj = SUB * cb + rl;
        f32x4 v;
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] = (rb != cb || gj + r <= gi) ? acc[r] * (SC_K * unit) : 0.0f;
        uint2 hi, lo;
        split_h4(v, hi, lo);
        *reinterpret_cast<uint2*>(Mg + panel_index(CH, gi, gj)) = hi;
        *reinterpret_cast<uint2*>(Mg + PLANE8 / 2 + panel_index(CH, gi, gj)) = lo;
    };
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    float kep[32], qep[32];                       // k e^{G_i - G_0}, 8 q e^{G_i - G_0}: the row side of every tile
    {
        f32x4 accL = zero, accM = zero;
        uint16_t* kgT = reinterpret_cast<uint16_t*>(wsc + WS_KGT);
        const float* eB = fac + wave * DK + 8 * g;
        const float* eSuf = fac + (4 + wave) * DK + 8 * g;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const f32x4 b0 = *reinterpret_cast<const f32x4*>(eB + 32 * p), b1 = *reinterpret_cast<const f32x4*>(eB + 32 * p + 4);
            const f32x4 s0 = *reinterpret_cast<const f32x4*>(eSuf + 32 * p), s1 = *reinterpret_cast<const f32x4*>(eSuf + 32 * p + 4);
            float qg[8], kc[8], kd[8], kgt[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int ch = 8 * p + e;
                const float Gi = G[ch];
                const float G0 = row_lane<0>(Gi);
                const float ep = __builtin_amdgcn_exp2f(Gi - G0);
                const float rp = fast_rcp(ep);                  // e^{G_0 - G_i}, up to e^87
                const float last = row_lane<SUB - 1>(ep);       // e^{G_15 - G_0}
                const float kraw = (ch & 1) ? __uint_as_float(kr[ch >> 1] & 0xffff0000u) : __uint_as_float(kr[ch >> 1] << 16);
                const float qraw = (ch & 1) ? __uint_as_float(qr[ch >> 1] & 0xffff0000u) : __uint_as_float(qr[ch >> 1] << 16);
                const float kh = kraw * kinv, qh = qraw * qinv;
                const float kcd = kh * rp;
                kep[ch] = kh * ep;
                qep[ch] = qh * ep;
                accL = __builtin_amdgcn_mfma_f32_16x16x4f32(kcd, kep[ch], accL, 0, 0, 0);
                accM = __builtin_amdgcn_mfma_f32_16x16x4f32(kcd, qep[ch], accM, 0, 0, 0);
                const float fb = e < 4 ? b0[e] : b1[e - 4], fs = e < 4 ? s0[e] : s1[e - 4];
                kd[e] = -(kep[ch] * fb);                        // -2^14 k e^{G_i} from the chunk's start
                qg[e] = qep[ch] * fb;                           // 2^17 q e^{G_i}
                kc[e] = kcd * last;                             // k e^{G_15 - G_i}
                kgt[e] = kc[e] * fs;                            // 2^14 k e^{G_last - G_i}
            }
            // Kg into the workspace [key][row]: transposed four rows at a time, the hi and the lo plane each
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const int key = 32 * p + 8 * (cl_t >> 2) + 4 * hf + (cl_t & 3);
                uint32_t h01, l01, h23, l23;
                split_h2(kgt[4 * hf], kgt[4 * hf + 1], h01, l01);
                split_h2(kgt[4 * hf + 2], kgt[4 * hf + 3], h23, l23);
                const f32x4 yh = transpose16(h01, h23, ident), yl = transpose16(l01, l23, ident);
                uint16_t* dst = kgT + panel_index(DK, key, SUB * wave + rl_t);
                *reinterpret_cast<uint2*>(dst) = make_uint2(pack_h2(yh[0], yh[1]), pack_h2(yh[2], yh[3]));
                *reinterpret_cast<uint2*>(dst + PLANE16 / 2) = make_uint2(pack_h2(yl[0], yl[1]), pack_h2(yl[2], yl[3]));
            }
            {
                u32x4 hi, lo;
                split_h8(kd, hi, lo);
                unsigned char* dst = wsc + WS_KD + panel_index(CH, R, 32 * p + 8 * g) * 2;
                *reinterpret_cast<u32x4*>(dst) = hi;
                *reinterpret_cast<u32x4*>(dst + PLANE16) = lo;
                split_h8(qg, hi, lo);
                dst = wsc + WS_QG + panel_index(CH, R, 32 * p + 8 * g) * 2;
                *reinterpret_cast<u32x4*>(dst) = hi;
                *reinterpret_cast<u32x4*>(dst + PLANE16) = lo;
            }
            if (wave < 3) {
                float kcs[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) kcs[e] = kc[e] * SC_K;
                u32x4 hi, lo;
                split_h8(kcs, hi, lo);
                uint16_t* dst = KcE + (wave * SUB + i) * LD128 + 32 * p + 8 * g;
                *reinterpret_cast<u32x4*>(dst) = hi;
                *reinterpret_cast<u32x4*>(dst + KC_PLANE) = lo;
            }
        }
        put_L(accL, wave, wave, 1.0f);
        put_M(accM, wave, wave, 1.0f);
    }
    __syncthreads();                              // the column operands of every sub-chunk are in place
    uint16_t* TT = reinterpret_cast<uint16_t*>(smem + I_TT);
    if (wave == 0) {
        // Sub-chunk 0 has no tiles left of its diagonal, so while the other waves compute theirs wave 0 does what
        // needs the diagonal blocks only.
        // M and T' are zero above the block diagonal. The inter pass reads a row's columns 0..31 always and 32..63
        // from row 32 on, so of the six blocks there it meets two, (0,1) and (2,3): those are written as zeros, in
        // 128-bit pieces (two per row of a block), both planes; the other four stay as they are, unread. (-L above the
        // diagonal is never read either: the solve below starts a block column at its diagonal block.)
        {
            const int blk = lane >> 5, r = (lane >> 1) & 15, half = lane & 1;
            const int rb = 2 * blk, cb = 2 * blk + 1;
            const u32x4 z = {0u, 0u, 0u, 0u};
            uint16_t* Tz = reinterpret_cast<uint16_t*>(wsc + WS_TP);
            *reinterpret_cast<u32x4*>(Mg + panel_index(CH, SUB * rb + r, SUB * cb + 8 * half)) = z;
            *reinterpret_cast<u32x4*>(Mg + PLANE8 / 2 + panel_index(CH, SUB * rb + r, SUB * cb + 8 * half)) = z;
            *reinterpret_cast<u32x4*>(Tz + panel_index(CH, SUB * rb + r, SUB * cb + 8 * half)) = z;
            *reinterpret_cast<u32x4*>(Tz + PLANE8 / 2 + panel_index(CH, SUB * rb + r, SUB * cb + 8 * half)) = z;
        }
        // ---- the diagonal blocks of T = (I + L)^-1 in f32 by forward substitution: lane (a, j) solves column j of
        // block a and leaves it as fp16 pairs (scale 2), scaled by beta_j (T' = T diag(beta)) and plain.
        const int a = lane >> 4, j = lane & 15;
        const float bj = beta_s[lane];
        // the block's strictly lower triangle into registers (rows as 128-bit pieces), then the substitution
        // column by column: once x[m] is known every later row takes its term, sixteen independent chains
        float l[SUB][SUB];
#pragma unroll
        for (int i = 1; i < SUB; ++i)
#pragma unroll
            for (int p = 0; p < (i + 3) / 4; ++p) {
                const f32x4 v = *reinterpret_cast<const f32x4*>(Ld + (SUB * a + i) * LDD + 4 * p);
#pragma unroll
                for (int e = 0; e < 4; ++e) l[i][4 * p + e] = v[e];
            }
        float acc[SUB], x[SUB];
#pragma unroll
        for (int i = 0; i < SUB; ++i) acc[i] = 0.0f;
#pragma unroll
        for (int m = 0; m < SUB; ++m) {
            x[m] = m < j ? 0.0f : (m == j ? 1.0f : -acc[m]);
#pragma unroll
            for (int i = m + 1; i < SUB; ++i) acc[i] = __builtin_fmaf(l[i][m], x[m], acc[i]);
        }
#pragma unroll
        for (int i = 0; i < SUB; ++i) {
            const float tp = x[i] * (bj * SC_T), tn = x[i] * SC_T;
            const uint16_t tph = f2h(tp), tnh = f2h(tn);
            uint16_t* row = TT + (SUB * a + i) * LDT;
            row[j] = tph;
            row[SUB + j] = tnh;
            row[TT_PLANE + j] = f2h(tp - h2f(tph));
            row[TT_PLANE + SUB + j] = f2h(tn - h2f(tnh));
        }
    } else {
        // tiles left of the diagonal: rows of sub-chunk `wave` against the columns of sub-chunk cb. Both sides have
        // exponents <= 0 here (the column side relative to its sub-chunk's end, the row side with the decay between
        // the sub-chunks in its factor), so they fit fp16 pairs with scale 2^14 and the tiles take the fp16 matrix
        // instruction: 24 of 16 cycles per pair of tiles instead of 64 of 32 on the f32 one, for the cost of
        // splitting the row side once per column block. In step p lane group g supplies channels 32 p + 8 g .. + 7
        // on both sides; the accumulators are in units of 2^28.
#pragma unroll 1
        for (int cb = 0; cb < wave; ++cb) {
            const float* df = fac + factor_index(wave, cb) * DK + 8 * g;
            f32x4 accL = zero, accM = zero;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const f32x4 d0 = *reinterpret_cast<const f32x4*>(df + 32 * p), d1 = *reinterpret_cast<const f32x4*>(df + 32 * p + 4);
                float rk[8], rq[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float f = e < 4 ? d0[e] : d1[e - 4];
                    rk[e] = kep[8 * p + e] * f;
                    rq[e] = qep[8 * p + e] * f;
                }
                u32x4 kh, kl, qh, ql;
                split_h8(rk, kh, kl);
                split_h8(rq, qh, ql);
                const uint4 ch = frag(KcE, LD128, cb * SUB, 32 * p, lane), cl2 = frag(KcE + KC_PLANE, LD128, cb * SUB, 32 * p, lane);
                accL = mfma_hl(ch, cl2, make_uint4(kh[0], kh[1], kh[2], kh[3]), make_uint4(kl[0], kl[1], kl[2], kl[3]), accL);
                accM = mfma_hl(ch, cl2, make_uint4(qh[0], qh[1], qh[2], qh[3]), make_uint4(ql[0], ql[1], ql[2], ql[3]), accM);
            }
            put_L(accL, wave, cb, 1.0f / (SC_K * SC_K));
            put_M(accM, wave, cb, 1.0f / (SC_K * SC_K));
        }
    }
    __syncthreads();                              // L and TT are complete; the factors and column operands are dead
    if (c + 1 < min(chunks, c_first + INTRA_CPW)) load_own(r0 + CH);   // the next chunk's rows

    // ---- T' = (I + L)^-1 diag(beta) without ever forming the blocks of T below the diagonal: block forward
    // substitution on R = I (64 rows, 64 columns), held transposed in LDS ([column][row]) and solved in place.
    // Wave w owns the sixteen columns of block column w; no barrier:
    //   Z_a = -sum_{b<a} L_ab X_b,   X_a = T'_aa R_a + T_aa Z_a,   from a = w on (the blocks above are zero).
    // Every operand is an fp16 pair with scale 2 (L: 2^14).
    {
        uint16_t* RT = reinterpret_cast<uint16_t*>(smem + I_RT);
        uint16_t* Zs = reinterpret_cast<uint16_t*>(smem + I_Z);
        // the wave's columns of the identity (2.0 as fp16: the scale), lo plane zero: lane (column cl, rows 16 q ..)
        {
            const int q = lane >> 4;
            uint32_t w[8];
#pragma unroll
            for (int m = 0; m < 8; ++m)
                w[m] = (q == wave && (cl >> 1) == m) ? ((cl & 1) ? 0x40000000u : 0x4000u) : 0u;
            uint16_t* dst = RT + (SUB * wave + cl) * LD64 + SUB * q;
            const u32x4 z = {0u, 0u, 0u, 0u};
            *reinterpret_cast<u32x4*>(dst) = u32x4{w[0], w[1], w[2], w[3]};
            *reinterpret_cast<u32x4*>(dst + 8) = u32x4{w[4], w[5], w[6], w[7]};
            *reinterpret_cast<u32x4*>(dst + RT_PLANE) = z;
            *reinterpret_cast<u32x4*>(dst + RT_PLANE + 8) = z;
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        uint16_t* Tg = reinterpret_cast<uint16_t*>(wsc + WS_TP);
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            if (a < wave) continue;               // (wave is uniform: whole iterations drop out)
            const uint4 tth = frag(TT, LDT, SUB * a, 0, lane), ttl = frag(TT + TT_PLANE, LDT, SUB * a, 0, lane);
            if (a > wave) {
                // Z tile [16 rows j][16 columns c]: a lane ends with four consecutive rows of one column
                f32x4 z = zero;
                z = mfma_hl(frag(Ln, LD64, SUB * a, 0, lane), frag(Ln + LN_PLANE, LD64, SUB * a, 0, lane),
                            frag(RT, LD64, SUB * wave, 0, lane), frag(RT + RT_PLANE, LD64, SUB * wave, 0, lane), z);
                if (a == 3)
                    z = mfma_hl(frag(Ln, LD64, SUB * a, 32, lane), frag(Ln + LN_PLANE, LD64, SUB * a, 32, lane),
                                frag(RT, LD64, SUB * wave, 32, lane), frag(RT + RT_PLANE, LD64, SUB * wave, 32, lane), z);
                uint2 hi, lo;
                split_h4(scaled(z, 1.0f / SC_K), hi, lo);
                *reinterpret_cast<uint2*>(Zs + (wave * SUB + cl) * LDZ + rl) = hi;
                *reinterpret_cast<uint2*>(Zs + Z_PLANE + (wave * SUB + cl) * LDZ + rl) = lo;
                // other lanes of the wave read the tile back below: the order of those LDS accesses is pinned (no
                // instruction is emitted for either line; a wave's LDS accesses complete in order)
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
            // [R_a | Z_a] of the column tile as an operand [16 columns][K = 32]: k < 16 is R_a (lanes 0..31), k >= 16
            // is Z_a (lanes 32..63): one read per plane at a per-lane offset, no branch
            const int off_r = I_RT + ((SUB * wave + cl) * LD64 + SUB * a + 8 * (lane >> 4)) * 2;
            const int off_z = I_Z + ((wave * SUB + cl) * LDZ + 8 * ((lane >> 4) - 2)) * 2;
            uint4 rzh = *reinterpret_cast<const uint4*>(smem + (lane < 32 ? off_r : off_z));
            uint4 rzl = *reinterpret_cast<const uint4*>(smem + (lane < 32 ? off_r + RT_PLANE * 2 : off_z + Z_PLANE * 2));
            if (a == wave) {                      // Z_w = 0
                const uint32_t keep = lane < 32 ? 0xffffffffu : 0u;
                rzh = make_uint4(rzh.x & keep, rzh.y & keep, rzh.z & keep, rzh.w & keep);
                rzl = make_uint4(rzl.x & keep, rzl.y & keep, rzl.z & keep, rzl.w & keep);
            }
            // both ways round: the X tile [16 rows][16 columns] leaves a lane four consecutive rows of one column for
            // R^T, the X^T tile four consecutive columns of one row of T' [row][column] for the workspace
            const f32x4 x = mfma_hl(tth, ttl, rzh, rzl, zero);
            const f32x4 xt = mfma_hl(rzh, rzl, tth, ttl, zero);
            uint2 hi, lo;
            split_h4(scaled(x, 1.0f / SC_T), hi, lo);
            *reinterpret_cast<uint2*>(RT + (SUB * wave + cl) * LD64 + SUB * a + rl) = hi;
            *reinterpret_cast<uint2*>(RT + RT_PLANE + (SUB * wave + cl) * LD64 + SUB * a + rl) = lo;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");      // the next block's fragments of R^T read these
            __builtin_amdgcn_wave_barrier();
            split_h4(scaled(xt, 1.0f / SC_T), hi, lo);
            *reinterpret_cast<uint2*>(Tg + panel_index(CH, SUB * a + cl, SUB * wave + rl)) = hi;
            *reinterpret_cast<uint2*>(Tg + PLANE8 / 2 + panel_index(CH, SUB * a + cl, SUB * wave + rl)) = lo;
        }
    }
    __syncthreads();                              // the next chunk's conv writes VT before its first barrier
    }
}

// LDS map of inter_kernel, bytes: only what the waves share, each as an fp16 pair of planes.
// Row strides and placement of what the waves exchange. A row is padded by 32 bytes and the 16-byte pieces of rows
// 4..7 and 12..15 of every sixteen swap places in pairs: with that a fragment read (ds_read_b128: sixteen rows, four
// pieces) runs at the full LDS rate and a tile store (ds_write_b64: sixteen rows, four elements) at the stores' best,
// where 16 bytes of padding alone gave 0.63 and 0.93 of those rates (measured in a probe of the two access patterns
// over strides and swizzles; this launch's first phase is bound by its 128 KB of fragment reads per chunk).
constexpr int NLD128 = 144, NLD64 = 80;
__device__ __forceinline__ int piece_swap(int row) { return ((row >> 2) & 1) << 3; }      // in 16-bit elements
__device__ __forceinline__ uint4 nfrag(const uint16_t* base, int ld, int row0, int k0, int lane) {
    return *reinterpret_cast<const uint4*>(base + (row0 + (lane & 15)) * ld + ((k0 + 8 * (lane >> 4)) ^ piece_swap(lane & 15)));
}
constexpr int S_PLANE = NV * NLD128, P_PLANE = NV * NLD64;   // elements from a hi plane to its lo plane
constexpr int N_S = 0;                            // fp16 x 2 [NV][NLD128]: the state, transposed
constexpr int N_P = N_S + 2 * S_PLANE * 2;    // fp16 x 2 [NV][NLD64]: P, transposed
constexpr int N_V = N_P + 2 * P_PLANE * 2;        // fp16 x 2 [NV][NLD64]: V', transposed
constexpr int N_X = N_V + 2 * P_PLANE * 2;         // int [4]: per state wave, the exponent of the largest |S| entering the chunk
constexpr int INTER_LDS = N_X + 16;

// The scale of S, P and V' in a chunk. Those three pass through fp16 pairs, so they are carried times a power of two,
// 2^es, chosen per chunk from a bound on everything the chunk can produce. With N a bound on the 2-norm of every value
// column of the state entering the chunk and m the largest |v| in it: k is normalised, beta and the decay are at most
// one, so every row of the recurrence lengthens a column by at most m, and an entry of S, of P = V - Kd S and of
// V' = T' P (the recurrence's own deltas) stays below N + 64 m. N follows the state one chunk behind, which keeps the
// bookkeeping off the chain: for chunk c + 1 it is sqrt(128) times the largest entry of the state that entered
// chunk c (measured by the state waves while they wait for that chunk's V', read by everyone behind the chunk's
// last matrix products) plus chunk c's 64 m. Only exponents are kept (integers: no rounding, so the scales, and
// with them every bit of the result, do not depend on where the passes are cut): with |x| < 2^(e + 1) written
// e(x), the terms of the bound are below 2^(e(S) + 5) and 2^(e(m) + 7), their sum below 2^(E + 2) with E the
// largest of the exponents, and es = 15 - (E + 2) puts everything below 2^15, half of fp16's largest number; what
// the exponents round up costs at most four of the pairs' forty bits of range below the bound. A launch's first
// chunk takes its term from the state it loads (a request's first rows) or from what the launch before left in
// the workspace (WS_CARRY). es is kept in [-50, 50]: a state beyond 2^61 (2e18) becomes infinite, below 2^-39 the
// pairs' absolute floor of 2^-75 shows. What one scale per chunk cannot follow is a state that collapses by more
// than 2^25 inside a chunk while the values stay small: the next chunk still carries the old bound, and values
// more than 2^40 below it are lost to that chunk.
constexpr int kScaleMin = -50, kScaleMax = 50;
__device__ __forceinline__ int exponent_of(uint32_t bits) { return (int)((bits >> 23) & 0xffu) - 127; }   // |x| < 2^(e + 1)
// es from X (the largest exponent term of the chunks before) and the exponent of this chunk's largest |v|
__device__ __forceinline__ int chunk_scale(int x, int ev) { return min(max(15 - (max(x, ev + 7) + 2), kScaleMin), kScaleMax); }
__device__ __forceinline__ float pow2i(int e) { return __uint_as_float((uint32_t)(e + 127) << 23); }   // -126 <= e <= 127
// The largest |x| over a wave's accumulators as a bit pattern, the same in every lane (the patterns of non-negative
// floats order like unsigned integers: integer maxima, no conversions).
__device__ __forceinline__ uint32_t wave_max_abs_bits(const f32x4 (&a)[2][NT]) {
    uint32_t m = 0u;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int r = 0; r < 4; ++r) m = max(m, __float_as_uint(a[mt][nt][r]) & 0x7fffffffu);
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0xB1, 0xf, 0xf, true));       // lanes ^ 1
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x4E, 0xf, 0xf, true));       // lanes ^ 2
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x124, 0xf, 0xf, true));      // rotate by 4 inside a row of 16
    m = max(m, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)m, 0x128, 0xf, 0xf, true));      // rotate by 8
    return max(max((uint32_t)__builtin_amdgcn_readlane((int)m, 0), (uint32_t)__builtin_amdgcn_readlane((int)m, 16)),
               max((uint32_t)__builtin_amdgcn_readlane((int)m, 32), (uint32_t)__builtin_amdgcn_readlane((int)m, 48)));
}

template <typename S>
__device__ __forceinline__ float load_state_elem4(const S* p, float (&v)[4]);
template <>
__device__ __forceinline__ float load_state_elem4<float>(const float* p, float (&v)[4]) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
    return 0.0f;
}
template <>
__device__ __forceinline__ float load_state_elem4<bf16_t>(const bf16_t* p, float (&v)[4]) {
    const uint2 x = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(x.x << 16); v[1] = __uint_as_float(x.x & 0xffff0000u);
    v[2] = __uint_as_float(x.y << 16); v[3] = __uint_as_float(x.y & 0xffff0000u);
    return 0.0f;
}
__device__ __forceinline__ void store_state_elem4(float* p, const f32x4 v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store_state_elem4(bf16_t* p, const f32x4 v) {
    *reinterpret_cast<uint2*>(p) = make_uint2(f2bf2(v[0], v[1]), f2bf2(v[2], v[3]));
}

// One chunk's operands of inter_kernel as a wave holds them: MFMA fragments straight from the workspace, hi and lo
// plane. The workgroup has two kinds of wave. State wave w (waves 0..3) owns rows 16 w .. 16 w + 15 of the chunk
// for P (Kd, V) and keys 32 w .. 32 w + 31 of the state (Kg, e^{G_last}); read-out wave w (waves 4..7) owns rows
// 16 w .. 16 w + 15 of the chunk for V' (T') and Y (Qg, M). Nothing a wave loads is used by another wave, so none
// of it passes through LDS.
struct StateOperands {
    u32x4 kd[2][4];                               // [plane] rows 16 w + l % 16, keys 32 ks + 8 (l / 16) ..
    u32x4 k[2][2][2];                             // [plane] keys 32 w + 16 mt + l % 16, chunk rows 32 ks + 8 (l / 16) ..
    uint2 v[NT];                                  // bf16: value column of (nt, l % 16), rows 16 w + 4 (l / 16) ..
    f32x4 e[2];                                   // keys 32 w + 16 mt + 4 (l / 16) ..
};
struct ReadoutOperands {
    u32x4 q[2][4];                                // [plane] rows 16 w + l % 16, keys 32 ks + 8 (l / 16) ..
    u32x4 m[2][2];                                // [plane] rows 16 w + l % 16, chunk rows 32 ks + 8 (l / 16) ..
    u32x4 t[2][2];                                // the same of T'
};
constexpr int INTER_THREADS = 512;
static_assert(NT == 2, "the value-column order below pairs two tiles");
// Row m of value tile nt (of a workgroup's transposed state, P and V') is value column 8 (m / 4) + 4 nt + m % 4 of
// the block: a read-out accumulator holds rows 4 g .. 4 g + 3 of both tiles, which is then eight consecutive values
// of one output row, one 128-bit store.
__device__ __forceinline__ int value_col(int nt, int m) { return 8 * (m >> 2) + 4 * nt + (m & 3); }

// Pass 2: one head's NV value columns of one request through the chunks of the pass, in order. The state
// S[128 keys][NV] lives in the MFMA accumulators of the state waves (wave w owns keys 32 w .. 32 w + 31), in units of
// 2^14 2^e S: the scale of Kg times the chunk's scale of V' (chunk_scale). Per chunk, three barriers:
//   state waves:    S -> LDS | P = V - Kd S -> LDS         | max |S|; S <- e^{G_last} S      | S += Kg^T V'; next scale
//   read-out waves:          | store rows c - 1; Y = Qg S  | V' = T' P -> LDS                | Y += M V'
// so the chain from one chunk's state to the next is three products, and in every interval the read-out waves have
// no more to do than the state waves (with the whole of Y after the third barrier they held up the next chunk's
// first barrier: 3.4 us per chunk instead of 3.1 with the workspace in HBM, 2.6 with it in the cache behind the L2).
template <typename S>
__global__ void __launch_bounds__(INTER_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) inter_kernel(
        int H, const int32_t* __restrict__ cu_rows, int rows1, int sub0, int chunks,
        const S* state_in, S* state_out, const long long* __restrict__ state_off,
        bf16_t* __restrict__ out, long long out_stride, const unsigned char* __restrict__ ws, unsigned char* carry_ws) {
    extern __shared__ __align__(16) unsigned char smem[];
    // Workgroups go to the eight XCDs round robin by their linear index. The value-column blocks of one head
    // read the same Kd, Qg, Kg, M and T', so they are spaced H apart (a multiple of 8 for the model's 64 heads):
    // they run on one XCD and share its L2 instead of fetching the workspace once per block.
    const int h = blockIdx.x % H, vb = blockIdx.x / H, b = blockIdx.y;
    const RowRange rr = request_rows(cu_rows, b, rows1);
    const int t = threadIdx.x, lane = t & 63;
    const int wave8 = __builtin_amdgcn_readfirstlane(t >> 6);
    const bool state_wave = wave8 < 4;
    const int wave = wave8 & 3;
    const int left = rr.rows - sub0;                              // rows of this request from this pass on
    const int nch = left <= 0 ? 0 : min(chunks, (left + CH - 1) / CH);
    if (nch == 0 && sub0 > 0) return;                             // nothing left: the state is already written
    const long long sbase = (state_off != nullptr ? state_off[b] : 0) + (long long)h * DV * DK;
    const int rl = 4 * (lane >> 4), cl = lane & 15;

    uint16_t* Sl = reinterpret_cast<uint16_t*>(smem + N_S);
    uint16_t* Pl = reinterpret_cast<uint16_t*>(smem + N_P);
    uint16_t* Vl = reinterpret_cast<uint16_t*>(smem + N_V);
    const unsigned char* wsh = ws + ((long long)b * H + h) * chunks * (long long)WS_BYTES;
    // (the same slot through the pointer that may write: the carry words are only ever touched through this one)
    int* carry = reinterpret_cast<int*>(carry_ws + ((long long)b * H + h) * chunks * (long long)WS_BYTES + WS_CARRY + 4 * vb);
    // Per-lane byte offsets of the fragments inside a chunk's workspace.
    const unsigned off_a = (unsigned)(((SUB * wave + cl) * 32 + 8 * (lane >> 4)) * 2);   // Kd, Qg, M, T': + 4096 ks
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    auto as_u4 = [](const u32x4 v) { return make_uint4(v[0], v[1], v[2], v[3]); };
    // The chunks' scales (chunk_scale), the same integers in every wave of the workgroup. ev_*: the exponents of the
    // largest |v| of the chunk before, this chunk and the next. The one after the next is requested at the top of
    // a chunk's iteration and turned into an exponent at its end (the conversion waits for the load; loaded words
    // that live across the loop's back edge cost a register copy there, with a wait for the load in front of it).
    auto ev_request = [&](int c) {
        return *reinterpret_cast<const u32x4*>(wsh + (long long)min(c, nch - 1) * WS_BYTES + WS_VMAX);
    };
    auto ev_of = [](const u32x4 v) {                               // (positive floats order like their bit patterns)
        return __builtin_amdgcn_readfirstlane(exponent_of(max(max(v[0], v[1]), max(v[2], v[3]))));
    };
    int* mx = reinterpret_cast<int*>(smem + N_X);
    // The exponent of the largest |S| that entered the chunk, over the four state waves.
    auto state_exponent = [&]() {
        const u32x4 m4 = *reinterpret_cast<const u32x4*>(mx);
        return __builtin_amdgcn_readfirstlane(max(max((int)m4[0], (int)m4[1]), max((int)m4[2], (int)m4[3])));
    };
    int ev_cur = 0, ev_next = 0;
    int x_cur = 0;                                // the next chunk's exponent term of what came before it
    int es = 0;
    // Chunk c's step of the bookkeeping, anywhere between its third barrier and the next chunk's first: the next
    // chunk's scale from the state that entered chunk c and the values of chunks c and c + 1.
    auto step = [&](const u32x4 ev_after_raw) __attribute__((always_inline)) {
        x_cur = max(state_exponent() + 5, ev_cur + 7);
        ev_cur = ev_next;
        ev_next = ev_of(ev_after_raw);
        return chunk_scale(x_cur, ev_cur);
    };
    // Before the first chunk: the term comes from the loaded state (whose exponent the state waves have put in mx,
    // a barrier ago) or from the launch before.
    // (What it loads is requested here, ahead of the state and of the first chunk's operands: vector loads arrive in
    // order, and the first chunk's scale is needed before any of those.)
    const int nch1 = max(nch, 1);
    const u32x4 ev0_raw = *reinterpret_cast<const u32x4*>(wsh + WS_VMAX);
    const u32x4 ev1_raw = *reinterpret_cast<const u32x4*>(wsh + (long long)min(1, nch1 - 1) * WS_BYTES + WS_VMAX);
    const int carry_raw = *carry;
    auto first_scale = [&]() __attribute__((always_inline)) {
        ev_cur = ev_of(ev0_raw);
        ev_next = ev_of(ev1_raw);
        x_cur = sub0 == 0 ? state_exponent() + 5 : __builtin_amdgcn_readfirstlane(carry_raw);
        return chunk_scale(x_cur, ev_cur);
    };

    if (state_wave) {
        // the state: accS[mt][nt][r] = 2^eu S[key 32 w + 16 mt + rl + r][value NV vb + value_col(nt, cl)]
        f32x4 accS[2][NT];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                float v4[4];
                load_state_elem4<S>(state_in + sbase + (long long)(NV * vb + value_col(nt, cl)) * DK + 32 * wave + SUB * mt + rl, v4);
                accS[mt][nt] = f32x4{v4[0], v4[1], v4[2], v4[3]};
            }
        int eu = 0;                               // the accumulators hold 2^eu S
        const unsigned off_k = (unsigned)(WS_KGT + ((32 * wave + cl) * 32 + 8 * (lane >> 4)) * 2);  // + 1024 mt + 8192 ks
        const unsigned off_v = (unsigned)(WS_VT + ((NV * vb + value_col(0, cl)) * CH + SUB * wave + rl) * 2);   // + 512 nt
        const unsigned off_e = (unsigned)(WS_E + (32 * wave + rl) * 4);                             // + 64 mt
        // The loads of chunk C_ into the operand set X_, one group at a time: each group is requested again, for the
        // next chunk, as soon as this chunk has used it, so a request has all but one phase of a chunk to arrive (a
        // second set, requested two chunks ahead, costs 80 registers and measured 2 % slower).
        // Unconditional: past the end they repeat the last chunk.
#define KDA_LOAD_KD(X_, C_)                                                                                         \
        {                                                                                                           \
            const unsigned char* src_ = wsh + (long long)(C_) * WS_BYTES;                                           \
            _Pragma("unroll") for (int pl = 0; pl < 2; ++pl)                                                        \
                _Pragma("unroll") for (int ks = 0; ks < 4; ++ks)                                                    \
                    X_.kd[pl][ks] = *reinterpret_cast<const u32x4*>(src_ + WS_KD + PLANE16 * pl + off_a + 4096 * ks); \
            _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)                                                        \
                X_.v[nt] = *reinterpret_cast<const uint2*>(src_ + off_v + 512 * nt);                                 \
        }
#define KDA_LOAD_K(X_, C_)                                                                                          \
        {                                                                                                           \
            const unsigned char* src_ = wsh + (long long)(C_) * WS_BYTES;                                           \
            _Pragma("unroll") for (int mt = 0; mt < 2; ++mt)                                                        \
                _Pragma("unroll") for (int pl = 0; pl < 2; ++pl)                                                    \
                    _Pragma("unroll") for (int ks = 0; ks < 2; ++ks)                                                \
                        X_.k[pl][mt][ks] = *reinterpret_cast<const u32x4*>(src_ + PLANE16 * pl + off_k + 1024 * mt + 8192 * ks); \
        }
#define KDA_LOAD_E(X_, C_)                                                                                          \
        {                                                                                                           \
            const unsigned char* src_ = wsh + (long long)(C_) * WS_BYTES;                                           \
            _Pragma("unroll") for (int mt = 0; mt < 2; ++mt)                                                        \
                X_.e[mt] = *reinterpret_cast<const f32x4*>(src_ + off_e + 64 * mt);                                  \
        }
        if (nch > 0) {
            StateOperands x;
            KDA_LOAD_KD(x, 0) KDA_LOAD_K(x, 0) KDA_LOAD_E(x, 0)
            if (sub0 == 0) {                      // a request's first rows: the bound comes from the state itself
                const int e = exponent_of(wave_max_abs_bits(accS));
                if (lane == 0) mx[wave] = e;
                __syncthreads();
            }
            es = first_scale();
#pragma unroll 1
            for (int c = 0; c < nch; ++c) {
                const int c2 = min(c + 1, nch - 1);
                const u32x4 ev_after_raw = ev_request(c + 2);
                // S^T as an fp16 pair for the products of the chunk, times the chunk's scale
                {
                    const float f = pow2i(es - eu);
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt) {
                            uint2 hi, lo;
                            split_h4(scaled(accS[mt][nt], f), hi, lo);
                            uint16_t* dst = Sl + (SUB * nt + cl) * NLD128 + ((32 * wave + SUB * mt + rl) ^ piece_swap(cl));
                            *reinterpret_cast<uint2*>(dst) = hi;
                            *reinterpret_cast<uint2*>(dst + S_PLANE) = lo;
                        }
                }
                __syncthreads();
                // P = V - Kd S: wave w takes rows 16 w .. 16 w + 15. The workspace holds -Kd (scale 2^14), so the
                // accumulators start at 2^14 2^es V and end at 2^14 2^es P.
                f32x4 accP[NT];
                {
                    const float f = SC_K * pow2i(es);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        const uint2 u = x.v[nt];
                        accP[nt] = f32x4{__uint_as_float(u.x << 16) * f, __uint_as_float(u.x & 0xffff0000u) * f,
                                         __uint_as_float(u.y << 16) * f, __uint_as_float(u.y & 0xffff0000u) * f};
                    }
                }
#pragma unroll
                for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
                        accP[nt] = mfma_hl(as_u4(x.kd[0][ks]), as_u4(x.kd[1][ks]), nfrag(Sl, NLD128, SUB * nt, 32 * ks, lane),
                                           nfrag(Sl + S_PLANE, NLD128, SUB * nt, 32 * ks, lane), accP[nt]);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    uint2 hi, lo;
                    split_h4(scaled(accP[nt], 1.0f / SC_K), hi, lo);
                    uint16_t* dst = Pl + (SUB * nt + cl) * NLD64 + ((SUB * wave + rl) ^ piece_swap(cl));
                    *reinterpret_cast<uint2*>(dst) = hi;
                    *reinterpret_cast<uint2*>(dst + P_PLANE) = lo;
                }
                KDA_LOAD_KD(x, c2)
                __syncthreads();
                // while the read-out waves form V': the exponent of the largest entry of the state that entered the chunk
                // (for the next chunk's scale), and the state's decay, which also takes the accumulators to this
                // chunk's units
                {
                    const int e = exponent_of(wave_max_abs_bits(accS)) - eu;
                    if (lane == 0) mx[wave] = e;
                }
                {
                    const int eu_new = 14 + es;
                    const float f = pow2i(eu_new - eu);
                    eu = eu_new;
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                            for (int r = 0; r < 4; ++r) accS[mt][nt][r] *= x.e[mt][r] * f;
                }
                KDA_LOAD_E(x, c2)
                __syncthreads();
                // S <- e^{G_last} S + Kg^T V'
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    uint4 vh[NT], vl[NT];
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        vh[nt] = nfrag(Vl, NLD64, SUB * nt, 32 * ks, lane);
                        vl[nt] = nfrag(Vl + P_PLANE, NLD64, SUB * nt, 32 * ks, lane);
                    }
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
                            accS[mt][nt] = mfma_hl(as_u4(x.k[0][mt][ks]), as_u4(x.k[1][mt][ks]), vh[nt], vl[nt], accS[mt][nt]);
                }
                KDA_LOAD_K(x, c2)
                es = step(ev_after_raw);
                if constexpr (sizeof(S) == 2) {
                    // a bf16 state is rounded at the end of every chunk, so the result does not depend on where passes
                    // end (the power-of-two units do not change which bits are kept)
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                            for (int r = 0; r < 4; ++r) accS[mt][nt][r] = bfround(accS[mt][nt][r]);
                }
            }
            // what the next pass starts from: the term of its first chunk's scale
            if (wave == 0 && lane == 0) *carry = x_cur;
        }
#undef KDA_LOAD_KD
#undef KDA_LOAD_K
#undef KDA_LOAD_E
        {
            const float f = pow2i(-eu);
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    store_state_elem4(state_out + sbase + (long long)(NV * vb + value_col(nt, cl)) * DK + 32 * wave + SUB * mt + rl,
                                      scaled(accS[mt][nt], f));
        }
    } else {
        // rows of `out` that start on 16-byte boundaries take eight values per store
        const bool wide_out = ((reinterpret_cast<size_t>(out) | (size_t)(out_stride * 2)) & 15) == 0;
        const int nks = wave >= 2 ? 2 : 1;        // T' and M are lower triangular: rows 0..31 have nothing in columns 32..63
#define KDA_LOAD_T(X_, C_)                                                                                          \
        {                                                                                                           \
            const unsigned char* src_ = wsh + (long long)(C_) * WS_BYTES;                                           \
            _Pragma("unroll") for (int pl = 0; pl < 2; ++pl) {                                                      \
                X_.t[pl][0] = *reinterpret_cast<const u32x4*>(src_ + WS_TP + PLANE8 * pl + off_a);                  \
                if (nks == 2) X_.t[pl][1] = *reinterpret_cast<const u32x4*>(src_ + WS_TP + PLANE8 * pl + off_a + 4096); \
            }                                                                                                       \
        }
#define KDA_LOAD_Q(X_, C_)                                                                                          \
        {                                                                                                           \
            const unsigned char* src_ = wsh + (long long)(C_) * WS_BYTES;                                           \
            _Pragma("unroll") for (int pl = 0; pl < 2; ++pl)                                                        \
                _Pragma("unroll") for (int ks = 0; ks < 4; ++ks)                                                    \
                    X_.q[pl][ks] = *reinterpret_cast<const u32x4*>(src_ + WS_QG + PLANE16 * pl + off_a + 4096 * ks);  \
        }
#define KDA_LOAD_M(X_, C_)                                                                                          \
        {                                                                                                           \
            const unsigned char* src_ = wsh + (long long)(C_) * WS_BYTES;                                           \
            _Pragma("unroll") for (int pl = 0; pl < 2; ++pl) {                                                      \
                X_.m[pl][0] = *reinterpret_cast<const u32x4*>(src_ + WS_M + PLANE8 * pl + off_a);                   \
                if (nks == 2) X_.m[pl][1] = *reinterpret_cast<const u32x4*>(src_ + WS_M + PLANE8 * pl + off_a + 4096); \
            }                                                                                                       \
        }
        f32x4 accY[NT];
        int st_c = -1;                            // the chunk whose read-out is in accY, not yet stored
        float st_inv = 0.0f;                      //   and what takes its accumulators back to y: 2^-17 2^-es of that chunk
        auto store_rows = [&]() __attribute__((always_inline)) {
            const int nrows = min(CH, left - st_c * CH);
            if (SUB * wave + cl < nrows) {
                // accY[nt][r] = 2^17 2^es y[row 16 w + cl][value NV vb + 2 rl + 4 nt + r]
                const float inv = st_inv;
                bf16_t* orow = out + (rr.row0 + sub0 + st_c * CH + SUB * wave + cl) * out_stride + h * DV + NV * vb + 2 * rl;
                const u32x4 y8 = {f2bf2(accY[0][0] * inv, accY[0][1] * inv), f2bf2(accY[0][2] * inv, accY[0][3] * inv),
                                  f2bf2(accY[1][0] * inv, accY[1][1] * inv), f2bf2(accY[1][2] * inv, accY[1][3] * inv)};
                if (wide_out) *reinterpret_cast<u32x4*>(orow) = y8;
                else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        orow[2 * e] = (bf16_t)(y8[e] & 0xffffu);
                        orow[2 * e + 1] = (bf16_t)(y8[e] >> 16);
                    }
                }
            }
        };
        if (nch > 0) {
            ReadoutOperands x;
            KDA_LOAD_T(x, 0) KDA_LOAD_Q(x, 0) KDA_LOAD_M(x, 0)
            if (sub0 == 0) __syncthreads();
            es = first_scale();
#pragma unroll 1
            for (int c = 0; c < nch; ++c) {
                const int c2 = min(c + 1, nch - 1);
                const u32x4 ev_after_raw = ev_request(c + 2);
                __syncthreads();                      // the chunk's state is in LDS
                if (st_c >= 0) store_rows();
                // Y^T = S^T Qg^T + V'^T M^T, the state and V' on the row side of the tiles, so that a lane ends up with four
                // consecutive values of one row. The state's part now, while the state waves form P:
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) accY[nt] = zero;
#pragma unroll
                for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
                        accY[nt] = mfma_hl(nfrag(Sl, NLD128, SUB * nt, 32 * ks, lane), nfrag(Sl + S_PLANE, NLD128, SUB * nt, 32 * ks, lane),
                                           as_u4(x.q[0][ks]), as_u4(x.q[1][ks]), accY[nt]);
                KDA_LOAD_Q(x, c2)
                __syncthreads();                      // P is in LDS
                // V' = T' P: wave w takes rows 16 w .. 16 w + 15 (the scale of T' taken out again)
                f32x4 accV[NT];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    accV[nt] = mfma_hl(as_u4(x.t[0][0]), as_u4(x.t[1][0]), nfrag(Pl, NLD64, SUB * nt, 0, lane),
                                       nfrag(Pl + P_PLANE, NLD64, SUB * nt, 0, lane), zero);
                    if (nks == 2)
                        accV[nt] = mfma_hl(as_u4(x.t[0][1]), as_u4(x.t[1][1]), nfrag(Pl, NLD64, SUB * nt, 32, lane),
                                           nfrag(Pl + P_PLANE, NLD64, SUB * nt, 32, lane), accV[nt]);
                }
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    uint2 hi, lo;
                    split_h4(scaled(accV[nt], 1.0f / SC_T), hi, lo);
                    uint16_t* dst = Vl + (SUB * nt + cl) * NLD64 + ((SUB * wave + rl) ^ piece_swap(cl));
                    *reinterpret_cast<uint2*>(dst) = hi;
                    *reinterpret_cast<uint2*>(dst + P_PLANE) = lo;
                }
                KDA_LOAD_T(x, c2)
                __syncthreads();                      // V' is in LDS
                // the rest of Y, while the state waves update the state
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    accY[nt] = mfma_hl(nfrag(Vl, NLD64, SUB * nt, 0, lane), nfrag(Vl + P_PLANE, NLD64, SUB * nt, 0, lane),
                                       as_u4(x.m[0][0]), as_u4(x.m[1][0]), accY[nt]);
                    if (nks == 2)
                        accY[nt] = mfma_hl(nfrag(Vl, NLD64, SUB * nt, 32, lane), nfrag(Vl + P_PLANE, NLD64, SUB * nt, 32, lane),
                                           as_u4(x.m[0][1]), as_u4(x.m[1][1]), accY[nt]);
                }
                st_inv = pow2i(-17 - es);
                es = step(ev_after_raw);
                KDA_LOAD_M(x, c2)
                st_c = c;
            }
            store_rows();
        }
#undef KDA_LOAD_T
#undef KDA_LOAD_Q
#undef KDA_LOAD_M
    }
}

// The call's last launch: the conv windows' advance, and the gated RMSNorm over the bf16 read-outs the inter pass
// left in `out` (reference: kda_prefill.cu:542-570,
// cpu.rs:361-376). Sixteen lanes per (row, head), eight values per lane in 128-bit pieces when `wide` (rows of `out`
// and the gate 16-byte aligned); else a wave per (row, head), two values per lane.
__global__ void __launch_bounds__(THREADS) norm_kernel(int H, const int32_t* __restrict__ cu_rows, int rows1,
                                                       const bf16_t* __restrict__ G, long long g_stride,
                                                       const bf16_t* __restrict__ norm_w, float eps, bf16_t* out,
                                                       long long out_stride, int wide, bf16_t* conv,
                                                       const long long* __restrict__ conv_off,
                                                       const bf16_t* __restrict__ P, long long p_stride) {
    const RowRange rr = request_rows(cu_rows, blockIdx.y, rows1);
    // The request's conv window moves past all its rows, in place (reference: kda_prefill.cu:574-590): every channel
    // is one lane's, which reads its three values before it writes them. Here because this is the call's last
    // launch: every pass has read the window by now.
    {
        const int C = 3 * H * DK;
        bf16_t* win = conv + (conv_off != nullptr ? conv_off[blockIdx.y] : 0);
        for (long long c = (long long)blockIdx.x * THREADS + threadIdx.x; c < C; c += (long long)gridDim.x * THREADS) {
            bf16_t x[WINDOW];
#pragma unroll
            for (int j = 0; j < WINDOW; ++j) {
                const long long src = (long long)rr.rows + j;
                x[j] = src < WINDOW ? win[src * C + c] : P[(rr.row0 + src - WINDOW) * p_stride + c];
            }
#pragma unroll
            for (int j = 0; j < WINDOW; ++j) win[(long long)j * C + c] = x[j];
        }
    }
    const long long tasks = (long long)rr.rows * H;
    const int lane = threadIdx.x & 63;
    if (wide) {
        const int sub = lane & 15;                                   // this lane's eight values: 8 sub .. 8 sub + 7
        const u32x4 wv = *reinterpret_cast<const u32x4*>(norm_w + 8 * sub);
        const int per_block = THREADS / 16;
        for (long long task = (long long)blockIdx.x * per_block + (threadIdx.x >> 4); task < tasks;
             task += (long long)gridDim.x * per_block) {
            const long long r = rr.row0 + task / H;
            const int h = (int)(task % H);
            u32x4* o = reinterpret_cast<u32x4*>(out + r * out_stride + h * DV + 8 * sub);
            const u32x4 yy = *o;
            const u32x4 gg = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(G + r * g_stride + h * DV + 8 * sub));
            float y[8], ss = 0.0f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                y[2 * e] = __uint_as_float(yy[e] << 16);
                y[2 * e + 1] = __uint_as_float(yy[e] & 0xffff0000u);
                ss = __builtin_fmaf(y[2 * e], y[2 * e], ss);
                ss = __builtin_fmaf(y[2 * e + 1], y[2 * e + 1], ss);
            }
            ss = ss + lane_xor16<1>(ss);
            ss = ss + lane_xor16<2>(ss);
            ss = ss + lane_xor16<4>(ss);
            ss = ss + lane_xor16<8>(ss);
            const float rinv = __builtin_amdgcn_rsqf(ss * (1.0f / (float)DV) + eps);
            u32x4 res;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float g0 = __uint_as_float(gg[e] << 16), g1 = __uint_as_float(gg[e] & 0xffff0000u);
                const float w0 = __uint_as_float(wv[e] << 16), w1 = __uint_as_float(wv[e] & 0xffff0000u);
                res[e] = f2bf2(w0 * (y[2 * e] * rinv) * fast_sigmoid(g0), w1 * (y[2 * e + 1] * rinv) * fast_sigmoid(g1));
            }
            *o = res;
        }
        return;
    }
    const int wpb = THREADS / 64;
    const uint32_t wpair = reinterpret_cast<const uint32_t*>(norm_w)[lane];
    const float w0 = __uint_as_float(wpair << 16), w1 = __uint_as_float(wpair & 0xffff0000u);
    for (long long task = (long long)blockIdx.x * wpb + (threadIdx.x >> 6); task < tasks;
         task += (long long)gridDim.x * wpb) {
        const long long r = rr.row0 + task / H;
        const int h = (int)(task % H);
        uint32_t* o = reinterpret_cast<uint32_t*>(out + r * out_stride + h * DV);
        const uint32_t yy = o[lane];
        const uint32_t gg = reinterpret_cast<const uint32_t*>(G + r * g_stride + h * DV)[lane];
        const float y0 = __uint_as_float(yy << 16), y1 = __uint_as_float(yy & 0xffff0000u);
        float ss = __builtin_fmaf(y1, y1, y0 * y0);
        ss = ss + lane_xor16<1>(ss);
        ss = ss + lane_xor16<2>(ss);
        ss = ss + lane_xor16<4>(ss);
        ss = ss + lane_xor16<8>(ss);
        ss = ss + __shfl_xor(ss, 16, 64);
        ss = ss + __shfl_xor(ss, 32, 64);
        const float rinv = __builtin_amdgcn_rsqf(ss * (1.0f / (float)DV) + eps);
        const float g0 = __uint_as_float(gg << 16), g1 = __uint_as_float(gg & 0xffff0000u);
        o[lane] = f2bf2(w0 * (y0 * rinv) * fast_sigmoid(g0), w1 * (y1 * rinv) * fast_sigmoid(g1));
    }
}

inline const bf16_t* bfp(const glm53f_bf16* x) { return reinterpret_cast<const bf16_t*>(x); }
inline bf16_t* bfp(glm53f_bf16* x) { return reinterpret_cast<bf16_t*>(x); }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr int kNormBlocks = 1024;


// More than 64 KiB of LDS per workgroup is an attribute of each device's copy of a kernel: set once per device, under
// a lock (two host threads may make their first calls together). The first call on a device therefore does more
// than launch kernels and should come before a stream capture.
int allow_large_lds() {
    constexpr int kMaxDevices = 64;
    static std::mutex lock;
    static bool done_on[kMaxDevices] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(lock);
    if (done_on[dev]) return 0;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&intra_kernel<true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, INTRA_LDS) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&intra_kernel<false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, INTRA_LDS) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&inter_kernel<float>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, INTER_LDS) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(&inter_kernel<bf16_t>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, INTER_LDS) != hipSuccess)
        return (int)hipGetLastError();
    done_on[dev] = true;
    return 0;
}

// The passes over every sub-segment, the norm and the conv-window advance, in stream order (reference:
// kda_prefill.cu:630-691).
template <typename S>
int launch(int32_t heads, int32_t batch, const int32_t* cu_rows, int32_t rows1, int32_t max_rows, const glm53f_bf16* p,
           int64_t p_stride, int64_t b_off, const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g,
           int64_t g_stride, glm53f_bf16* conv, const int64_t* conv_off, const glm53f_bf16* conv_w, const S* state_in,
           S* state_out, const int64_t* state_off, const float* a_log, const float* dt_bias,
           const glm53f_bf16* norm_w, float eps, float lower, glm53f_bf16* out, int64_t out_stride,
           int32_t value_blocks, float* workspace, int64_t workspace_bytes, glm53f_stream_t stream) {
    if (heads < 1 || heads > 65535 || batch < 1 || batch > 65535 || rows1 < 0 || max_rows < 0 || !p || !a || !g ||
        !conv || !conv_w || !state_in || !state_out || !a_log || !dt_bias || !norm_w || !out || !workspace)
        return kInvalid;
    // Fifteen rows of decay must stay above the smallest normal f32 in a sub-chunk's products.
    if (!(lower >= -5.8f && lower <= 0.0f)) return kInvalid;
    if (value_blocks != 0 && value_blocks != 1 && value_blocks != 2 && value_blocks != 4) return kInvalid;
    // 128-bit accesses to the workspace and the states, 64-bit to the conv weights, 32-bit to g and out rows.
    if (!aligned16(workspace) || !aligned16(state_in) || !aligned16(state_out)) return kInvalid;
    if ((reinterpret_cast<uintptr_t>(conv_w) & 7u) || (reinterpret_cast<uintptr_t>(out) & 3u) ||
        (reinterpret_cast<uintptr_t>(g) & 3u) || (out_stride & 1) || (g_stride & 1))
        return kInvalid;
    (void)value_blocks;   // checked as the reference checks it; this build always uses 32-column blocks
    const long long per_chunk = (long long)WS_BYTES * heads * batch;
    long long chunks = workspace_bytes / per_chunk;
    if (chunks < 1) return kInvalid;
    const long long needed = ((long long)max_rows + CH - 1) / CH;
    if (chunks > needed) chunks = needed > 0 ? needed : 1;
    if (chunks > 65535) chunks = 65535;
    // A pass's workspace is written by one launch and read by the next. While it fits the 256 MB cache behind the
    // L2 the second launch reads it from there: the 2048-row lane of 64 heads in one pass (303 MB) measured
    // 286 us, in two passes of 1024 rows 232 us. So the rows are cut into equal passes (whole pairs of chunks: an
    // intra workgroup takes two) that stay under kPassBytes, but not below kMinPassChunks chunks (short passes
    // leave the serial launch too little to hide its start behind).
    {
        constexpr long long kPassBytes = 160LL << 20, kMinPassChunks = 16;
        const long long fit = kPassBytes / per_chunk;
        const long long cap = fit > kMinPassChunks ? fit : kMinPassChunks;
        if (chunks > cap) {
            const long long total = needed > 0 ? needed : 1;
            const long long passes = (total + cap - 1) / cap;
            long long even = (total + passes - 1) / passes;
            even = (even + INTRA_CPW - 1) / INTRA_CPW * INTRA_CPW;
            chunks = even < chunks ? even : chunks;
        }
    }
    hipStream_t st = (hipStream_t)stream;
    const int arc = allow_large_lds();
    if (arc != 0) return arc;
    const long long* coff = reinterpret_cast<const long long*>(conv_off);
    const long long* soff = reinterpret_cast<const long long*>(state_off);
    unsigned char* ws = reinterpret_cast<unsigned char*>(workspace);
    // 128-bit input staging needs every q | k | v and gate row segment on a 16-byte boundary (the model's strides
    // are); other layouts take the 16-bit path. Conv-window offsets are device data: whole windows keep alignment.
    const int vec = aligned16(p) && aligned16(a) && aligned16(conv) && (p_stride % 8 == 0) && (a_stride % 8 == 0);
    const long long step = chunks * CH;
    for (long long sub0 = 0; sub0 == 0 || sub0 < max_rows; sub0 += step) {
        if (max_rows > 0) {
            const dim3 grid((unsigned)((chunks + INTRA_CPW - 1) / INTRA_CPW), heads, batch);
            if (vec)
                intra_kernel<true><<<grid, THREADS, INTRA_LDS, st>>>(heads, cu_rows, rows1, (int)sub0, (int)chunks, bfp(p),
                                                                     p_stride, b_off, bfp(a), a_stride, bfp(conv), coff,
                                                                     bfp(conv_w), a_log, dt_bias, lower, ws);
            else
                intra_kernel<false><<<grid, THREADS, INTRA_LDS, st>>>(heads, cu_rows, rows1, (int)sub0, (int)chunks, bfp(p),
                                                                      p_stride, b_off, bfp(a), a_stride, bfp(conv), coff,
                                                                      bfp(conv_w), a_log, dt_bias, lower, ws);
            const int rc = (int)hipGetLastError();
            if (rc != 0) return rc;
        }
        const S* s_in = sub0 == 0 ? state_in : state_out;
        inter_kernel<S><<<dim3(heads * VBLOCKS, batch), INTER_THREADS, INTER_LDS, st>>>(
            heads, cu_rows, rows1, (int)sub0, (int)chunks, s_in, state_out, soff, bfp(out), out_stride, ws, ws);
        const int rc = (int)hipGetLastError();
        if (rc != 0) return rc;
        if (max_rows == 0) break;
    }
    if (max_rows > 0) {
        const int wide = aligned16(out) && aligned16(g) && aligned16(norm_w) && out_stride % 8 == 0 && g_stride % 8 == 0;
        norm_kernel<<<dim3(kNormBlocks, batch), THREADS, 0, st>>>(heads, cu_rows, rows1, bfp(g), g_stride, bfp(norm_w),
                                                                  eps, bfp(out), out_stride, wide, bfp(conv), coff,
                                                                  bfp(p), p_stride);
        return (int)hipGetLastError();
    }
    return 0;                                     // no request has rows: the windows stay as they are
}

}  // namespace
}  // namespace kda

using namespace kda;

extern "C" int glm53f_kda_init(void) { return allow_large_lds(); }

extern "C" int64_t glm53f_kda_prefill_workspace_bytes(int32_t heads, int32_t batch, int32_t rows_per_pass) {
    if (heads < 1 || batch < 1 || rows_per_pass < 1) return 0;
    return (((int64_t)rows_per_pass + CH - 1) / CH) * WS_BYTES * (int64_t)heads * batch;
}

extern "C" int glm53f_kda_prefill(int32_t heads, int32_t rows, const glm53f_bf16* p, int64_t p_stride, int64_t b_off,
                                  const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g, int64_t g_stride,
                                  glm53f_bf16* conv, const glm53f_bf16* conv_w, const float* state_in,
                                  float* state_out, const float* a_log, const float* dt_bias,
                                  const glm53f_bf16* norm_w, float eps, float lower, glm53f_bf16* out,
                                  int64_t out_stride, int32_t value_blocks, float* workspace,
                                  int64_t workspace_bytes, glm53f_stream_t stream) {
    return launch<float>(heads, 1, nullptr, rows, rows, p, p_stride, b_off, a, a_stride, g, g_stride, conv, nullptr,
                         conv_w, state_in, state_out, nullptr, a_log, dt_bias, norm_w, eps, lower, out, out_stride,
                         value_blocks, workspace, workspace_bytes, stream);
}

extern "C" int glm53f_kda_prefill_batch(int32_t heads, int32_t batch, const int32_t* cu_rows, int32_t max_rows,
                                        const glm53f_bf16* p, int64_t p_stride, int64_t b_off, const glm53f_bf16* a,
                                        int64_t a_stride, const glm53f_bf16* g, int64_t g_stride, glm53f_bf16* conv,
                                        const int64_t* conv_off, const glm53f_bf16* conv_w, const float* state_in,
                                        float* state_out, const int64_t* state_off, const float* a_log,
                                        const float* dt_bias, const glm53f_bf16* norm_w, float eps, float lower,
                                        glm53f_bf16* out, int64_t out_stride, int32_t value_blocks, float* workspace,
                                        int64_t workspace_bytes, glm53f_stream_t stream) {
    if (!cu_rows || !conv_off || !state_off) return kInvalid;
    return launch<float>(heads, batch, cu_rows, 0, max_rows, p, p_stride, b_off, a, a_stride, g, g_stride, conv,
                         conv_off, conv_w, state_in, state_out, state_off, a_log, dt_bias, norm_w, eps, lower, out,
                         out_stride, value_blocks, workspace, workspace_bytes, stream);
}

extern "C" int glm53f_kda_prefill_batch_bf16state(int32_t heads, int32_t batch, const int32_t* cu_rows,
                                                  int32_t max_rows, const glm53f_bf16* p, int64_t p_stride,
                                                  int64_t b_off, const glm53f_bf16* a, int64_t a_stride,
                                                  const glm53f_bf16* g, int64_t g_stride, glm53f_bf16* conv,
                                                  const int64_t* conv_off, const glm53f_bf16* conv_w,
                                                  const glm53f_bf16* state_in, glm53f_bf16* state_out,
                                                  const int64_t* state_off, const float* a_log,
                                                  const float* dt_bias, const glm53f_bf16* norm_w, float eps,
                                                  float lower, glm53f_bf16* out, int64_t out_stride,
                                                  int32_t value_blocks, float* workspace, int64_t workspace_bytes,
                                                  glm53f_stream_t stream) {
    if (!cu_rows || !conv_off || !state_off) return kInvalid;
    return launch<bf16_t>(heads, batch, cu_rows, 0, max_rows, p, p_stride, b_off, a, a_stride, g, g_stride, conv,
                          conv_off, conv_w, bfp(state_in), bfp(state_out), state_off, a_log, dt_bias, norm_w, eps,
                          lower, out, out_stride, value_blocks, workspace, workspace_bytes, stream);
}
