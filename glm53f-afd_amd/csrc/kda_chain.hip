// KDA recurrent path on gfx950: the decode / verify chain, the replays, the conv-window shift and the
// checkpoint selection. One workgroup of 256 lanes (4 waves) per (head, request). The per-row arithmetic
// follows the reference's CPU model operation for operation (crates/glm53f-kda/src/cpu.rs:410-471); what is
// new is the mapping: every lane streams 128-bit pieces of the state (a value row per 16 or 32 lanes),
// keeps 64 state values in registers across the rows of a window, and sums over keys inside its wave.
//
// Compiled with floating-point contraction off: the state update must not fuse a multiply and an add, so
// that chain, replay and verify give the same bits (and those of the CPU model).

#include "kda_common.h"

namespace kda {
namespace {

constexpr int THREADS = 256;

// State access: a uniform base (bumped per step by a constant, scalar arithmetic) plus one 32-bit lane offset,
// so no per-step 64-bit lane addresses are kept alive.
template <typename S>
__device__ __forceinline__ unsigned lane_offset(int wave, int lane) {
    using M = StateMap<S>;
    return (unsigned)(M::row(0, wave, lane) * DK + M::key0(lane));
}

template <typename S>
__device__ __forceinline__ void load_state(const S* base, unsigned off, uint4 (&raw)[StateMap<S>::STEPS]) {
    using M = StateMap<S>;
#pragma unroll
    for (int j = 0; j < M::STEPS; ++j) raw[j] = ld128((base + j * M::RPS * DK) + off);
}

template <typename S>
__device__ __forceinline__ void store_raw(S* base, unsigned off, const uint4 (&raw)[StateMap<S>::STEPS]) {
    using M = StateMap<S>;
#pragma unroll
    for (int j = 0; j < M::STEPS; ++j) st128((base + j * M::RPS * DK) + off, raw[j]);
}

// The chain: conv + SiLU, gates, L2 norms, delta rule, read-out, gated RMSNorm, row after row
// (reference: kda.cu:98-210, cpu.rs:410-471). The state pointers are not __restrict__: a chain may run in
// place; each lane reads its 64 values before the first row and writes the same 64 after the last.
// ckpt (bf16 states only): the state after every row, global row r at ckpt + r * H * 16384.
template <typename S>
__global__ void __launch_bounds__(THREADS, 4) chain_kernel(
        int H, const int32_t* __restrict__ cu_rows, int rows1,
        const bf16_t* __restrict__ P, long long p_stride, long long b_off,
        const bf16_t* __restrict__ A, long long a_stride, const bf16_t* __restrict__ G, long long g_stride,
        const bf16_t* conv, const long long* __restrict__ conv_off, const bf16_t* __restrict__ cw,
        const S* state_in, S* state_out, const long long* __restrict__ state_off,
        const float* __restrict__ a_log, const float* __restrict__ dt_bias, const bf16_t* __restrict__ norm_w,
        float eps, float lower, bf16_t* __restrict__ out, long long out_stride, S* __restrict__ ckpt,
        float* __restrict__ k_save, bf16_t* __restrict__ v_save, float* __restrict__ g_save,
        float* __restrict__ b_save, int shift) {
    using M = StateMap<S>;
    constexpr int KPL = M::KPL;
    const long long C = 3LL * H * DK;
    const int h = blockIdx.x, b = blockIdx.y;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
    const RowRange rr = request_rows(cu_rows, b, rows1);
    const int rows = rr.rows;
    const bf16_t* cs = conv + (conv_off != nullptr ? conv_off[b] : 0);
    const long long sbase = (state_off != nullptr ? state_off[b] : 0) + (long long)h * DV * DK;

    __shared__ float qs[DK], ks[DK], vs[DV], gs[DK], ys[DV];
    __shared__ float beta_s, rinv_s;

    const unsigned soff_lane = lane_offset<S>(wave, lane);
    const int key0 = M::key0(lane);
    if (rows <= 0) {
        // A request without rows: its state is copied (with loads of its own, so that this path shares no
        // registers with the main one).
        if (state_out != nullptr && state_out != state_in) {
            uint4 cp[M::STEPS];
            load_state<S>(state_in + sbase, soff_lane, cp);
            store_raw<S>(state_out + sbase, soff_lane, cp);
        }
        return;
    }
    const float decay_rate = expf(a_log[h]);

    // Inputs reach the workgroup as 128-bit pieces, one per lane, staged in LDS: per-lane 16-bit loads would take
    // seventeen memory instructions per lane and row, and sixteen waves a CU issuing those keep its address
    // pipeline busy for microseconds before the state's loads can even start.
    //   weights, once: conv weights of the head's 384 channels (pieces 0..191), dt_bias (192..223), norm weight
    //   (224..239);  a row: its four conv taps of q | k | v (pieces 0..191, tap-major), its forget-gate inputs
    //   (192..207) and output-gate logits (208..223). Piece i lands at byte 16 i of its staging array.
    __shared__ __align__(16) unsigned char w_stage[240 * 16];
    __shared__ __align__(16) unsigned char x_stage[224 * 16];
    const bf16_t* xs = reinterpret_cast<const bf16_t*>(x_stage);              // [4 taps][q | k | v][128]
    const bf16_t* a_sh = xs + TAPS * 3 * DK;                                  // [128]
    const bf16_t* gate_sh = a_sh + DK;                                        // [128]
    // 16 bytes from an address with 2-byte alignment or better
    auto load_piece = [](const void* p) -> u32x4_t {
        if ((reinterpret_cast<uintptr_t>(p) & 15u) == 0) return *reinterpret_cast<const u32x4_t*>(p);
        const uint16_t* q = reinterpret_cast<const uint16_t*>(p);
        u32x4_t v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (uint32_t)q[2 * e] | ((uint32_t)q[2 * e + 1] << 16);
        return v;
    };
    auto weight_piece = [&]() -> u32x4_t {
        const int i = min(t, 239);
        const void* p;
        if (i < 192) p = cw + ((size_t)(i >> 6) * H * DK + (size_t)h * DK) * TAPS + (i & 63) * 8;
        else if (i < 224) p = dt_bias + h * DK + (i - 192) * 4;
        else p = norm_w + (i - 224) * 8;
        return load_piece(p);
    };
    auto row_piece = [&](int r) -> u32x4_t {
        const long long gr = rr.row0 + r;
        const int i = min(t, 223);
        const bf16_t* p;
        if (i < 192) {
            const int j = i / 48, rem = i - 48 * j, at = r + j;
            const bf16_t* row = at < WINDOW ? cs + (long long)at * C : P + (rr.row0 + at - WINDOW) * p_stride;
            p = row + (long long)(rem >> 4) * H * DK + h * DK + (rem & 15) * 8;
        } else if (i < 208) {
            p = A + gr * a_stride + h * DK + (i - 192) * 8;
        } else {
            p = G + gr * g_stride + h * DV + (i - 208) * 8;
        }
        return load_piece(p);
    };
    auto beta_logit = [&](int r) -> bf16_t { return *uniform_ptr(P + (rr.row0 + r) * p_stride + b_off + h); };

    // The first row's inputs and the weights are requested before the state (the scheduling barriers keep that
    // order), so the prologue waits for them alone and runs while the state streams in. Between rows the state
    // stays in its stored form (`raw`: packed bf16 pairs, or f32 bits): a bf16 state is rounded after every row
    // anyway, and the packed form halves the registers it holds. With a bf16 state there are registers to spare and
    // the next row's piece is requested before this row's update; an f32 state requests it after the epilogue.
    constexpr bool kPrefetch = M::kRound;
    const int i7 = t & (DK - 1);
    uint4 raw[M::STEPS];
    u32x4_t xpiece = row_piece(0);
    bf16_t b_raw = beta_logit(0);
    {
        const u32x4_t wpiece = weight_piece();
        __builtin_amdgcn_sched_barrier(0);
        load_state<S>(state_in + sbase, soff_lane, raw);
        __builtin_amdgcn_sched_barrier(0);
        if (t < 240) *reinterpret_cast<u32x4_t*>(w_stage + t * 16) = wpiece;
    }
    __syncthreads();
    // This lane's weights: conv channel t of q | k, v channel t % 128, the forget-gate bias of key t % 128 and the
    // norm weight of value t % 128. They stay staged for all rows; with a bf16 state there are registers to keep
    // them in, an f32 state reads them again for every row.
    struct LaneWeights {
        uint2 w0, w1;
        float dtb, normw;
    };
    auto lane_weights = [&]() -> LaneWeights {
        return {*reinterpret_cast<const uint2*>(w_stage + t * 8), *reinterpret_cast<const uint2*>(w_stage + (2 * DK + i7) * 8),
                *reinterpret_cast<const float*>(w_stage + 192 * 16 + i7 * 4),
                bf2f(*reinterpret_cast<const bf16_t*>(w_stage + 224 * 16 + i7 * 2))};
    };
    LaneWeights kept = {};
    if constexpr (kPrefetch) kept = lane_weights();
    float gate_r = 0.0f, normw_r = 0.0f;                                      // the epilogue's operands

    // A row's prologue from its staged piece: conv + SiLU, gates, L2 norms.
    auto prologue = [&]() {
        if (t < 224) *reinterpret_cast<u32x4_t*>(x_stage + t * 16) = xpiece;
        __syncthreads();
        bf16_t x0[TAPS], x1[TAPS];
#pragma unroll
        for (int tap = 0; tap < TAPS; ++tap) {
            x0[tap] = xs[tap * 3 * DK + t];                 // q channel t, or k channel t - 128
            x1[tap] = xs[tap * 3 * DK + 2 * DK + i7];
        }
        const bf16_t a_raw = a_sh[i7];
        gate_r = bf2f(gate_sh[i7]);
        const LaneWeights lw = kPrefetch ? kept : lane_weights();
        const uint2 w0 = lw.w0, w1 = lw.w1;
        const float dtb = lw.dtb;
        normw_r = lw.normw;
        // conv + SiLU, one bf16 rounding (cpu.rs:257-281)
        auto conv1 = [&](const uint2 w4, const bf16_t (&x)[TAPS]) -> float {
            const float wt[TAPS] = {__uint_as_float(w4.x << 16), __uint_as_float(w4.x & 0xffff0000u),
                                    __uint_as_float(w4.y << 16), __uint_as_float(w4.y & 0xffff0000u)};
            float acc = 0.0f;
#pragma unroll
            for (int tap = 0; tap < TAPS; ++tap) acc = acc + wt[tap] * bf2f(x[tap]);
            return bfround(acc / (1.0f + expf(-acc)));
        };
        const float act0 = conv1(w0, x0);
        if (t < DK) qs[i7] = act0; else ks[i7] = act0;
        if (t < DK) {
            vs[i7] = conv1(w1, x1);
        } else {
            gs[i7] = expf(lower * sigmoidf_(decay_rate * (bf2f(a_raw) + dtb)));   // cpu.rs:247-249
        }
        if (t == THREADS - 1) beta_s = bfround(sigmoidf_(bf2f(b_raw)));
        __syncthreads();
        if (wave == 0) {
            float* x = lane < 32 ? qs : ks;    // L2 norms (cpu.rs:305-315): lanes 0..31 take q, lanes 32..63 take k
            const int l32 = lane & 31;
            float v4[4];
            const float ss = sumsq128(x, l32, v4);
            const float inv = 1.0f / sqrtf(ss + 1e-6f);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float y = v4[i] * inv;
                if (lane < 32) y = y * (1.0f / sqrtf((float)DK));
                x[l32 * 4 + i] = y;
            }
        }
        __syncthreads();
    };

    int r = 0;
    do {   // rows >= 1 here; a do-while leaves no zero-trip path that would keep the loaded state alive
        const long long gr = rr.row0 + r;
        prologue();
        // shift: the request's conv window moves past all its rows, in place (what conv_shift_kernel does with
        // keep = rows, reference kda.cu:258-277). The new window is taps 1..3 of the last row, staged in LDS as
        // pieces 48..191; this workgroup is the only one that reads or writes its head's channels, and its last
        // read of the window (this row's piece) landed before the prologue. Stored here, ahead of the update, the
        // writes drain while the state is worked on.
        if (shift && r + 1 == rows && t >= 48 && t < 192) {
            const int j = t / 48, rem = t - 48 * j;
            bf16_t* dst = const_cast<bf16_t*>(cs) + (long long)(j - 1) * C + (long long)(rem >> 4) * H * DK + h * DK +
                          (rem & 15) * 8;
            const u32x4_t v = *reinterpret_cast<const u32x4_t*>(x_stage + t * 16);
            if ((reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
                // nontemporal: lines left dirty in the L2 would be written back at the end of the kernel, on its
                // critical path
                __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>(dst));
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    dst[2 * e] = (bf16_t)(v[e] & 0xffffu);
                    dst[2 * e + 1] = (bf16_t)(v[e] >> 16);
                }
            }
        }
        if constexpr (kPrefetch) {
            if (r + 1 < rows) {
                xpiece = row_piece(r + 1);
                b_raw = beta_logit(r + 1);
            }
        }
        const float beta = beta_s;
        // Stores leave as soon as a step's 16 or 8 value rows are final, so they overlap the remaining steps
        // and the row's epilogue: the checkpoint of every row, and the state itself in the last row.
        S* const ck_row = ckpt != nullptr ? uniform_ptr(ckpt + (gr * H + h) * (long long)(DV * DK)) : nullptr;
        S* const st_row = (state_out != nullptr && r + 1 == rows) ? uniform_ptr(state_out + sbase) : nullptr;
        float kk[KPL], qq[KPL], gg[KPL];
#pragma unroll
        for (int c = 0; c < KPL; ++c) {
            kk[c] = ks[key0 + c];
            qq[c] = qs[key0 + c];
            gg[c] = gs[key0 + c];
        }
#pragma unroll
        for (int j = 0; j < M::STEPS; ++j) {
            const int row = M::row(j, wave, lane);
            float s[KPL];
            unpack<S>(raw[j], s);
            update_row<S>(s, kk, gg, vs[row], beta);
            const float o = read_row<S>(s, qq);
            if (lane % M::LPR == 0) ys[row] = bfround(o);
            raw[j] = pack<S>(s);        // rounds a bf16 state (after the row's read-out)
            if constexpr (M::kRound) {
                // a bf16 state has registers to spare for the eight offsets: 32 bits on top of a scalar base
                const unsigned off_j = soff_lane + (unsigned)(j * M::RPS * DK);
                if (ck_row != nullptr) st128(ck_row + off_j, raw[j]);
                if (st_row != nullptr) st128(st_row + off_j, raw[j]);
            } else {
                if (ck_row != nullptr) st128((ck_row + j * M::RPS * DK) + soff_lane, raw[j]);
                if (st_row != nullptr) st128((st_row + j * M::RPS * DK) + soff_lane, raw[j]);
            }
        }
        if (k_save != nullptr) {
            const long long base = (gr * H + h) * DK;
            if (t < DK) {
                uniform_ptr(k_save + base)[(unsigned)t] = ks[t];
                uniform_ptr(g_save + base)[(unsigned)t] = gs[t];
            } else {
                uniform_ptr(v_save + base)[(unsigned)(t - DK)] = f2bf(vs[t - DK]);
            }
            if (t == 0) b_save[gr * H + h] = beta;
        }
        __syncthreads();
        // Gated RMSNorm (cpu.rs:361-376).
        if (wave == 0 && lane < 32) {
            float v4[4];
            const float ss = sumsq128(ys, lane, v4);
            if (lane == 0) rinv_s = 1.0f / sqrtf(ss / (float)DV + eps);
        }
        __syncthreads();
        if (t < DV) {
            const float yn = ys[t] * rinv_s;
            const float yw = normw_r * yn;
            uniform_ptr(out + gr * out_stride + h * DV)[(unsigned)t] = f2bf(yw * sigmoidf_(gate_r));
        }
        __syncthreads();
        if constexpr (!kPrefetch) {
            if (r + 1 < rows) {
                xpiece = row_piece(r + 1);
                b_raw = beta_logit(r + 1);
            }
        }
    } while (++r < rows);
}

// Replay of saved rows (reference: kda.cu:214-253, cpu.rs:486-508): workgroup (layer * H + h, b). Waves are
// independent here: every lane reads its own keys' k and exp(g) and its rows' v straight from the saves.
template <typename S>
__global__ void __launch_bounds__(THREADS, 4) replay_kernel(
        int H, const int32_t* __restrict__ cu_rows, const int32_t* __restrict__ keep, int rows1,
        const S* state_in, S* state_out, long long state_stride, const long long* __restrict__ state_off,
        const float* __restrict__ k_save, const bf16_t* __restrict__ v_save, const float* __restrict__ g_save,
        const float* __restrict__ b_save, long long kv_stride, long long b_stride) {
    using M = StateMap<S>;
    constexpr int KPL = M::KPL;
    const int layer = blockIdx.x / H, h = blockIdx.x % H, b = blockIdx.y;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
    const long long row0 = cu_rows != nullptr ? cu_rows[b] : 0;
    const int rows = keep != nullptr ? keep[b] : rows1;
    const long long sbase = (long long)layer * state_stride + (state_off != nullptr ? state_off[b] : 0) +
                            (long long)h * DV * DK;
    const float* ksv = k_save + layer * kv_stride;
    const bf16_t* vsv = v_save + layer * kv_stride;
    const float* gsv = g_save + layer * kv_stride;
    const float* bsv = b_save + layer * b_stride;
    const int key0 = M::key0(lane);
    const unsigned soff_lane = lane_offset<S>(wave, lane);
    const unsigned row_lane = (unsigned)M::row(0, wave, lane);

    uint4 raw[M::STEPS];
    load_state<S>(state_in + sbase, soff_lane, raw);
    for (int r = 0; r < rows; ++r) {
        const long long gr = row0 + r;
        const long long base = (gr * H + h) * DK;
        float kk[KPL], gg[KPL];
#pragma unroll
        for (int c = 0; c < KPL; c += 4) {
            const float4 k4 = *reinterpret_cast<const float4*>((ksv + base) + (unsigned)(key0 + c));
            const float4 g4 = *reinterpret_cast<const float4*>((gsv + base) + (unsigned)(key0 + c));
            kk[c] = k4.x; kk[c + 1] = k4.y; kk[c + 2] = k4.z; kk[c + 3] = k4.w;
            gg[c] = g4.x; gg[c + 1] = g4.y; gg[c + 2] = g4.z; gg[c + 3] = g4.w;
        }
        const float beta = bsv[gr * H + h];
#pragma unroll
        for (int j = 0; j < M::STEPS; ++j) {
            float s[KPL];
            unpack<S>(raw[j], s);
            update_row<S>(s, kk, gg, bf2f((vsv + base + j * M::RPS)[row_lane]), beta);
            raw[j] = pack<S>(s);
        }
    }
    store_raw<S>(state_out + sbase, soff_lane, raw);
}

// Conv-window shift (reference: kda.cu:258-277, cpu.rs:512-527): lane (channel, layer, request) reads its
// three values before writing them, so the shift runs in place.
__global__ void conv_shift_kernel(int C, const int32_t* __restrict__ cu_rows, const int32_t* __restrict__ keep,
                                  int keep1, bf16_t* conv, long long conv_stride,
                                  const long long* __restrict__ conv_off, const bf16_t* P,
                                  long long p_layer_stride, long long p_stride) {
    const int layer = blockIdx.y, b = blockIdx.z;
    const long long row0 = cu_rows != nullptr ? cu_rows[b] : 0;
    const int k = keep != nullptr ? keep[b] : keep1;
    bf16_t* win = conv + (long long)layer * conv_stride + (conv_off != nullptr ? conv_off[b] : 0);
    const bf16_t* rows = P + (long long)layer * p_layer_stride + row0 * p_stride;
    // Eight channels per lane in 128-bit pieces when every row involved is 16-byte aligned (uniform over the
    // workgroup), else one channel per lane; the grid covers C channels either way (see the launcher).
    const bool wide = (C % 8 == 0) && (p_stride % 8 == 0) &&
                      ((reinterpret_cast<uintptr_t>(win) | reinterpret_cast<uintptr_t>(rows)) & 15u) == 0;
    if (wide) {
        const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
        if (c >= C) return;
        uint4 v[WINDOW];
#pragma unroll
        for (int j = 0; j < WINDOW; ++j) {
            const long long src = (long long)k + j;
            v[j] = ld128(src < WINDOW ? win + src * C + c : rows + (src - WINDOW) * p_stride + c);
        }
#pragma unroll
        for (int j = 0; j < WINDOW; ++j) st128(win + (long long)j * C + c, v[j]);
        return;
    }
    for (int c = blockIdx.x * blockDim.x * 8 + threadIdx.x; c < min(C, (int)(blockIdx.x + 1) * (int)blockDim.x * 8);
         c += blockDim.x) {
        bf16_t v[WINDOW];
#pragma unroll
        for (int j = 0; j < WINDOW; ++j) {
            const long long src = (long long)k + j;
            v[j] = src < WINDOW ? win[src * C + c] : rows[(src - WINDOW) * p_stride + c];
        }
#pragma unroll
        for (int j = 0; j < WINDOW; ++j) win[(long long)j * C + c] = v[j];
    }
}

// Commit by selection: workgroup (layer * H + h, b) copies one head of the checkpoint after row keep[b] - 1.
__global__ void __launch_bounds__(THREADS) select_kernel(
        int H, const int32_t* __restrict__ cu_rows, const int32_t* __restrict__ keep,
        const bf16_t* __restrict__ ckpt, long long ckpt_layer_stride, bf16_t* __restrict__ state,
        long long state_stride, const long long* __restrict__ state_off) {
    const int layer = blockIdx.x / H, h = blockIdx.x % H, b = blockIdx.y;
    const int k = keep[b];
    if (k <= 0) return;
    const long long gr = (long long)cu_rows[b] + k - 1;
    const bf16_t* src = ckpt + (long long)layer * ckpt_layer_stride + (gr * H + h) * (long long)(DV * DK);
    bf16_t* dst = state + (long long)layer * state_stride + state_off[b] + (long long)h * DV * DK;
    uint4 v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = ld128(src + (i * THREADS + threadIdx.x) * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) st128(dst + (i * THREADS + threadIdx.x) * 8, v[i]);
}

inline int launched() { return (int)hipGetLastError(); }

// States, checkpoints and saves move in 128-bit pieces: their base pointers must be 16-byte aligned (and the
// device-side offsets multiples of 8 elements, which whole heads always are).
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline const bf16_t* bfp(const glm53f_bf16* x) { return reinterpret_cast<const bf16_t*>(x); }
inline bf16_t* bfp(glm53f_bf16* x) { return reinterpret_cast<bf16_t*>(x); }

// Host-side checks shared by the chain entry points (reference: kda.cu:290-299).
inline bool chain_args_ok(int32_t heads, const void* p, const void* a, const void* g, const void* conv,
                          const void* conv_w, const void* state_in, const void* a_log, const void* dt_bias,
                          const void* norm_w, const void* out, const void* k_save, const void* v_save,
                          const void* g_save, const void* b_save) {
    if (heads < 1 || heads > 65535) return false;
    if (!p || !a || !g || !conv || !conv_w || !state_in || !a_log || !dt_bias || !norm_w || !out) return false;
    const int saves = (k_save != nullptr) + (v_save != nullptr) + (g_save != nullptr) + (b_save != nullptr);
    return saves == 0 || saves == 4;
}

template <typename S>
int chain_batch_launch(int32_t heads, int32_t batch, const int32_t* cu_rows, const glm53f_bf16* p, int64_t p_stride,
                       int64_t b_off, const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g, int64_t g_stride,
                       const glm53f_bf16* conv, const int64_t* conv_off, const glm53f_bf16* conv_w, const S* state_in,
                       S* state_out, const int64_t* state_off, const float* a_log, const float* dt_bias,
                       const glm53f_bf16* norm_w, float eps, float lower, glm53f_bf16* out, int64_t out_stride,
                       S* ckpt, float* k_save, glm53f_bf16* v_save, float* g_save, float* b_save,
                       glm53f_stream_t stream, int shift = 0) {
    if (batch < 1 || batch > 65535 || !cu_rows || !conv_off || !state_off ||
        !chain_args_ok(heads, p, a, g, conv, conv_w, state_in, a_log, dt_bias, norm_w, out, k_save, v_save, g_save,
                       b_save))
        return kInvalid;
    if (!aligned16(state_in) || !aligned16(state_out) || !aligned16(ckpt)) return kInvalid;
    chain_kernel<S><<<dim3(heads, batch), THREADS, 0, (hipStream_t)stream>>>(
        heads, cu_rows, 0, bfp(p), p_stride, b_off, bfp(a), a_stride, bfp(g), g_stride, bfp(conv),
        reinterpret_cast<const long long*>(conv_off), bfp(conv_w), state_in, state_out,
        reinterpret_cast<const long long*>(state_off), a_log, dt_bias, bfp(norm_w), eps, lower, bfp(out), out_stride,
        ckpt, k_save, bfp(v_save), g_save, b_save, shift);
    return launched();
}

// Host-side checks of the replays (reference: kda.cu:376-388).
template <typename S>
int replay_launch(int32_t heads, int32_t layers, int32_t batch, const int32_t* cu_rows, const int32_t* keep,
                  int32_t rows, const S* state_in, S* state_out, int64_t state_stride, const int64_t* state_off,
                  const float* k_save, const glm53f_bf16* v_save, const float* g_save, const float* b_save,
                  int64_t kv_stride, int64_t b_stride, glm53f_stream_t stream) {
    if (heads < 1 || layers < 1 || batch < 1 || batch > 65535 || (long long)heads * layers > 0x7fffffffLL ||
        !state_in || !state_out || !k_save || !v_save || !g_save || !b_save || rows < 0)
        return kInvalid;
    if (!aligned16(state_in) || !aligned16(state_out) || !aligned16(k_save) || !aligned16(g_save) ||
        (kv_stride & 3) != 0)
        return kInvalid;
    replay_kernel<S><<<dim3(heads * layers, batch), THREADS, 0, (hipStream_t)stream>>>(
        heads, cu_rows, keep, rows, state_in, state_out, state_stride,
        reinterpret_cast<const long long*>(state_off), k_save, bfp(v_save), g_save, b_save, kv_stride, b_stride);
    return launched();
}

constexpr int kShiftThreads = 256;

// Host-side checks of the conv shift (reference: kda.cu:433-444).
inline int conv_shift_launch(int32_t channels, int32_t layers, int32_t batch, const int32_t* cu_rows,
                             const int32_t* keep, int32_t keep1, glm53f_bf16* conv, int64_t conv_stride,
                             const int64_t* conv_off, const glm53f_bf16* p, int64_t p_layer_stride, int64_t p_stride,
                             glm53f_stream_t stream) {
    if (channels < 1 || layers < 1 || layers > 65535 || batch < 1 || batch > 65535 || !conv || !p || keep1 < 0)
        return kInvalid;
    const dim3 grid((channels + 8 * kShiftThreads - 1) / (8 * kShiftThreads), layers, batch);   // 8 channels per lane
    conv_shift_kernel<<<grid, kShiftThreads, 0, (hipStream_t)stream>>>(
        channels, cu_rows, keep, keep1, bfp(conv), conv_stride, reinterpret_cast<const long long*>(conv_off), bfp(p),
        p_layer_stride, p_stride);
    return launched();
}

}  // namespace
}  // namespace kda

using namespace kda;

extern "C" int glm53f_kda_chain(int32_t heads, int32_t rows, const glm53f_bf16* p, int64_t p_stride, int64_t b_off,
                                const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g, int64_t g_stride,
                                const glm53f_bf16* conv, const glm53f_bf16* conv_w, const float* state_in,
                                float* state_out, const float* a_log, const float* dt_bias,
                                const glm53f_bf16* norm_w, float eps, float lower, glm53f_bf16* out,
                                int64_t out_stride, float* k_save, glm53f_bf16* v_save, float* g_save,
                                float* b_save, glm53f_stream_t stream) {
    if (rows < 1 || !chain_args_ok(heads, p, a, g, conv, conv_w, state_in, a_log, dt_bias, norm_w, out, k_save,
                                   v_save, g_save, b_save))
        return kInvalid;
    if (!aligned16(state_in) || !aligned16(state_out)) return kInvalid;
    chain_kernel<float><<<dim3(heads, 1), THREADS, 0, (hipStream_t)stream>>>(
        heads, nullptr, rows, bfp(p), p_stride, b_off, bfp(a), a_stride, bfp(g), g_stride, bfp(conv), nullptr,
        bfp(conv_w), state_in, state_out, nullptr, a_log, dt_bias, bfp(norm_w), eps, lower, bfp(out), out_stride,
        nullptr, k_save, bfp(v_save), g_save, b_save, 0);
    return launched();
}

extern "C" int glm53f_kda_chain_batch(int32_t heads, int32_t batch, const int32_t* cu_rows, const glm53f_bf16* p,
                                      int64_t p_stride, int64_t b_off, const glm53f_bf16* a, int64_t a_stride,
                                      const glm53f_bf16* g, int64_t g_stride, const glm53f_bf16* conv,
                                      const int64_t* conv_off, const glm53f_bf16* conv_w, const float* state_in,
                                      float* state_out, const int64_t* state_off, const float* a_log,
                                      const float* dt_bias, const glm53f_bf16* norm_w, float eps, float lower,
                                      glm53f_bf16* out, int64_t out_stride, float* k_save, glm53f_bf16* v_save,
                                      float* g_save, float* b_save, glm53f_stream_t stream) {
    return chain_batch_launch<float>(heads, batch, cu_rows, p, p_stride, b_off, a, a_stride, g, g_stride, conv,
                                     conv_off, conv_w, state_in, state_out, state_off, a_log, dt_bias, norm_w, eps,
                                     lower, out, out_stride, nullptr, k_save, v_save, g_save, b_save, stream);
}

extern "C" int glm53f_kda_chain_batch_bf16state(int32_t heads, int32_t batch, const int32_t* cu_rows,
                                                const glm53f_bf16* p, int64_t p_stride, int64_t b_off,
                                                const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g,
                                                int64_t g_stride, const glm53f_bf16* conv, const int64_t* conv_off,
                                                const glm53f_bf16* conv_w, const glm53f_bf16* state_in,
                                                glm53f_bf16* state_out, const int64_t* state_off,
                                                const float* a_log, const float* dt_bias,
                                                const glm53f_bf16* norm_w, float eps, float lower,
                                                glm53f_bf16* out, int64_t out_stride, float* k_save,
                                                glm53f_bf16* v_save, float* g_save, float* b_save,
                                                glm53f_stream_t stream) {
    return chain_batch_launch<bf16_t>(heads, batch, cu_rows, p, p_stride, b_off, a, a_stride, g, g_stride, conv,
                                      conv_off, conv_w, bfp(state_in), bfp(state_out), state_off, a_log, dt_bias,
                                      norm_w, eps, lower, out, out_stride, nullptr, k_save, v_save, g_save, b_save,
                                      stream);
}

extern "C" int glm53f_kda_chain_shift_batch(int32_t heads, int32_t batch, const int32_t* cu_rows, const glm53f_bf16* p,
                                            int64_t p_stride, int64_t b_off, const glm53f_bf16* a, int64_t a_stride,
                                            const glm53f_bf16* g, int64_t g_stride, glm53f_bf16* conv,
                                            const int64_t* conv_off, const glm53f_bf16* conv_w,
                                            const float* state_in, float* state_out, const int64_t* state_off,
                                            const float* a_log, const float* dt_bias, const glm53f_bf16* norm_w,
                                            float eps, float lower, glm53f_bf16* out, int64_t out_stride,
                                            float* k_save, glm53f_bf16* v_save, float* g_save, float* b_save,
                                            glm53f_stream_t stream) {
    return chain_batch_launch<float>(heads, batch, cu_rows, p, p_stride, b_off, a, a_stride, g, g_stride, conv,
                                     conv_off, conv_w, state_in, state_out, state_off, a_log, dt_bias, norm_w, eps,
                                     lower, out, out_stride, nullptr, k_save, v_save, g_save, b_save, stream, 1);
}

extern "C" int glm53f_kda_chain_shift_batch_bf16state(int32_t heads, int32_t batch, const int32_t* cu_rows,
                                                      const glm53f_bf16* p, int64_t p_stride, int64_t b_off,
                                                      const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g,
                                                      int64_t g_stride, glm53f_bf16* conv, const int64_t* conv_off,
                                                      const glm53f_bf16* conv_w, const glm53f_bf16* state_in,
                                                      glm53f_bf16* state_out, const int64_t* state_off,
                                                      const float* a_log, const float* dt_bias,
                                                      const glm53f_bf16* norm_w, float eps, float lower,
                                                      glm53f_bf16* out, int64_t out_stride, float* k_save,
                                                      glm53f_bf16* v_save, float* g_save, float* b_save,
                                                      glm53f_stream_t stream) {
    return chain_batch_launch<bf16_t>(heads, batch, cu_rows, p, p_stride, b_off, a, a_stride, g, g_stride, conv,
                                      conv_off, conv_w, bfp(state_in), bfp(state_out), state_off, a_log, dt_bias,
                                      norm_w, eps, lower, out, out_stride, nullptr, k_save, v_save, g_save, b_save,
                                      stream, 1);
}

extern "C" int glm53f_kda_verify_batch_bf16state(int32_t heads, int32_t batch, const int32_t* cu_rows,
                                                 const glm53f_bf16* p, int64_t p_stride, int64_t b_off,
                                                 const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g,
                                                 int64_t g_stride, const glm53f_bf16* conv, const int64_t* conv_off,
                                                 const glm53f_bf16* conv_w, const glm53f_bf16* state_in,
                                                 const int64_t* state_off, const float* a_log,
                                                 const float* dt_bias, const glm53f_bf16* norm_w, float eps,
                                                 float lower, glm53f_bf16* out, int64_t out_stride,
                                                 glm53f_bf16* ckpt, float* k_save, glm53f_bf16* v_save,
                                                 float* g_save, float* b_save, glm53f_stream_t stream) {
    if (!ckpt) return kInvalid;
    return chain_batch_launch<bf16_t>(heads, batch, cu_rows, p, p_stride, b_off, a, a_stride, g, g_stride, conv,
                                      conv_off, conv_w, bfp(state_in), nullptr, state_off, a_log, dt_bias, norm_w,
                                      eps, lower, out, out_stride, bfp(ckpt), k_save, v_save, g_save, b_save, stream);
}

extern "C" int glm53f_kda_select_batch_bf16state(int32_t heads, int32_t layers, int32_t batch,
                                                 const int32_t* cu_rows, const int32_t* keep,
                                                 const glm53f_bf16* ckpt, int64_t ckpt_layer_stride,
                                                 glm53f_bf16* state, int64_t state_stride,
                                                 const int64_t* state_off, glm53f_stream_t stream) {
    if (heads < 1 || layers < 1 || batch < 1 || batch > 65535 || (long long)heads * layers > 0x7fffffffLL ||
        !cu_rows || !keep || !ckpt || !state || !state_off || !aligned16(ckpt) || !aligned16(state) ||
        (ckpt_layer_stride & 7) != 0 || (state_stride & 7) != 0)
        return kInvalid;
    select_kernel<<<dim3(heads * layers, batch), THREADS, 0, (hipStream_t)stream>>>(
        heads, cu_rows, keep, bfp(ckpt), ckpt_layer_stride, bfp(state), state_stride,
        reinterpret_cast<const long long*>(state_off));
    return launched();
}

extern "C" int glm53f_kda_replay(int32_t heads, int32_t rows, const float* state_in, float* state_out,
                                 const float* k_save, const glm53f_bf16* v_save, const float* g_save,
                                 const float* b_save, glm53f_stream_t stream) {
    return replay_launch<float>(heads, 1, 1, nullptr, nullptr, rows, state_in, state_out, 0, nullptr, k_save, v_save,
                                g_save, b_save, 0, 0, stream);
}

extern "C" int glm53f_kda_replay_layers(int32_t heads, int32_t layers, int32_t rows, const float* state_in,
                                        float* state_out, int64_t state_stride, const float* k_save,
                                        const glm53f_bf16* v_save, const float* g_save, const float* b_save,
                                        int64_t kv_stride, int64_t b_stride, glm53f_stream_t stream) {
    return replay_launch<float>(heads, layers, 1, nullptr, nullptr, rows, state_in, state_out, state_stride, nullptr,
                                k_save, v_save, g_save, b_save, kv_stride, b_stride, stream);
}

extern "C" int glm53f_kda_replay_batch(int32_t heads, int32_t layers, int32_t batch, const int32_t* cu_rows,
                                       const int32_t* keep, const float* state_in, float* state_out,
                                       int64_t state_stride, const int64_t* state_off, const float* k_save,
                                       const glm53f_bf16* v_save, const float* g_save, const float* b_save,
                                       int64_t kv_stride, int64_t b_stride, glm53f_stream_t stream) {
    if (!cu_rows || !keep || !state_off) return kInvalid;
    return replay_launch<float>(heads, layers, batch, cu_rows, keep, 0, state_in, state_out, state_stride, state_off,
                                k_save, v_save, g_save, b_save, kv_stride, b_stride, stream);
}

extern "C" int glm53f_kda_replay_batch_bf16state(int32_t heads, int32_t layers, int32_t batch,
                                                 const int32_t* cu_rows, const int32_t* keep,
                                                 const glm53f_bf16* state_in, glm53f_bf16* state_out,
                                                 int64_t state_stride, const int64_t* state_off,
                                                 const float* k_save, const glm53f_bf16* v_save,
                                                 const float* g_save, const float* b_save, int64_t kv_stride,
                                                 int64_t b_stride, glm53f_stream_t stream) {
    if (!cu_rows || !keep || !state_off) return kInvalid;
    return replay_launch<bf16_t>(heads, layers, batch, cu_rows, keep, 0, bfp(state_in), bfp(state_out), state_stride,
                                 state_off, k_save, v_save, g_save, b_save, kv_stride, b_stride, stream);
}

extern "C" int glm53f_kda_conv_shift(int32_t channels, int32_t keep, glm53f_bf16* conv, const glm53f_bf16* p,
                                     int64_t p_stride, glm53f_stream_t stream) {
    return conv_shift_launch(channels, 1, 1, nullptr, nullptr, keep, conv, 0, nullptr, p, 0, p_stride, stream);
}

extern "C" int glm53f_kda_conv_shift_batch(int32_t channels, int32_t layers, int32_t batch, const int32_t* cu_rows,
                                           const int32_t* keep, glm53f_bf16* conv, int64_t conv_stride,
                                           const int64_t* conv_off, const glm53f_bf16* p, int64_t p_layer_stride,
                                           int64_t p_stride, glm53f_stream_t stream) {
    if (!cu_rows || !keep || !conv_off) return kInvalid;
    return conv_shift_launch(channels, layers, batch, cu_rows, keep, 0, conv, conv_stride, conv_off, p,
                             p_layer_stride, p_stride, stream);
}

extern "C" const char* glm53f_kda_arch(void) { return "gfx950"; }
