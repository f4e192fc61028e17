/* TEST INFRASTRUCTURE ONLY: see kda_ref.h. Build: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp.
 *
 * Every sum is written `acc = acc + x` and the file is compiled with floating-point contraction off, so no
 * multiply and add fuse: the reference's Rust never contracts (cpu.rs:49-51). The only fused operations
 * are the explicit fmaf calls of the prefill host model (chunked.rs:292, :300).
 */
#include "kda_ref.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define DK KDA_DK
#define DV KDA_DV
#define TAPS KDA_TAPS
#define WINDOW KDA_WINDOW

static int64_t channels(int32_t heads) { return 3 * (int64_t)heads * DK; }

/* ------------------------------------------------------------------ bf16 (src/bf16.rs:6-46) */

static uint32_t f2u(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static float u2f(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

uint16_t kda_bf16_from_f32(float x) {
    uint32_t u = f2u(x);
    if (x != x) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    return (uint16_t)((u + (0x7fffu + lsb)) >> 16);
}

float kda_bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }

float kda_bf16_round(float x) { return kda_bf16_to_f32(kda_bf16_from_f32(x)); }

static int32_t ordered(uint16_t x) { return (x & 0x8000u) ? -(int32_t)(x & 0x7fffu) : (int32_t)x; }

uint32_t kda_bf16_ulp_distance(uint16_t a, uint16_t b) {
    int32_t d = ordered(a) - ordered(b);
    return (uint32_t)(d < 0 ? -d : d);
}

void kda_bf16_encode(const float* x, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = kda_bf16_from_f32(x[i]);
}

void kda_bf16_decode(const uint16_t* b, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = kda_bf16_to_f32(b[i]);
}

/* ------------------------------------------------------------------ rng (src/synth.rs:10-45) */

void kda_rng_new(kda_rng* r, uint64_t seed) { r->s = seed ^ 0x6a09e667f3bcc909ull; }

uint64_t kda_rng_next_u64(kda_rng* r) {
    r->s += 0x9e3779b97f4a7c15ull;
    uint64_t z = r->s;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

float kda_rng_uniform(kda_rng* r, float lo, float hi) {
    float u = (float)(kda_rng_next_u64(r) >> 40) / (float)(1ull << 24);
    return lo + (hi - lo) * u;
}

float kda_rng_uniform_bf16(kda_rng* r, float lo, float hi) { return kda_bf16_round(kda_rng_uniform(r, lo, hi)); }

void kda_rng_fill(kda_rng* r, float* out, int64_t n, float lo, float hi) {
    for (int64_t i = 0; i < n; ++i) out[i] = kda_rng_uniform(r, lo, hi);
}

void kda_rng_fill_bf16(kda_rng* r, float* out, int64_t n, float lo, float hi) {
    for (int64_t i = 0; i < n; ++i) out[i] = kda_rng_uniform_bf16(r, lo, hi);
}

float kda_rng_normal(kda_rng* r) {
    /* u1 in (0, 1], u2 in [0, 1): 24-bit uniforms, evaluated in double so the draw does not depend on libm's
     * float variants. */
    double u1 = ((double)(kda_rng_next_u64(r) >> 40) + 1.0) / 16777216.0;
    double u2 = (double)(kda_rng_next_u64(r) >> 40) / 16777216.0;
    return (float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2));
}

void kda_rng_fill_normal(kda_rng* r, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = kda_rng_normal(r);
}

/* src/synth.rs:49-83 */
void kda_synth_layer(int32_t heads, uint64_t seed, float* conv_w, float* a_log, float* dt_bias, float* norm_w) {
    kda_rng r;
    kda_rng_new(&r, (seed * 3ull) ^ 0x11ull);
    kda_rng_fill_bf16(&r, conv_w, channels(heads) * TAPS, -0.6f, 0.6f);
    kda_rng_fill(&r, a_log, heads, -1.5f, 1.5f);
    kda_rng_fill(&r, dt_bias, (int64_t)heads * DK, -1.0f, 1.0f);
    kda_rng_fill_bf16(&r, norm_w, DV, 0.25f, 1.75f);
}

void kda_synth_rows(int32_t heads, int32_t rows, uint64_t seed, float* qkv, float* a, float* b, float* gate) {
    kda_rng r;
    kda_rng_new(&r, (seed * 5ull) ^ 0x22ull);
    kda_rng_fill_bf16(&r, qkv, (int64_t)rows * channels(heads), -2.0f, 2.0f);
    kda_rng_fill_bf16(&r, a, (int64_t)rows * heads * DK, -4.0f, 4.0f);
    kda_rng_fill_bf16(&r, b, (int64_t)rows * heads, -4.0f, 4.0f);
    kda_rng_fill_bf16(&r, gate, (int64_t)rows * heads * DV, -4.0f, 4.0f);
}

void kda_synth_conv_window(int32_t heads, uint64_t seed, float* conv) {
    kda_rng r;
    kda_rng_new(&r, (seed * 7ull) ^ 0x33ull);
    kda_rng_fill_bf16(&r, conv, WINDOW * channels(heads), -2.0f, 2.0f);
}

void kda_synth_state(int32_t heads, uint64_t seed, float scale, float* state) {
    kda_rng r;
    kda_rng_new(&r, (seed * 11ull) ^ 0x44ull);
    kda_rng_fill(&r, state, (int64_t)heads * DV * DK, -scale, scale);
}

/* ------------------------------------------------------------------ scalar pieces (cpu.rs:202-254) */

float kda_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

float kda_silu(float x) { return x / (1.0f + expf(-x)); }

/* cpu.rs:214-225: the 32-lane xor butterfly, offsets 16, 8, 4, 2, 1. */
float kda_warp_sum(const float lanes[32]) {
    float x[32], prev[32];
    memcpy(x, lanes, sizeof x);
    for (int o = 16; o > 0; o >>= 1) {
        memcpy(prev, x, sizeof x);
        for (int l = 0; l < 32; ++l) x[l] = prev[l] + prev[l ^ o];
    }
    return x[0];
}

/* cpu.rs:229-239 */
float kda_dot128(const float* a, const float* b) {
    float lanes[32];
    for (int l = 0; l < 32; ++l) {
        float acc = 0.0f;
        for (int i = 0; i < 4; ++i) acc = acc + a[4 * l + i] * b[4 * l + i];
        lanes[l] = acc;
    }
    return kda_warp_sum(lanes);
}

/* cpu.rs:242-244 */
float kda_log_decay(float a, float dt_bias, float a_log, float lower) {
    return lower * kda_sigmoid(expf(a_log) * (a + dt_bias));
}

/* cpu.rs:247-249 */
float kda_decay(float a, float dt_bias, float decay_rate, float lower) {
    return expf(lower * kda_sigmoid(decay_rate * (a + dt_bias)));
}

/* cpu.rs:252-254 */
float kda_beta(float b) { return kda_bf16_round(kda_sigmoid(b)); }

/* cpu.rs:318-320 */
float kda_q_scale(void) { return 1.0f / sqrtf((float)DK); }

static float round_as(int mode, float x) { return mode == KDA_F32 ? x : kda_bf16_round(x); }

/* ------------------------------------------------------------------ per-row pieces */

/* cpu.rs:257-281 */
float kda_conv_channel(const kda_layer* p, const float* conv, const kda_rows* rows, int32_t r, int32_t c,
                       int mode) {
    const int64_t cn = channels(p->heads);
    float acc = 0.0f;
    for (int tap = 0; tap < TAPS; ++tap) {
        const int64_t at = (int64_t)r + tap;
        const float x = at < WINDOW ? conv[at * cn + c] : rows->qkv[(at - WINDOW) * cn + c];
        acc = acc + p->conv_w[(int64_t)c * TAPS + tap] * x;
    }
    switch (mode) {
        case KDA_FUSED: return kda_bf16_round(kda_silu(acc));
        case KDA_UNFUSED: return kda_bf16_round(kda_silu(kda_bf16_round(acc)));
        default: return kda_silu(acc);
    }
}

/* cpu.rs:284-302 */
void kda_conv_qkv(const kda_layer* p, const float* conv, const kda_rows* rows, int32_t r, int32_t h, int mode,
                  float* q, float* k, float* v) {
    const int32_t hd = p->heads * DK;
    for (int i = 0; i < DK; ++i) {
        q[i] = kda_conv_channel(p, conv, rows, r, h * DK + i, mode);
        k[i] = kda_conv_channel(p, conv, rows, r, hd + h * DK + i, mode);
        v[i] = kda_conv_channel(p, conv, rows, r, 2 * hd + h * DK + i, mode);
    }
}

/* cpu.rs:305-315 */
void kda_l2norm(const float* x, float scale, float* y) {
    const float inv = 1.0f / sqrtf(kda_dot128(x, x) + KDA_L2_EPS);
    for (int i = 0; i < DK; ++i) {
        float t = x[i] * inv;
        if (scale > 0.0f) t = t * scale;
        y[i] = t;
    }
}

/* cpu.rs:324-344 */
void kda_update(float* s, const float* k, const float* g, const float* v, float beta) {
    for (int row = 0; row < DV; ++row) {
        float* sr = s + row * DK;
        float lanes[32];
        for (int l = 0; l < 32; ++l) {
            float kv = 0.0f;
            for (int i = 0; i < 4; ++i) {
                const int c = 4 * l + i;
                sr[c] = sr[c] * g[c];
                kv = kv + sr[c] * k[c];
            }
            lanes[l] = kv;
        }
        const float kv = kda_warp_sum(lanes);
        const float delta = (v[row] - kv) * beta;
        for (int c = 0; c < DK; ++c) sr[c] = sr[c] + k[c] * delta;
    }
}

/* cpu.rs:347-353 */
void kda_read_out(const float* s, const float* q, float* y) {
    for (int row = 0; row < DV; ++row) y[row] = kda_dot128(s + row * DK, q);
}

/* cpu.rs:361-376 */
void kda_gated_rmsnorm_as(const float* y, const float* norm_w, const float* gate, float eps, int mode, float* o) {
    const float rinv = 1.0f / sqrtf(kda_dot128(y, y) / (float)DV + eps);
    for (int t = 0; t < DV; ++t) {
        const float yn = y[t] * rinv;
        const float yw = norm_w[t] * yn;
        o[t] = round_as(mode, yw * kda_sigmoid(gate[t]));
    }
}

static void round_state(float* s, int64_t n) {
    for (int64_t i = 0; i < n; ++i) s[i] = kda_bf16_round(s[i]);
}

/* ------------------------------------------------------------------ chain (cpu.rs:410-471) */

void kda_chain_with(const kda_layer* p, const float* conv, const float* state, const kda_rows* rows, int mode,
                    int bf16_state, float* out, float* y_out, float* state_out, float* k_save, float* v_save,
                    float* g_save, float* b_save, int threads) {
    const int32_t hn = p->heads, rn = rows->rows;
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(dynamic, 1)
    for (int32_t h = 0; h < hn; ++h) {
        const float decay_rate = expf(p->a_log[h]);
        float s[DV * DK];
        memcpy(s, state + (int64_t)h * DV * DK, sizeof s);
        for (int32_t r = 0; r < rn; ++r) {
            float q[DK], k[DK], v[DV], g[DK], qn[DK], kn[DK], y[DV], o[DV];
            kda_conv_qkv(p, conv, rows, r, h, mode, q, k, v);
            for (int i = 0; i < DK; ++i)
                g[i] = kda_decay(rows->a[((int64_t)r * hn + h) * DK + i], p->dt_bias[h * DK + i], decay_rate,
                                 p->lower);
            const float b = round_as(mode, kda_sigmoid(rows->b[(int64_t)r * hn + h]));
            kda_l2norm(q, kda_q_scale(), qn);
            kda_l2norm(k, 0.0f, kn);
            kda_update(s, kn, g, v, b);
            kda_read_out(s, qn, y);
            for (int i = 0; i < DV; ++i) y[i] = round_as(mode, y[i]);
            if (bf16_state) round_state(s, DV * DK);
            const float* gate = rows->gate + ((int64_t)r * hn + h) * DV;
            kda_gated_rmsnorm_as(y, p->norm_w, gate, p->eps, mode, o);
            const int64_t at = ((int64_t)r * hn + h) * DV;
            if (out) memcpy(out + at, o, sizeof o);
            if (y_out) memcpy(y_out + at, y, sizeof y);
            if (k_save) {
                memcpy(k_save + at, kn, sizeof kn);
                memcpy(v_save + at, v, sizeof v);
                memcpy(g_save + at, g, sizeof g);
                b_save[(int64_t)r * hn + h] = b;
            }
        }
        if (state_out) memcpy(state_out + (int64_t)h * DV * DK, s, sizeof s);
    }
}

/* cpu.rs:486-508 */
void kda_replay_with(int32_t heads, const float* state, const float* k_save, const float* v_save,
                     const float* g_save, const float* b_save, int32_t keep, int bf16_state, float* state_out) {
    if (state_out != state) memcpy(state_out, state, sizeof(float) * (size_t)heads * DV * DK);
    for (int32_t h = 0; h < heads; ++h) {
        float* s = state_out + (int64_t)h * DV * DK;
        for (int32_t r = 0; r < keep; ++r) {
            const int64_t at = ((int64_t)r * heads + h) * DK;
            kda_update(s, k_save + at, g_save + at, v_save + at, b_save[(int64_t)r * heads + h]);
            if (bf16_state) round_state(s, DV * DK);
        }
    }
}

/* tests/gpu_prefill.rs:502-519 */
void kda_exact_replay(int32_t heads, const float* state, const float* k_save, const float* v_save,
                      const float* g_save, const float* b_save, int32_t rows, double* state_out, int threads) {
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(dynamic)
    for (int32_t h = 0; h < heads; ++h) {
        double* s = state_out + (int64_t)h * DV * DK;
        for (int i = 0; i < DV * DK; ++i) s[i] = (double)state[(int64_t)h * DV * DK + i];
        for (int32_t r = 0; r < rows; ++r) {
            const int64_t at = ((int64_t)r * heads + h) * DK;
            const double beta = (double)b_save[(int64_t)r * heads + h];
            for (int row = 0; row < DV; ++row) {
                double* sr = s + row * DK;
                double kv = 0.0;
                for (int k = 0; k < DK; ++k) {
                    sr[k] *= (double)g_save[at + k];
                    kv += sr[k] * (double)k_save[at + k];
                }
                const double delta = ((double)v_save[at + row] - kv) * beta;
                for (int k = 0; k < DK; ++k) sr[k] += (double)k_save[at + k] * delta;
            }
        }
    }
}

/* cpu.rs:512-527 */
void kda_conv_shift(int32_t heads, const float* conv, const float* qkv, int32_t rows, int32_t keep, float* out) {
    const int64_t cn = channels(heads);
    (void)rows;
    float* tmp = (float*)malloc(sizeof(float) * WINDOW * cn);
    for (int j = 0; j < WINDOW; ++j) {
        const int64_t src = (int64_t)keep + j;
        const float* from = src < WINDOW ? conv + src * cn : qkv + (src - WINDOW) * cn;
        memcpy(tmp + j * cn, from, sizeof(float) * cn);
    }
    memcpy(out, tmp, sizeof(float) * WINDOW * cn);
    free(tmp);
}

/* cpu.rs:531-547: [n/(128*128)][A][B] -> [..][B][A]. */
void kda_transpose_state(const float* s, float* t, int64_t n) {
    for (int64_t h = 0; h < n / (DK * DV); ++h) {
        const float* hs = s + h * DK * DV;
        float* ht = t + h * DK * DV;
        for (int a = 0; a < DV; ++a)
            for (int b = 0; b < DK; ++b) ht[b * DV + a] = hs[a * DK + b];
    }
}

/* ------------------------------------------------------------------ literal (cpu.rs:553-686) */

/* cpu.rs:557-568 */
void kda_literal_l2norm(const float* x, float* y) {
    float ss = 0.0f;
    for (int i = 0; i < DK; ++i) ss = ss + x[i] * x[i];
    const float n = sqrtf(ss + KDA_L2_EPS);
    for (int i = 0; i < DK; ++i) y[i] = x[i] / n;
}

/* cpu.rs:573-610 */
void kda_literal_step(float* s, const float* q, const float* k, const float* v, const float* g, float beta,
                      float* y) {
    float qn[DK], kn[DK], qs[DK], delta[DV];
    kda_literal_l2norm(q, qn);
    kda_literal_l2norm(k, kn);
    const float scale = kda_q_scale();
    for (int i = 0; i < DK; ++i) qs[i] = qn[i] * scale;
    for (int kk = 0; kk < DK; ++kk) {
        const float e = expf(g[kk]);
        for (int vv = 0; vv < DV; ++vv) s[kk * DV + vv] = s[kk * DV + vv] * e;
    }
    for (int vv = 0; vv < DV; ++vv) {
        float kv = 0.0f;
        for (int kk = 0; kk < DK; ++kk) kv = kv + s[kk * DV + vv] * kn[kk];
        delta[vv] = (v[vv] - kv) * beta;
    }
    for (int kk = 0; kk < DK; ++kk)
        for (int vv = 0; vv < DV; ++vv) s[kk * DV + vv] = s[kk * DV + vv] + kn[kk] * delta[vv];
    for (int vv = 0; vv < DV; ++vv) {
        float o = 0.0f;
        for (int kk = 0; kk < DK; ++kk) o = o + s[kk * DV + vv] * qs[kk];
        y[vv] = o;
    }
}

/* cpu.rs:618-635 */
void kda_literal_gated_rmsnorm_as(const float* y, const float* norm_w, const float* gate, float eps, int mode,
                                  float* o) {
    float ss = 0.0f;
    for (int i = 0; i < DV; ++i) ss = ss + y[i] * y[i];
    const float r = 1.0f / sqrtf(ss / (float)DV + eps);
    for (int t = 0; t < DV; ++t) o[t] = round_as(mode, norm_w[t] * (y[t] * r) * kda_sigmoid(gate[t]));
}

/* cpu.rs:639-685 */
void kda_literal_chain(const kda_layer* p, const float* conv, const float* state, const kda_rows* rows, int mode,
                       float* out, float* y_out, float* state_out, float* k_save, float* v_save, float* g_save,
                       float* b_save, int threads) {
    const int32_t hn = p->heads, rn = rows->rows;
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(dynamic, 1)
    for (int32_t h = 0; h < hn; ++h) {
        float s[DK * DV];
        kda_transpose_state(state + (int64_t)h * DV * DK, s, DK * DV);
        for (int32_t r = 0; r < rn; ++r) {
            float q[DK], k[DK], v[DV], g[DK], y[DV], o[DV], kn[DK];
            kda_conv_qkv(p, conv, rows, r, h, mode, q, k, v);
            for (int i = 0; i < DK; ++i)
                g[i] = kda_log_decay(rows->a[((int64_t)r * hn + h) * DK + i], p->dt_bias[h * DK + i], p->a_log[h],
                                     p->lower);
            const float b = round_as(mode, kda_sigmoid(rows->b[(int64_t)r * hn + h]));
            kda_literal_step(s, q, k, v, g, b, y);
            for (int i = 0; i < DV; ++i) y[i] = round_as(mode, y[i]);
            const float* gate = rows->gate + ((int64_t)r * hn + h) * DV;
            kda_literal_gated_rmsnorm_as(y, p->norm_w, gate, p->eps, mode, o);
            const int64_t at = ((int64_t)r * hn + h) * DV;
            if (out) memcpy(out + at, o, sizeof o);
            if (y_out) memcpy(y_out + at, y, sizeof y);
            if (k_save) {
                kda_literal_l2norm(k, kn);
                memcpy(k_save + at, kn, sizeof kn);
                memcpy(v_save + at, v, sizeof v);
                for (int i = 0; i < DK; ++i) g_save[at + i] = expf(g[i]);
                b_save[(int64_t)r * hn + h] = b;
            }
        }
        if (state_out) kda_transpose_state(s, state_out + (int64_t)h * DV * DK, DK * DV);
    }
}

/* ------------------------------------------------------------------ chunked (chunked.rs:67-198) */

void kda_chunked_head(const float* q, const float* k, const float* v, const float* g, const float* beta,
                      int32_t t, float* state, int32_t chunk, float* out) {
    const int c = chunk;
    float* gc = (float*)malloc(sizeof(float) * c * DK);
    float* a = (float*)malloc(sizeof(float) * c * c);
    float* rowi = (float*)malloc(sizeof(float) * c);
    float* u = (float*)malloc(sizeof(float) * c * DV);
    float* w = (float*)malloc(sizeof(float) * c * DK);
    float* vnew = (float*)malloc(sizeof(float) * c * DV);
    float* m = (float*)malloc(sizeof(float) * c);
    int32_t start = 0;
    while (start < t) {
        const int n = c < t - start ? c : t - start;
#define AT(w_, i_) ((int64_t)(start + (i_)) * (w_))
        /* Cumulative log decay within the chunk (chunked.rs:92-98). */
        for (int i = 0; i < n; ++i)
            for (int d = 0; d < DK; ++d) {
                const float prev = i == 0 ? 0.0f : gc[(i - 1) * DK + d];
                gc[i * DK + d] = prev + g[AT(DK, i) + d];
            }
        /* 1. A, strictly lower triangular, and the forward substitution (chunked.rs:100-124). */
        memset(a, 0, sizeof(float) * n * n);
        for (int i = 0; i < n; ++i) {
            const float bi = beta[start + i];
            for (int j = 0; j < i; ++j) {
                float acc = 0.0f;
                for (int d = 0; d < DK; ++d) {
                    const float kb = k[AT(DK, i) + d] * bi;
                    acc = acc + kb * k[AT(DK, j) + d] * expf(gc[i * DK + d] - gc[j * DK + d]);
                }
                a[i * n + j] = -acc;
            }
        }
        for (int i = 1; i < n; ++i) {
            memcpy(rowi, a + i * n, sizeof(float) * i);
            for (int col = 0; col < i; ++col) {
                float acc = 0.0f;
                for (int mm = 0; mm < i; ++mm) acc = acc + rowi[mm] * a[mm * n + col];
                a[i * n + col] = rowi[col] + acc;
            }
        }
        for (int i = 0; i < n; ++i) a[i * n + i] = a[i * n + i] + 1.0f;
        /* 2. U = T (beta V), W = T (beta K exp(G)) (chunked.rs:126-145). */
        for (int i = 0; i < n; ++i) {
            for (int vv = 0; vv < DV; ++vv) {
                float acc = 0.0f;
                for (int j = 0; j < n; ++j) acc = acc + a[i * n + j] * (v[AT(DV, j) + vv] * beta[start + j]);
                u[i * DV + vv] = acc;
            }
            for (int d = 0; d < DK; ++d) {
                float acc = 0.0f;
                for (int j = 0; j < n; ++j)
                    acc = acc + a[i * n + j] * (k[AT(DK, j) + d] * beta[start + j] * expf(gc[j * DK + d]));
                w[i * DK + d] = acc;
            }
        }
        /* 3. The chunk against the incoming state (chunked.rs:147-194). */
        for (int i = 0; i < n; ++i)
            for (int vv = 0; vv < DV; ++vv) {
                float acc = 0.0f;
                for (int d = 0; d < DK; ++d) acc = acc + w[i * DK + d] * state[d * DV + vv];
                vnew[i * DV + vv] = u[i * DV + vv] - acc;
            }
        for (int i = 0; i < n; ++i) {
            for (int j = 0; j <= i; ++j) {
                float acc = 0.0f;
                for (int d = 0; d < DK; ++d)
                    acc = acc + q[AT(DK, i) + d] * k[AT(DK, j) + d] * expf(gc[i * DK + d] - gc[j * DK + d]);
                m[j] = acc;
            }
            for (int vv = 0; vv < DV; ++vv) {
                float inter = 0.0f;
                for (int d = 0; d < DK; ++d)
                    inter = inter + q[AT(DK, i) + d] * expf(gc[i * DK + d]) * state[d * DV + vv];
                float intra = 0.0f;
                for (int j = 0; j <= i; ++j) intra = intra + m[j] * vnew[j * DV + vv];
                out[(int64_t)(start + i) * DV + vv] = inter + intra;
            }
        }
        const int last = n - 1;
        for (int d = 0; d < DK; ++d) {
            const float decay_all = expf(gc[last * DK + d]);
            for (int vv = 0; vv < DV; ++vv) {
                float acc = 0.0f;
                for (int i = 0; i < n; ++i)
                    acc = acc + k[AT(DK, i) + d] * expf(gc[last * DK + d] - gc[i * DK + d]) * vnew[i * DV + vv];
                state[d * DV + vv] = state[d * DV + vv] * decay_all + acc;
            }
        }
#undef AT
        start += n;
    }
    free(gc); free(a); free(rowi); free(u); free(w); free(vnew); free(m);
}

/* Gather one head's rows out of a [t][H][w] tensor. */
static void gather_head(const float* x, int32_t t, int32_t heads, int32_t h, int w, float* out) {
    for (int32_t r = 0; r < t; ++r) memcpy(out + (int64_t)r * w, x + ((int64_t)r * heads + h) * w, sizeof(float) * w);
}

/* chunked.rs:205-254 */
void kda_chunked_layer(int32_t heads, const float* q, const float* k, const float* v, const float* g,
                       const float* beta, int32_t t, float* state, int32_t chunk, float* out, int threads) {
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(dynamic, 1)
    for (int32_t h = 0; h < heads; ++h) {
        float* qh = (float*)malloc(sizeof(float) * (size_t)t * DK);
        float* kh = (float*)malloc(sizeof(float) * (size_t)t * DK);
        float* vh = (float*)malloc(sizeof(float) * (size_t)t * DV);
        float* gh = (float*)malloc(sizeof(float) * (size_t)t * DK);
        float* bh = (float*)malloc(sizeof(float) * (size_t)t);
        float* o = (float*)malloc(sizeof(float) * (size_t)t * DV);
        const float scale = kda_q_scale();
        for (int32_t r = 0; r < t; ++r) {
            kda_literal_l2norm(q + ((int64_t)r * heads + h) * DK, qh + (int64_t)r * DK);
            for (int i = 0; i < DK; ++i) qh[(int64_t)r * DK + i] = qh[(int64_t)r * DK + i] * scale;
            kda_literal_l2norm(k + ((int64_t)r * heads + h) * DK, kh + (int64_t)r * DK);
            bh[r] = beta[(int64_t)r * heads + h];
        }
        gather_head(v, t, heads, h, DV, vh);
        gather_head(g, t, heads, h, DK, gh);
        kda_chunked_head(qh, kh, vh, gh, bh, t, state + (int64_t)h * DK * DV, chunk, o);
        for (int32_t r = 0; r < t; ++r)
            memcpy(out + ((int64_t)r * heads + h) * DV, o + (int64_t)r * DV, sizeof(float) * DV);
        free(qh); free(kh); free(vh); free(gh); free(bh); free(o);
    }
}

/* The recurrence on the same core-level inputs: literal_step per row (tests/cpu_reference.rs:354-369). */
void kda_recurrent_layer(int32_t heads, const float* q, const float* k, const float* v, const float* g,
                         const float* beta, int32_t t, float* state, float* out, int threads) {
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(dynamic, 1)
    for (int32_t h = 0; h < heads; ++h) {
        float* s = state + (int64_t)h * DK * DV;
        for (int32_t r = 0; r < t; ++r) {
            const int64_t i = (int64_t)r * heads + h;
            kda_literal_step(s, q + i * DK, k + i * DK, v + i * DV, g + i * DK, beta[i], out + i * DV);
        }
    }
}

/* ------------------------------------------------------------------ prefill host model (chunked.rs:263-400) */

void kda_prefill_head(const float* qn, const float* kn, const float* v, const float* d, const float* beta,
                      int32_t t, float* s, float* y) {
    enum { CH = KDA_PREFILL_CHUNK };
    float lf[CH * DK], hi[DK], lo[DK], d0[DK], last[DK], elast[DK];
    float a[CH * DK], aq[CH * DK], b[CH * DK], l[CH * CH], m[CH * CH], tm[CH * CH];
    float w[CH * DK], u[CH * DV], delta[CH * DV];
    int32_t start = 0;
    while (start < t) {
        const int n = CH < t - start ? CH : t - start;
#define ROW(w_, i_) ((int64_t)(start + (i_)) * (w_))
        /* Decay products from the chunk's first row, each rounded once (chunked.rs:282-301). */
        for (int i = 0; i < n * DK; ++i) lf[i] = 1.0f;
        for (int k = 0; k < DK; ++k) { hi[k] = 1.0f; lo[k] = 0.0f; }
        for (int i = 1; i < n; ++i)
            for (int k = 0; k < DK; ++k) {
                const float dk = d[ROW(DK, i) + k];
                const float p = hi[k] * dk;
                lo[k] = fmaf(lo[k], dk, fmaf(hi[k], dk, -p));
                hi[k] = p;
                lf[i * DK + k] = hi[k] + lo[k];
            }
        for (int k = 0; k < DK; ++k) {
            d0[k] = d[ROW(DK, 0) + k];
            last[k] = lf[(n - 1) * DK + k];
            elast[k] = fmaf(d0[k], hi[k], d0[k] * lo[k]);
        }
        for (int i = 0; i < n; ++i)
            for (int k = 0; k < DK; ++k) {
                const float f = lf[i * DK + k];
                a[i * DK + k] = kn[ROW(DK, i) + k] * f;
                aq[i * DK + k] = qn[ROW(DK, i) + k] * f;
                b[i * DK + k] = kn[ROW(DK, i) + k] / f;
            }
        /* L and M (chunked.rs:314-328). */
        memset(l, 0, sizeof l);
        memset(m, 0, sizeof m);
        for (int i = 0; i < n; ++i)
            for (int j = 0; j <= i; ++j) {
                float sl = 0.0f, sm = 0.0f;
                for (int k = 0; k < DK; ++k) {
                    sl = sl + a[i * DK + k] * b[j * DK + k];
                    sm = sm + aq[i * DK + k] * b[j * DK + k];
                }
                m[i * n + j] = sm;
                if (j < i) l[i * n + j] = beta[start + i] * sl;
            }
        /* T = (I + L)^-1, then T' = T diag(beta) (chunked.rs:330-345). */
        memset(tm, 0, sizeof tm);
        for (int i = 0; i < n; ++i) {
            tm[i * n + i] = 1.0f;
            for (int j = 0; j < i; ++j) {
                float acc = l[i * n + j];
                for (int mm = j + 1; mm < i; ++mm) acc = acc + l[i * n + mm] * tm[mm * n + j];
                tm[i * n + j] = -acc;
            }
        }
        for (int i = 0; i < n; ++i)
            for (int j = 0; j <= i; ++j) tm[i * n + j] = tm[i * n + j] * beta[start + j];
        /* W = d0 * T'A, U = T'V (chunked.rs:347-364). */
        for (int i = 0; i < n; ++i) {
            for (int k = 0; k < DK; ++k) {
                float acc = 0.0f;
                for (int j = 0; j <= i; ++j) acc = acc + tm[i * n + j] * a[j * DK + k];
                w[i * DK + k] = d0[k] * acc;
            }
            for (int vv = 0; vv < DV; ++vv) {
                float acc = 0.0f;
                for (int j = 0; j <= i; ++j) acc = acc + tm[i * n + j] * v[ROW(DV, j) + vv];
                u[i * DV + vv] = acc;
            }
        }
        /* The chunk against the incoming state, s[v][k] (chunked.rs:366-396). */
        for (int i = 0; i < n; ++i)
            for (int vv = 0; vv < DV; ++vv) {
                float acc = 0.0f;
                for (int k = 0; k < DK; ++k) acc = acc + w[i * DK + k] * s[vv * DK + k];
                delta[i * DV + vv] = u[i * DV + vv] - acc;
            }
        for (int i = 0; i < n; ++i)
            for (int vv = 0; vv < DV; ++vv) {
                float acc = 0.0f;
                for (int k = 0; k < DK; ++k) acc = acc + (aq[i * DK + k] * d0[k]) * s[vv * DK + k];
                for (int j = 0; j <= i; ++j) acc = acc + m[i * n + j] * delta[j * DV + vv];
                y[(int64_t)(start + i) * DV + vv] = acc;
            }
        for (int vv = 0; vv < DV; ++vv)
            for (int k = 0; k < DK; ++k) {
                float acc = s[vv * DK + k] * elast[k];
                for (int i = 0; i < n; ++i) acc = acc + (b[i * DK + k] * last[k]) * delta[i * DV + vv];
                s[vv * DK + k] = acc;
            }
#undef ROW
        start += n;
    }
}

/* chunked.rs:405-467 */
void kda_prefill(const kda_layer* p, const float* conv, const float* state, const kda_rows* rows, int mode,
                 float* out, float* y_out, float* state_out, int threads) {
    const int32_t hn = p->heads, rn = rows->rows;
#pragma omp parallel for num_threads(threads > 1 ? threads : 1) schedule(dynamic, 1)
    for (int32_t h = 0; h < hn; ++h) {
        const float decay_rate = expf(p->a_log[h]);
        const size_t n = (size_t)(rn > 0 ? rn : 1);
        float* qn = (float*)malloc(sizeof(float) * n * DK);
        float* kn = (float*)malloc(sizeof(float) * n * DK);
        float* v = (float*)malloc(sizeof(float) * n * DV);
        float* d = (float*)malloc(sizeof(float) * n * DK);
        float* beta = (float*)malloc(sizeof(float) * n);
        float* y = (float*)malloc(sizeof(float) * n * DV);
        float s[DV * DK];
        memcpy(s, state + (int64_t)h * DV * DK, sizeof s);
        for (int32_t r = 0; r < rn; ++r) {
            float q[DK], k[DK];
            kda_conv_qkv(p, conv, rows, r, h, mode, q, k, v + (int64_t)r * DV);
            kda_l2norm(q, kda_q_scale(), qn + (int64_t)r * DK);
            kda_l2norm(k, 0.0f, kn + (int64_t)r * DK);
            for (int i = 0; i < DK; ++i)
                d[(int64_t)r * DK + i] = kda_decay(rows->a[((int64_t)r * hn + h) * DK + i], p->dt_bias[h * DK + i],
                                                   decay_rate, p->lower);
            beta[r] = round_as(mode, kda_sigmoid(rows->b[(int64_t)r * hn + h]));
        }
        kda_prefill_head(qn, kn, v, d, beta, rn, s, y);
        for (int32_t r = 0; r < rn; ++r) {
            float yr[DV], o[DV];
            for (int i = 0; i < DV; ++i) yr[i] = round_as(mode, y[(int64_t)r * DV + i]);
            const float* gate = rows->gate + ((int64_t)r * hn + h) * DV;
            kda_gated_rmsnorm_as(yr, p->norm_w, gate, p->eps, mode, o);
            const int64_t at = ((int64_t)r * hn + h) * DV;
            if (out) memcpy(out + at, o, sizeof o);
            if (y_out) memcpy(y_out + at, yr, sizeof yr);
        }
        if (state_out) memcpy(state_out + (int64_t)h * DV * DK, s, sizeof s);
        free(qn); free(kn); free(v); free(d); free(beta); free(y);
    }
}
