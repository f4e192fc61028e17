/* TEST INFRASTRUCTURE ONLY: the CPU oracle of the KDA hot path.
 *
 * A plain-C restatement, in f32, of the reference's own CPU formulation of Kimi delta attention
 * (crates/glm53f-kda/src/cpu.rs, src/chunked.rs, src/bf16.rs, src/synth.rs of the reference). It is the
 * checker for the HIP kernels and the CPU baseline of the benchmark. Nothing in the shipped library links,
 * loads or calls it: only tests, the smoke check and the benchmark's CPU-baseline leg may.
 *
 * Parity status of each function (what pins it without the reference's toolchain):
 *   bf16 conversions         known answers of src/bf16.rs:52-77, and torch's bfloat16 cast
 *   rng                      Vigna's published SplitMix64 vector
 *   gates, beta              closed forms / known answers of tests/cpu_reference.rs:36-55
 *   conv, conv_shift         known answers of tests/cpu_reference.rs:66-100
 *   warp_sum, dot128         known answers of tests/cpu_reference.rs:103-121
 *   l2norm, gated_rmsnorm    known answers of tests/cpu_reference.rs:124-145
 *   update, read_out, chain  invariants of tests/cpu_reference.rs:148-257, an f64 textbook recurrence
 *   literal_*                tests/cpu_reference.rs:260-285, the f64 textbook recurrence
 *   exact_replay             the same f64 recurrence written independently in the tests (numpy), small inputs
 *   chunked_head/layer       exact-arithmetic identity with the recurrence, tests/cpu_reference.rs:348-384
 *   prefill_head/prefill     tests/cpu_reference.rs:399-450
 * Bit-level agreement with the transformers 5.17.0 `chunk_kimi_delta_attention` on real activations is
 * "parity unpinned": the package and the golden payloads are absent.
 *
 * Layouts (elements, row major): state [H][DV][DK] ("kernel layout", value row major) unless a function says
 * [DK][DV] ("reference layout"); conv window [3][C], oldest first, C = 3*H*128 (q | k | v); conv weight [C][4],
 * tap 3 multiplies the current row. bfloat16 tensors are carried as f32 holding bfloat16-exact values.
 */
#ifndef KDA_REF_H
#define KDA_REF_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KDA_DK 128
#define KDA_DV 128
#define KDA_TAPS 4
#define KDA_WINDOW 3
#define KDA_L2_EPS 1e-6f
#define KDA_PREFILL_CHUNK 16

/* Rounding modes (cpu.rs:57-80). */
enum { KDA_FUSED = 0, KDA_UNFUSED = 1, KDA_F32 = 2 };

/* ---- bf16 (src/bf16.rs:6-46) ---- */
uint16_t kda_bf16_from_f32(float x);
float kda_bf16_to_f32(uint16_t b);
float kda_bf16_round(float x);
uint32_t kda_bf16_ulp_distance(uint16_t a, uint16_t b);
void kda_bf16_encode(const float* x, uint16_t* out, int64_t n);
void kda_bf16_decode(const uint16_t* b, float* out, int64_t n);

/* ---- SplitMix64 (src/synth.rs:10-45) ---- */
typedef struct { uint64_t s; } kda_rng;
void kda_rng_new(kda_rng* r, uint64_t seed);
uint64_t kda_rng_next_u64(kda_rng* r);
float kda_rng_uniform(kda_rng* r, float lo, float hi);
float kda_rng_uniform_bf16(kda_rng* r, float lo, float hi);
void kda_rng_fill(kda_rng* r, float* out, int64_t n, float lo, float hi);
void kda_rng_fill_bf16(kda_rng* r, float* out, int64_t n, float lo, float hi);
/* Standard normal by Box-Muller on two 24-bit uniforms (not in the reference: the benchmark definition's distributions). */
float kda_rng_normal(kda_rng* r);
void kda_rng_fill_normal(kda_rng* r, float* out, int64_t n);

/* synth::layer / rows / conv_window / state (src/synth.rs:49-83). */
void kda_synth_layer(int32_t heads, uint64_t seed, float* conv_w, float* a_log, float* dt_bias, float* norm_w);
void kda_synth_rows(int32_t heads, int32_t rows, uint64_t seed, float* qkv, float* a, float* b, float* gate);
void kda_synth_conv_window(int32_t heads, uint64_t seed, float* conv);
void kda_synth_state(int32_t heads, uint64_t seed, float scale, float* state);

/* ---- scalar pieces (cpu.rs:202-254) ---- */
float kda_sigmoid(float x);
float kda_silu(float x);
float kda_warp_sum(const float lanes[32]);
float kda_dot128(const float* a, const float* b);
float kda_log_decay(float a, float dt_bias, float a_log, float lower);
float kda_decay(float a, float dt_bias, float decay_rate, float lower);
float kda_beta(float b);
float kda_q_scale(void);

/* One layer's parameters (cpu.rs:82-98). */
typedef struct {
    int32_t heads;
    const float* conv_w;  /* [C][4] */
    const float* a_log;   /* [H] */
    const float* dt_bias; /* [H*DK] */
    const float* norm_w;  /* [DV] */
    float eps;
    float lower;
} kda_layer;

/* Projection rows (cpu.rs:122-135). */
typedef struct {
    int32_t heads;
    int32_t rows;
    const float* qkv;  /* [rows][C] */
    const float* a;    /* [rows][H*DK] */
    const float* b;    /* [rows][H] */
    const float* gate; /* [rows][H*DV] */
} kda_rows;

/* ---- per-row pieces (cpu.rs:256-376) ---- */
float kda_conv_channel(const kda_layer* p, const float* conv, const kda_rows* rows, int32_t r, int32_t c, int mode);
void kda_conv_qkv(const kda_layer* p, const float* conv, const kda_rows* rows, int32_t r, int32_t h, int mode,
                  float* q, float* k, float* v);
/* scale <= 0: none. */
void kda_l2norm(const float* x, float scale, float* y);
void kda_update(float* s, const float* k, const float* g, const float* v, float beta);
void kda_read_out(const float* s, const float* q, float* y);
void kda_gated_rmsnorm_as(const float* y, const float* norm_w, const float* gate, float eps, int mode, float* o);

/* ---- chain / replay / conv shift (cpu.rs:378-547) ----
 * out, y: [rows][H*DV]; state_out: [H][DV][DK]; saves (may all be NULL): k,g [rows][H][DK], v [rows][H][DV],
 * beta [rows][H]. threads > 1 runs heads in parallel (OpenMP); the arithmetic per head is unchanged. */
void kda_chain_with(const kda_layer* p, const float* conv, const float* state, const kda_rows* rows, int mode,
                    int bf16_state, float* out, float* y, float* state_out, float* k_save, float* v_save,
                    float* g_save, float* b_save, int threads);
void kda_replay_with(int32_t heads, const float* state, const float* k_save, const float* v_save,
                     const float* g_save, const float* b_save, int32_t keep, int bf16_state, float* state_out);
/* The delta rule over saved rows in f64, from an f32 state: the exact-arithmetic yardstick of the reference's
 * accuracy tests (tests/gpu_prefill.rs:502-519, tests/gpu_bf16_state.rs:660-682). Heads run in parallel. */
void kda_exact_replay(int32_t heads, const float* state, const float* k_save, const float* v_save,
                      const float* g_save, const float* b_save, int32_t rows, double* state_out, int threads);
void kda_conv_shift(int32_t heads, const float* conv, const float* qkv, int32_t rows, int32_t keep, float* out);
void kda_transpose_state(const float* s, float* t, int64_t n);

/* ---- the reference's literal formulation (cpu.rs:553-686) ---- */
void kda_literal_l2norm(const float* x, float* y);
/* s: [DK][DV]. g: log space. y: read-out before rounding. */
void kda_literal_step(float* s, const float* q, const float* k, const float* v, const float* g, float beta,
                      float* y);
void kda_literal_gated_rmsnorm_as(const float* y, const float* norm_w, const float* gate, float eps, int mode,
                                  float* o);
void kda_literal_chain(const kda_layer* p, const float* conv, const float* state, const kda_rows* rows, int mode,
                       float* out, float* y, float* state_out, float* k_save, float* v_save, float* g_save,
                       float* b_save, int threads);

/* ---- chunked (WY/UT) form (chunked.rs:67-254) ----
 * head: q,k normalized [t][DK], v [t][DV], g log decay [t][DK], beta [t], state [DK][DV] in place,
 * out [t][DV] not rounded. layer: q,k,v [t][H][128] before the norms, g [t][H][DK], beta [t][H],
 * state [H][DK][DV] in place, out [t][H][DV]. */
void kda_chunked_head(const float* q, const float* k, const float* v, const float* g, const float* beta,
                      int32_t t, float* state, int32_t chunk, float* out);
void kda_chunked_layer(int32_t heads, const float* q, const float* k, const float* v, const float* g,
                       const float* beta, int32_t t, float* state, int32_t chunk, float* out, int threads);
/* The recurrent counterpart of kda_chunked_layer: literal_step row by row on the same core-level inputs. */
void kda_recurrent_layer(int32_t heads, const float* q, const float* k, const float* v, const float* g,
                         const float* beta, int32_t t, float* state, float* out, int threads);

/* ---- the reference prefill kernel's 16-row host model (chunked.rs:256-467) ---- */
void kda_prefill_head(const float* qn, const float* kn, const float* v, const float* d, const float* beta,
                      int32_t t, float* s, float* y);
void kda_prefill(const kda_layer* p, const float* conv, const float* state, const kda_rows* rows, int mode,
                 float* out, float* y, float* state_out, int threads);

#ifdef __cplusplus
}
#endif
#endif /* KDA_REF_H */
