/* glm53f-kda for MI355X (gfx950): the C ABI of the Kimi delta attention (KDA) hot path.
 *
 * Drop-in boundary: the 13 entry points below have the names, argument order and meaning of the
 * reference's crates/glm53f-kda/kernels/glm53f_kda.h:73-270, which its Rust bindings mirror in
 * crates/glm53f-kda/src/ffi.rs:16-287 and which crates/glm53f-forward calls directly
 * (src/forward.rs:1980-2039, :3585-3760). Only the stream handle changes: a HIP stream.
 * More entry points (end of this file) have no counterpart in the reference: the speculative-verify step
 * with per-position state checkpoints (the reference's rollback recomputes from saved rows) and the decode
 * round in one launch.
 *
 * Conventions (reference header :5-9): every pointer is a DEVICE pointer; strides and offsets count
 * ELEMENTS, not bytes; the return value is a hipError_t as int: 0 on success, 1 (hipErrorInvalidValue)
 * when the host rejects an argument, otherwise the launch error. Launches are asynchronous on `stream`
 * (NULL: the default stream). Nothing is allocated, freed or synchronized inside; device metadata arrays
 * (cu_rows, keep, *_off) are not read on the host.
 *
 * Geometry: DK = DV = 128, 4 conv taps, H >= 1 heads (64 in GLM-5.3-Flash), C = 3*H*128 conv channels
 * laid out q | k | v.
 *
 * Layouts in HBM (row major, elements):
 *   state        f32 or bf16 [H][128 value][128 key]; value-row major, the transpose per head of the
 *                model's [H][K][V]. One head is 64 KiB in f32, 32 KiB in bf16; a layer of 64 heads is
 *                4 MiB / 2 MiB per slot. Kernels move it with 128-bit accesses, one 256- or 512-byte
 *                value row per 16 or 32 lanes.
 *   conv window  bf16 [3][C]: the q|k|v projection rows of the three positions before the first row,
 *                oldest first.
 *   conv weight  bf16 [C][4]; tap 3 multiplies the current row.
 *   replay saves per global row r and head h: normalized k (f32) and the decay multipliers exp(g) (f32)
 *                at (r*H + h)*128, v (bf16) at the same index, beta (f32) at r*H + h.
 *   checkpoints  bf16 [rows][H][128][128]: the state after global row r at r*H*16384.
 *
 * Numerics (the reference's contract, header :26-32): conv + SiLU in f32 with one bf16 rounding; q and k
 * L2-normalized in f32 (eps 1e-6 inside the sum, q also times 128^-0.5); per-channel decay
 * exp(lower * sigmoid(exp(A_log) * (a + dt_bias))); beta = bf16(sigmoid(b)); the delta rule in f32 with no
 * fused multiply-add; the read-out rounded to bf16; gated RMSNorm
 * bf16(w * (y / sqrt(mean(y^2) + eps)) * sigmoid(gate)). The state update is one routine shared by the
 * chain, the replays and the verify step, so a replayed or checkpointed prefix of a window has the bits
 * of serial single-row steps. Its 128-term sums run in the order of the reference's CPU model
 * (crates/glm53f-kda/src/cpu.rs:229-239, :324-344): 32 partial sums of 4 consecutive products, then an
 * xor butterfly over offsets 16, 8, 4, 2, 1.
 */
#ifndef GLM53F_KDA_H
#define GLM53F_KDA_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

struct ihipStream_t;
/** Same type as hipStream_t. NULL is the default stream. (reference header :43-45, CUDA stream there) */
typedef struct ihipStream_t* glm53f_stream_t;
/** Raw bfloat16 bits. */
typedef uint16_t glm53f_bf16;

#define GLM53F_KDA_DK 128
#define GLM53F_KDA_DV 128
#define GLM53F_KDA_TAPS 4
/** Rows per chunk of the chunked prefill on this build (the reference's kernel uses 16). */
#define GLM53F_KDA_PREFILL_CHUNK 64

/**
 * One layer, one request, `rows` >= 1 consecutive rows from the committed state. Replaces the
 * reference's glm53f_kda_chain (header :73-83, kda.cu:303-318).
 *
 * p, p_stride   bf16 projection rows: row r has q|k|v in [0, C) of p + r*p_stride and the H beta
 *               logits (before the sigmoid) in [b_off, b_off + H); b_off may be negative.
 * a, a_stride   bf16 forget-gate rows, [H*128] each, before dt_bias.
 * g, g_stride   bf16 output-gate rows, [H*128] each.
 * conv          bf16 conv window [3][C], read only. conv_w: bf16 [C][4].
 * state_in      f32 [H][128][128]. state_out: the state after the last row; NULL (not written) or equal
 *               to state_in (in place) or disjoint from it.
 * a_log f32 [H]; dt_bias f32 [H*128]; norm_w bf16 [128]; eps of the gated RMSNorm; lower: the gate's
 * lower bound (-5).
 * out           bf16 rows of [H*128] at out + r*out_stride.
 * k_save, v_save, g_save, b_save: replay inputs of rows 0..rows-1, all NULL or all set.
 */
int glm53f_kda_chain(int32_t heads, int32_t rows, const glm53f_bf16* p, int64_t p_stride, int64_t b_off,
    const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g, int64_t g_stride, const glm53f_bf16* conv,
    const glm53f_bf16* conv_w, const float* state_in, float* state_out, const float* a_log,
    const float* dt_bias, const glm53f_bf16* norm_w, float eps, float lower, glm53f_bf16* out,
    int64_t out_stride, float* k_save, glm53f_bf16* v_save, float* g_save, float* b_save,
    glm53f_stream_t stream);

/**
 * One layer, `batch` requests; workgroup (h, b) runs head h of request b. Replaces
 * glm53f_kda_chain_batch (header :97-108, kda.cu:343-354).
 *
 * cu_rows    device int32 [batch+1], non-decreasing: request b owns global rows
 *            [cu_rows[b], cu_rows[b+1]) of p, a, g, out and the saves. Zero rows: its state is copied.
 * conv_off   device int64 [batch]: request b's window is conv + conv_off[b].
 * state_off  device int64 [batch]: request b's state is state_in + state_off[b], written to
 *            state_out + state_off[b]. Regions of different requests must not overlap.
 */
int glm53f_kda_chain_batch(int32_t heads, int32_t batch, const int32_t* cu_rows, const glm53f_bf16* p,
    int64_t p_stride, int64_t b_off, const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g,
    int64_t g_stride, const glm53f_bf16* conv, const int64_t* conv_off, const glm53f_bf16* conv_w,
    const float* state_in, float* state_out, const int64_t* state_off, const float* a_log, const float* dt_bias,
    const glm53f_bf16* norm_w, float eps, float lower, glm53f_bf16* out, int64_t out_stride, float* k_save,
    glm53f_bf16* v_save, float* g_save, float* b_save, glm53f_stream_t stream);

/**
 * glm53f_kda_chain_batch with bf16 states (state_in, state_out, state_off in bf16 elements): f32
 * arithmetic on the widened state, rounded to bf16 after every row, after that row's read-out, so a window
 * of R rows has the bits of R serial single-row calls. The decode step. Replaces
 * glm53f_kda_chain_batch_bf16state (header :118-130, kda.cu:356-371).
 */
int glm53f_kda_chain_batch_bf16state(int32_t heads, int32_t batch, const int32_t* cu_rows, const glm53f_bf16* p,
    int64_t p_stride, int64_t b_off, const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g,
    int64_t g_stride, const glm53f_bf16* conv, const int64_t* conv_off, const glm53f_bf16* conv_w,
    const glm53f_bf16* state_in, glm53f_bf16* state_out, const int64_t* state_off, const float* a_log,
    const float* dt_bias, const glm53f_bf16* norm_w, float eps, float lower, glm53f_bf16* out,
    int64_t out_stride, float* k_save, glm53f_bf16* v_save, float* g_save, float* b_save,
    glm53f_stream_t stream);

/**
 * The state after the first `rows` >= 0 saved rows of a chain (0 copies). state_out may equal state_in.
 * Replaces glm53f_kda_replay (header :136-138, kda.cu:392-397).
 */
int glm53f_kda_replay(int32_t heads, int32_t rows, const float* state_in, float* state_out, const float* k_save,
    const glm53f_bf16* v_save, const float* g_save, const float* b_save, glm53f_stream_t stream);

/**
 * Every layer of one request: layer l's state at state_in/state_out + l*state_stride, its saves at
 * k_save/v_save/g_save + l*kv_stride and b_save + l*b_stride. Replaces glm53f_kda_replay_layers
 * (header :144-148, kda.cu:399-405).
 */
int glm53f_kda_replay_layers(int32_t heads, int32_t layers, int32_t rows, const float* state_in,
    float* state_out, int64_t state_stride, const float* k_save, const glm53f_bf16* v_save, const float* g_save,
    const float* b_save, int64_t kv_stride, int64_t b_stride, glm53f_stream_t stream);

/**
 * Every layer of every request (the commit after a verify round): workgroup (l*H + h, b) replays keep[b]
 * rows of request b from its global row cu_rows[b], from state_in + l*state_stride + state_off[b] into
 * state_out + the same offset. keep: device int32 [batch], 0 <= keep[b] <= rows of b. Replaces
 * glm53f_kda_replay_batch (header :157-163, kda.cu:407-415).
 */
int glm53f_kda_replay_batch(int32_t heads, int32_t layers, int32_t batch, const int32_t* cu_rows,
    const int32_t* keep, const float* state_in, float* state_out, int64_t state_stride,
    const int64_t* state_off, const float* k_save, const glm53f_bf16* v_save, const float* g_save,
    const float* b_save, int64_t kv_stride, int64_t b_stride, glm53f_stream_t stream);

/**
 * glm53f_kda_replay_batch with bf16 states, rounded after every replayed row: keeping k rows gives the
 * bits of k serial single-row calls. Replaces glm53f_kda_replay_batch_bf16state (header :170-176,
 * kda.cu:417-427).
 */
int glm53f_kda_replay_batch_bf16state(int32_t heads, int32_t layers, int32_t batch, const int32_t* cu_rows,
    const int32_t* keep, const glm53f_bf16* state_in, glm53f_bf16* state_out, int64_t state_stride,
    const int64_t* state_off, const float* k_save, const glm53f_bf16* v_save, const float* g_save,
    const float* b_save, int64_t kv_stride, int64_t b_stride, glm53f_stream_t stream);

/**
 * Advance a conv window past `keep` >= 0 kept rows, in place: window row j becomes row keep + j of
 * [window; new rows], new row r being [0, channels) of p + r*p_stride. Replaces glm53f_kda_conv_shift
 * (header :183-184, kda.cu:448-451).
 */
int glm53f_kda_conv_shift(int32_t channels, int32_t keep, glm53f_bf16* conv, const glm53f_bf16* p,
    int64_t p_stride, glm53f_stream_t stream);

/**
 * glm53f_kda_conv_shift for every layer of every request: the window of (l, b) is
 * conv + l*conv_stride + conv_off[b]; its new rows start at p + l*p_layer_stride + cu_rows[b]*p_stride; it
 * keeps keep[b] rows. Replaces glm53f_kda_conv_shift_batch (header :191-195, kda.cu:453-460).
 */
int glm53f_kda_conv_shift_batch(int32_t channels, int32_t layers, int32_t batch, const int32_t* cu_rows,
    const int32_t* keep, glm53f_bf16* conv, int64_t conv_stride, const int64_t* conv_off, const glm53f_bf16* p,
    int64_t p_layer_stride, int64_t p_stride, glm53f_stream_t stream);

/**
 * Bytes of workspace for the prefill to run `rows_per_pass` rows of every request per pass; 0 on bad
 * arguments. On this build a chunk is 64 rows and costs 148,096 bytes per head and request (every operand of the
 * state-carrying pass as a pair of fp16 planes, and 128 bytes of per-chunk scale bookkeeping). Replaces glm53f_kda_prefill_workspace_bytes (header :204,
 * kda_prefill.cu:695-698; 34,816 bytes per 16 rows there).
 */
int64_t glm53f_kda_prefill_workspace_bytes(int32_t heads, int32_t batch, int32_t rows_per_pass);

/**
 * Chunked prefill: one layer, one request, `rows` >= 0 rows from the committed state and conv window,
 * through the chunked (WY/UT) form of the delta rule on the matrix cores. Inputs and outputs as
 * glm53f_kda_chain without replay inputs; the conv window is advanced past the rows in place.
 * state_out must not be NULL (it may equal state_in). lower must lie in [-5.8, 0].
 * value_blocks: 0, 1, 2 or 4 are accepted as the reference accepts them (anything else is rejected) and have no
 * effect: this build always runs four workgroups of 32 value columns per head in the state-carrying pass.
 * workspace: at least glm53f_kda_prefill_workspace_bytes(heads, 1, 64) bytes; its size bounds the rows per
 * pass (the library may use less of it: passes are cut to what the 256 MB cache behind the L2 holds).
 * Numerics: every matrix-core operand is a pair of fp16 values (22 significant bits), accumulation is f32.
 * Against the chain: f32 states agree to about 1e-6 normwise (1e-4 where decay is slow enough that thousands of
 * rows are remembered) and about 0.05 % of the bf16 outputs fall on the other side of a rounding boundary; not bit
 * for bit. Results do not depend on the workspace size or on how requests are batched.
 * Domain: the state, V - Kd S and V' pass through fp16 pairs times a power of two that the state-carrying pass
 * chooses per chunk from a bound on everything the chunk can produce (the largest entry of the state that entered
 * the chunk before, and the largest |v| of both chunks), so states from 2^-39 to 2^61 in magnitude come out with the
 * same relative accuracy and a finite state stays finite, as in the f32 recurrence and in glm53f_kda_chain. One scale
 * per chunk spans 2^40 below the chunk's bound: when a state collapses by more than 2^25 inside one chunk (every
 * channel decaying by half every few rows, from a state that large against its values), the read-outs of the rows
 * that lie further below the bound than that lose their accuracy, and so do, for the one chunk that follows, values
 * more than 2^40 below the old bound. A non-finite state stays non-finite. The device arrays are not inspected on
 * the host.
 * The first call on a device also sets two kernel attributes (LDS above 64 KiB) under a lock; make one call on
 * each device before capturing a stream. Replaces glm53f_kda_prefill (header :223-232, kda_prefill.cu:700-710).
 */
int glm53f_kda_prefill(int32_t heads, int32_t rows, const glm53f_bf16* p, int64_t p_stride, int64_t b_off,
    const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g, int64_t g_stride, glm53f_bf16* conv,
    const glm53f_bf16* conv_w, const float* state_in, float* state_out, const float* a_log,
    const float* dt_bias, const glm53f_bf16* norm_w, float eps, float lower, glm53f_bf16* out,
    int64_t out_stride, int32_t value_blocks, float* workspace, int64_t workspace_bytes,
    glm53f_stream_t stream);

/**
 * glm53f_kda_prefill for a batch of requests with their own row ranges, states and conv windows.
 * max_rows (host) >= the longest request's rows. Windows and states of different requests must not
 * overlap. Replaces glm53f_kda_prefill_batch (header :240-250, kda_prefill.cu:712-725).
 */
int glm53f_kda_prefill_batch(int32_t heads, int32_t batch, const int32_t* cu_rows, int32_t max_rows,
    const glm53f_bf16* p, int64_t p_stride, int64_t b_off, const glm53f_bf16* a, int64_t a_stride,
    const glm53f_bf16* g, int64_t g_stride, glm53f_bf16* conv, const int64_t* conv_off,
    const glm53f_bf16* conv_w, const float* state_in, float* state_out, const int64_t* state_off,
    const float* a_log, const float* dt_bias, const glm53f_bf16* norm_w, float eps, float lower,
    glm53f_bf16* out, int64_t out_stride, int32_t value_blocks, float* workspace, int64_t workspace_bytes,
    glm53f_stream_t stream);

/**
 * glm53f_kda_prefill_batch with bf16 states in the pool. The state is carried in f32 accumulators across a
 * chunk of 64 rows and rounded to bf16 at the end of every chunk (chunks count from each request's first row),
 * so the results still do not depend on the workspace size. Replaces glm53f_kda_prefill_batch_bf16state (header :260-270,
 * kda_prefill.cu:727-742).
 */
int glm53f_kda_prefill_batch_bf16state(int32_t heads, int32_t batch, const int32_t* cu_rows, int32_t max_rows,
    const glm53f_bf16* p, int64_t p_stride, int64_t b_off, const glm53f_bf16* a, int64_t a_stride,
    const glm53f_bf16* g, int64_t g_stride, glm53f_bf16* conv, const int64_t* conv_off,
    const glm53f_bf16* conv_w, const glm53f_bf16* state_in, glm53f_bf16* state_out, const int64_t* state_off,
    const float* a_log, const float* dt_bias, const glm53f_bf16* norm_w, float eps, float lower,
    glm53f_bf16* out, int64_t out_stride, int32_t value_blocks, float* workspace, int64_t workspace_bytes,
    glm53f_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * Speculative verify with per-position state checkpoints. No counterpart in the reference: there a
 * verify round saves per-row inputs and the commit recomputes the kept prefix (the replay entry points
 * above, which stay available). Here the verify step also stores the state after every draft row, and the
 * commit selects one checkpoint per request.
 * ------------------------------------------------------------------------------------------------ */

/**
 * glm53f_kda_chain_batch_bf16state that leaves the pool state untouched and writes the bf16 state after
 * every row to `ckpt` (global row r at ckpt + r*H*16384). A checkpoint holds exactly the bits the chain
 * would have stored had the window ended at that row. The replay inputs may be NULL or all set.
 */
int glm53f_kda_verify_batch_bf16state(int32_t heads, int32_t batch, const int32_t* cu_rows,
    const glm53f_bf16* p, int64_t p_stride, int64_t b_off, const glm53f_bf16* a, int64_t a_stride,
    const glm53f_bf16* g, int64_t g_stride, const glm53f_bf16* conv, const int64_t* conv_off,
    const glm53f_bf16* conv_w, const glm53f_bf16* state_in, const int64_t* state_off, const float* a_log,
    const float* dt_bias, const glm53f_bf16* norm_w, float eps, float lower, glm53f_bf16* out,
    int64_t out_stride, glm53f_bf16* ckpt, float* k_save, glm53f_bf16* v_save, float* g_save, float* b_save,
    glm53f_stream_t stream);

/**
 * The commit by selection, every layer of every request: for keep[b] >= 1 the checkpoint of global row
 * cu_rows[b] + keep[b] - 1 of layer l (at ckpt + l*ckpt_layer_stride) is copied to
 * state + l*state_stride + state_off[b]; keep[b] == 0 leaves that state as it is. A pure copy: bit-exact.
 */
int glm53f_kda_select_batch_bf16state(int32_t heads, int32_t layers, int32_t batch, const int32_t* cu_rows,
    const int32_t* keep, const glm53f_bf16* ckpt, int64_t ckpt_layer_stride, glm53f_bf16* state,
    int64_t state_stride, const int64_t* state_off, glm53f_stream_t stream);

/* ------------------------------------------------------------------------------------------------
 * A decode round in one launch. No counterpart in the reference, whose engine runs the chain and then
 * glm53f_kda_conv_shift_batch with keep = rows for every layer (crates/glm53f-forward/src/forward.rs:3669-3760);
 * a single decode row's chain takes 15 us here and the shift's launch adds 4 us to it.
 * ------------------------------------------------------------------------------------------------ */

/**
 * glm53f_kda_chain_batch followed by the advance of every request's conv window past all of its rows (the
 * result of glm53f_kda_conv_shift_batch with keep[b] = rows of b, bit for bit), in the same launch. `conv` is
 * written: the windows of different requests must not overlap. A request without rows keeps its window.
 * Not for a verify round, whose windows must wait for the commit.
 */
int glm53f_kda_chain_shift_batch(int32_t heads, int32_t batch, const int32_t* cu_rows, const glm53f_bf16* p,
    int64_t p_stride, int64_t b_off, const glm53f_bf16* a, int64_t a_stride, const glm53f_bf16* g,
    int64_t g_stride, glm53f_bf16* conv, const int64_t* conv_off, const glm53f_bf16* conv_w,
    const float* state_in, float* state_out, const int64_t* state_off, const float* a_log, const float* dt_bias,
    const glm53f_bf16* norm_w, float eps, float lower, glm53f_bf16* out, int64_t out_stride, float* k_save,
    glm53f_bf16* v_save, float* g_save, float* b_save, glm53f_stream_t stream);

/** glm53f_kda_chain_shift_batch with bf16 states in the pool (as glm53f_kda_chain_batch_bf16state). */
int glm53f_kda_chain_shift_batch_bf16state(int32_t heads, int32_t batch, const int32_t* cu_rows,
    const glm53f_bf16* p, int64_t p_stride, int64_t b_off, const glm53f_bf16* a, int64_t a_stride,
    const glm53f_bf16* g, int64_t g_stride, glm53f_bf16* conv, const int64_t* conv_off,
    const glm53f_bf16* conv_w, const glm53f_bf16* state_in, glm53f_bf16* state_out, const int64_t* state_off,
    const float* a_log, const float* dt_bias, const glm53f_bf16* norm_w, float eps, float lower,
    glm53f_bf16* out, int64_t out_stride, float* k_save, glm53f_bf16* v_save, float* g_save, float* b_save,
    glm53f_stream_t stream);

/** The gfx architecture the kernels were compiled for ("gfx950"). */
const char* glm53f_kda_arch(void);

/**
 * Per-device set-up of the current device, once: the prefill kernels ask for more than 64 KiB of LDS, which is an
 * attribute of each device's copy of a kernel. Every prefill entry point does the same on its first call on a
 * device (under a lock), so calling this is only needed where that first call would come at a bad time: inside a
 * stream capture, or from two host threads that must not wait for each other. Launches nothing, allocates nothing;
 * returns 0 or the runtime's error code. No counterpart in the reference (its kernels stay under 48 KiB of shared
 * memory).
 */
int glm53f_kda_init(void);

#ifdef __cplusplus
}
#endif

#endif /* GLM53F_KDA_H */
