/* BF16 weight GEMV for MI355X (gfx950): the projections of a decode or verify step (1 to 8 rows), streamed from
 * HBM once.
 *
 * Drop-in boundary: names, argument order and meaning of crates/glm53f-forward/kernels/glm53f_forward.h:19-47,
 * bound by crates/glm53f-forward/src/ffi.rs:10-40 and called by crates/glm53f-forward/src/gemm.rs:238-291
 * (`Gemm::gemv`; the KDA projections of forward.rs:3494-3542 reach it through `Gemm::bf16`). Only the stream handle
 * changes: a HIP stream.
 *
 * Conventions (reference header :4-10): device pointers; strides in ELEMENTS; the return value is a hipError_t as
 * int32: 0 on success, 1 (hipErrorInvalidValue) when the host rejects an argument, otherwise the launch error.
 * Asynchronous on `stream`; nothing is allocated, freed or synchronized inside.
 *
 * Numerics (reference header :24-31, host model crates/glm53f-forward/src/reference.rs:27-71): for every K split,
 * 32 partial sums per output: partial l accumulates fma(x[k], w[k], acc) over k = lo + 8 l + 256 i + j (i outer,
 * j = 0..7); the 32 partials are added by an xor butterfly over offsets 16, 8, 4, 2, 1; the splits are added in
 * split order; the result is stored as f32 or rounded to bf16 (nearest even). A row's result depends on that row's
 * inputs and on (n, k, ksplit) only, never on `rows`: a verify window gives the bits of serial decode steps.
 */
#ifndef GLM53F_FWD_GEMV_H
#define GLM53F_FWD_GEMV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

struct ihipStream_t;

/** out[g][m][o] = sum_k x[g][m][k] * w[g][o][k] for g < groups, m < rows (1..8), o < n: x at
 *  x + g*x_gstride + m*ldx, w row o at w + g*w_gstride + o*ldw, out at out + g*o_gstride + m*ldo (bf16, or f32
 *  when out_f32 != 0). n % 8 == 0, k % 8 == 0, ldx, ldw, x_gstride, w_gstride % 8 == 0, x and w 16-byte aligned;
 *  ksplit divides k and every split is a multiple of 8 wide (use glm53f_fwd_gemv_ksplit). ksplit > 1 needs
 *  `partials` (f32 [groups][ksplit][rows][n]) and `sync` (at least groups * n / 8 zeroed counters, left zeroed).
 *  (reference: glm53f_forward.h:21-41, gemv_bf16.cu:29-139, :154-170) */
int32_t glm53f_fwd_gemv_bf16(const uint16_t* x, int64_t ldx, int64_t x_gstride, const uint16_t* w, int64_t ldw,
                             int64_t w_gstride, int32_t groups, int32_t rows, int32_t n, int32_t k, int32_t ksplit,
                             float* partials, uint32_t* sync, void* out, int32_t out_f32, int64_t ldo,
                             int64_t o_gstride, struct ihipStream_t* stream);

/** The K splits the GEMV uses for an [n][k] weight in `groups` groups: the fewest splits, each at least 1,024 wide
 *  and a multiple of 256, that give at least 512 blocks of 8 outputs. Shape only; part of the numerical contract.
 *  (reference: glm53f_forward.h:43-45, gemv_bf16.cu:141-152) */
int32_t glm53f_fwd_gemv_ksplit(int32_t groups, int32_t n, int32_t k);

/** glm53f_fwd_gemv_bf16 for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 *  harnesses that forbid hipMalloc): the same arguments without `partials` and `sync`, which live in an array the
 *  library holds on every GPU it runs on (1 MiB of partial sums and 4,096 counters, until the process ends). The
 *  same kernels, the same bits. It has no counterpart in the reference, whose callers bring their own scratch.
 *  With ksplit > 1 the call is rejected (1) when groups * ksplit * rows * n > 262,144 partial sums or
 *  groups * n / 8 > 4,096 counters; with ksplit == 1 the array is not touched. Calls no hipMalloc, hipFree or
 *  other allocating routine; the first call on a device looks the array's address up (make it before a capture).
 *  Every call on a GPU shares that GPU's array: the counters a call uses are cleared by a kernel on `stream` before
 *  its launch, and calls that overlap on one GPU (two streams, two threads) race. */
int32_t glm53f_fwd_gemv_bf16_static(const uint16_t* x, int64_t ldx, int64_t x_gstride, const uint16_t* w,
                                    int64_t ldw, int64_t w_gstride, int32_t groups, int32_t rows, int32_t n,
                                    int32_t k, int32_t ksplit, void* out, int32_t out_f32, int64_t ldo,
                                    int64_t o_gstride, struct ihipStream_t* stream);

/** out[g][m][o] = sum_k x[g][m][k] * w[g][o][k] for 9 to 64 rows (1 to 64 are accepted), with the weights streamed
 *  from HBM once like the GEMV's and the arithmetic on the matrix cores (v_mfma_f32_16x16x32_bf16). It has no
 *  counterpart in the reference's kernel ABI: above 8 rows the reference's engine calls the vendor GEMM
 *  (crates/glm53f-forward/src/gemm.rs:228-234, `Gemm::cublas` :293-325); this is what `Gemm::bf16` can call in
 *  its place for up to 64 rows (a decode step of 9 to 64 slots, a verify window), where the vendor's tiles leave
 *  close to half of the weight stream's rate unused (4096 -> 24,640 with sixteen rows: 52 us there, 31 us here). Arguments as glm53f_fwd_gemv_bf16 without the split and its scratch.
 *  n % 16 == 0, k % 128 == 0, ldx, ldw, x_gstride, w_gstride % 8 == 0, x and w 16-byte aligned, out 4-byte aligned,
 *  ldo and o_gstride even for bf16 outputs; anything else is rejected (1) and belongs to the vendor GEMM.
 *  Numerics: exact bf16 products, f32 accumulation over K in steps of 32 inside eighths or quarters of the K range
 *  (or the whole of it; n and k alone decide), those added in order; bf16 outputs rounded to nearest even. Results do not depend on `rows` beyond the row's own
 *  inputs; there is no bit-level contract with the GEMV (the reference has none between its GEMV and cuBLAS:
 *  tests/gemv.rs holds the two together within f32 rounding, and tests/test_gpu_gemm_skinny.py does the same). */
int32_t glm53f_fwd_gemm_bf16_skinny(const uint16_t* x, int64_t ldx, int64_t x_gstride, const uint16_t* w, int64_t ldw,
                                    int64_t w_gstride, int32_t groups, int32_t rows, int32_t n, int32_t k, void* out,
                                    int32_t out_f32, int64_t ldo, int64_t o_gstride, struct ihipStream_t* stream);

#ifdef __cplusplus
}
#endif

#endif
