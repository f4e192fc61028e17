/* Row gather and scatter for MI355X (gfx950): the two entry points of the reference's forward-kernel ABI that
 * move a slot's positional state (KDA states, conv windows, tails) into and out of the pages of a snapshot
 * mark.
 *
 * Drop-in boundary: names, argument order and meaning of crates/glm53f-forward/kernels/glm53f_forward.h:75-85,
 * bound by crates/glm53f-forward/src/ffi.rs:75-96 and called by the snapshot code
 * (crates/glm53f-forward/src/kv.rs:412-478), the expert loop (src/experts.rs:278-363) and the row packing of
 * the forward (src/forward.rs:2346-2390). Only the stream handle changes: a HIP stream.
 *
 * Conventions (reference header :1-20): every pointer is a DEVICE pointer; strides and sizes count BYTES;
 * the return value is a hipError_t as int32: 0 on success, 1 (hipErrorInvalidValue) when the host rejects an
 * argument, otherwise the launch error. Launches are asynchronous on `stream` (NULL: the default stream);
 * nothing is allocated, freed or synchronized inside. `idx` is device data and is not read on the host: its
 * entries must be valid row numbers of the indexed side, and distinct for a scatter.
 */
#ifndef GLM53F_FWD_ROWS_H
#define GLM53F_FWD_ROWS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

struct ihipStream_t;

/** dst[i] = src[idx[i]] for i < rows: rows of `bytes` bytes, src rows `src_stride` bytes apart, dst rows
 *  `dst_stride` bytes apart. bytes, strides and pointers are multiples of 16; strides are at least `bytes`.
 *  rows == 0 or bytes == 0 succeeds without a launch.
 *  (reference: glm53f_forward.h:75-79, glue.cu:101-110, :221-239) */
int32_t glm53f_fwd_gather_rows(const uint8_t* src, int64_t src_stride, const int32_t* idx, uint8_t* dst,
                               int64_t dst_stride, int32_t rows, int64_t bytes, struct ihipStream_t* stream);

/** dst[idx[i]] = src[i] for i < rows (same layout rules; idx entries distinct).
 *  (reference: glm53f_forward.h:81-85, glue.cu:101-110, :241-244) */
int32_t glm53f_fwd_scatter_rows(const uint8_t* src, int64_t src_stride, const int32_t* idx, uint8_t* dst,
                                int64_t dst_stride, int32_t rows, int64_t bytes, struct ihipStream_t* stream);

#ifdef __cplusplus
}
#endif

#endif
