// Row gather and scatter (gfx950): pure data movement in 128-bit pieces, bit-exact by construction.
// Reference: crates/glm53f-forward/kernels/glue.cu:101-110 (one 128-thread block per row) and :221-244 (the
// argument checks). Here a long row (a 386 KiB page of a snapshot mark) is split over many workgroups so that a
// mark of a few hundred pages fills all 256 CUs, and short rows (expert and packing gathers) share a workgroup.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "glm53f_fwd_rows.h"

namespace fwd_rows {
namespace {

constexpr int kInvalid = 1;                       // hipErrorInvalidValue
constexpr int THREADS = 256;
constexpr int UNROLL = 8;                         // 128-bit pieces in flight per lane of the long-row kernel
constexpr int SPAN = THREADS * UNROLL;            // pieces of one row per workgroup: 32 KiB
constexpr long long LONG_ROW = 1024;              // rows of at least this many pieces (16 KiB) take that kernel

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Workgroup x moves pieces [SPAN * (x % bpr), ...) of row x / bpr. The pieces stream through once, so they
// are loaded and stored nontemporal: a mark of 70 to 140 MiB would otherwise evict everything else cached.
__global__ void __launch_bounds__(THREADS) long_rows_kernel(const uint8_t* __restrict__ src, long long src_stride,
                                                            const int32_t* __restrict__ idx,
                                                            uint8_t* __restrict__ dst, long long dst_stride,
                                                            long long chunks, unsigned bpr, int scatter) {
    const unsigned i = blockIdx.x / bpr, part = blockIdx.x % bpr;
    const long long other = idx[i];
    const long long s_row = scatter ? (long long)i : other, d_row = scatter ? other : (long long)i;
    const u32x4* s = reinterpret_cast<const u32x4*>(src + s_row * src_stride);
    u32x4* d = reinterpret_cast<u32x4*>(dst + d_row * dst_stride);
    const long long c0 = (long long)part * SPAN + threadIdx.x;
    u32x4 x[UNROLL];
    if (c0 + (long long)(UNROLL - 1) * THREADS < chunks) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) x[u] = __builtin_nontemporal_load(s + c0 + u * THREADS);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) __builtin_nontemporal_store(x[u], d + c0 + u * THREADS);
    } else {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            if (c0 + u * THREADS < chunks) x[u] = __builtin_nontemporal_load(s + c0 + u * THREADS);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
            if (c0 + u * THREADS < chunks) __builtin_nontemporal_store(x[u], d + c0 + u * THREADS);
    }
}

// 2^shift lanes per row (the smallest power of two that covers the row's pieces, 256 at most), 256 >> shift rows
// per workgroup. Plain loads and stores: what these rows feed usually runs next and finds them in the cache.
__global__ void __launch_bounds__(THREADS) short_rows_kernel(const uint8_t* __restrict__ src, long long src_stride,
                                                             const int32_t* __restrict__ idx,
                                                             uint8_t* __restrict__ dst, long long dst_stride,
                                                             int chunks, int rows, int shift) {
    const long long i = ((long long)blockIdx.x << (8 - shift)) + (threadIdx.x >> shift);
    if (i >= rows) return;
    const int lanes = 1 << shift, c0 = threadIdx.x & (lanes - 1);
    const long long other = idx[i];
    const uint4* s = reinterpret_cast<const uint4*>(src + other * src_stride);
    uint4* d = reinterpret_cast<uint4*>(dst + i * dst_stride);
    for (int c = c0; c < chunks; c += lanes) d[c] = s[c];
}

__global__ void __launch_bounds__(THREADS) short_rows_scatter_kernel(const uint8_t* __restrict__ src,
                                                                     long long src_stride,
                                                                     const int32_t* __restrict__ idx,
                                                                     uint8_t* __restrict__ dst, long long dst_stride,
                                                                     int chunks, int rows, int shift) {
    const long long i = ((long long)blockIdx.x << (8 - shift)) + (threadIdx.x >> shift);
    if (i >= rows) return;
    const int lanes = 1 << shift, c0 = threadIdx.x & (lanes - 1);
    const long long other = idx[i];
    const uint4* s = reinterpret_cast<const uint4*>(src + i * src_stride);
    uint4* d = reinterpret_cast<uint4*>(dst + other * dst_stride);
    for (int c = c0; c < chunks; c += lanes) d[c] = s[c];
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// The reference's checks in the reference's order (glue.cu:221-233): sizes first, then the empty case, then
// the pointers.
int32_t gather_scatter(const uint8_t* src, int64_t src_stride, const int32_t* idx, uint8_t* dst, int64_t dst_stride,
                       int32_t rows, int64_t bytes, int scatter, hipStream_t stream) {
    if (rows < 0 || bytes < 0 || bytes % 16 || src_stride % 16 || dst_stride % 16 || src_stride < bytes ||
        dst_stride < bytes)
        return kInvalid;
    if (rows == 0 || bytes == 0) return 0;
    if (!src || !dst || !aligned16(src) || !aligned16(dst) || !idx) return kInvalid;
    const long long chunks = bytes / 16;
    if (chunks >= LONG_ROW) {
        const long long bpr = (chunks + SPAN - 1) / SPAN;
        if (bpr * rows > 0x7fffffffLL) return kInvalid;       // more workgroups than one launch takes
        long_rows_kernel<<<dim3((unsigned)(bpr * rows)), THREADS, 0, stream>>>(src, src_stride, idx, dst, dst_stride,
                                                                               chunks, (unsigned)bpr, scatter);
    } else {
        int shift = 0;
        while ((1 << shift) < chunks && shift < 8) ++shift;
        const int rows_per_block = THREADS >> shift;
        const unsigned blocks = (unsigned)(((long long)rows + rows_per_block - 1) / rows_per_block);
        if (scatter)
            short_rows_scatter_kernel<<<dim3(blocks), THREADS, 0, stream>>>(src, src_stride, idx, dst, dst_stride,
                                                                            (int)chunks, rows, shift);
        else
            short_rows_kernel<<<dim3(blocks), THREADS, 0, stream>>>(src, src_stride, idx, dst, dst_stride,
                                                                    (int)chunks, rows, shift);
    }
    return (int32_t)hipGetLastError();
}

}  // namespace
}  // namespace fwd_rows

extern "C" int32_t glm53f_fwd_gather_rows(const uint8_t* src, int64_t src_stride, const int32_t* idx, uint8_t* dst,
                                          int64_t dst_stride, int32_t rows, int64_t bytes, ihipStream_t* stream) {
    return fwd_rows::gather_scatter(src, src_stride, idx, dst, dst_stride, rows, bytes, 0, stream);
}

extern "C" int32_t glm53f_fwd_scatter_rows(const uint8_t* src, int64_t src_stride, const int32_t* idx, uint8_t* dst,
                                           int64_t dst_stride, int32_t rows, int64_t bytes, ihipStream_t* stream) {
    return fwd_rows::gather_scatter(src, src_stride, idx, dst, dst_stride, rows, bytes, 1, stream);
}
