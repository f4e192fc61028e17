// Yardstick kernels for bench.py: what this GPU moves for the memory traffic of the KDA kernels with no arithmetic
// behind it, and what one CU can stream. Not part of the product library (libglm53f_yardsticks.so is loaded by
// bench.py only); nothing here restates a reference kernel.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr int THREADS = 256, PIECES = 8;                 // 256 lanes x 8 pieces of 16 bytes: the 32 KB of a head's bf16 state

// Decode-shaped: workgroup (head, request) reads the 32 KB of its head in the request's slot and writes them back
// in place, nontemporal both ways (the chain kernel's accesses).
__global__ void __launch_bounds__(THREADS) update_in_place_kernel(u32x4* pool, const int32_t* __restrict__ slots,
                                                                 long long slot_pieces) {
    u32x4* p = pool + slots[blockIdx.y] * slot_pieces + (long long)blockIdx.x * (THREADS * PIECES) + threadIdx.x;
    u32x4 v[PIECES];
#pragma unroll
    for (int j = 0; j < PIECES; ++j) v[j] = __builtin_nontemporal_load(p + j * THREADS);
#pragma unroll
    for (int j = 0; j < PIECES; ++j) v[j] += 1u;
#pragma unroll
    for (int j = 0; j < PIECES; ++j) __builtin_nontemporal_store(v[j], p + j * THREADS);
}

// Verify-shaped: workgroup (head, slot) reads its 32 KB once and writes them to `rows` checkpoints
// ([slot][row][head][32 KB]), nontemporal.
__global__ void __launch_bounds__(THREADS) checkpoints_kernel(const u32x4* __restrict__ pool, u32x4* __restrict__ ckpt,
                                                             int rows) {
    const long long heads = gridDim.x;
    const u32x4* p = pool + ((long long)blockIdx.y * heads + blockIdx.x) * (THREADS * PIECES) + threadIdx.x;
    u32x4 v[PIECES];
#pragma unroll
    for (int j = 0; j < PIECES; ++j) v[j] = __builtin_nontemporal_load(p + j * THREADS);
    for (int r = 0; r < rows; ++r) {
        u32x4* q = ckpt + (((long long)blockIdx.y * rows + r) * heads + blockIdx.x) * (THREADS * PIECES) + threadIdx.x;
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
            v[j] += 1u;
            __builtin_nontemporal_store(v[j], q + j * THREADS);
        }
    }
}

// One workgroup per CU (100 KB of LDS asked for) streams its own region with 128-bit loads, eight in flight per
// lane. MODE 0: plain loads, 1: nontemporal, 2: agent scope (sc1).
template <int MODE>
__global__ void __launch_bounds__(THREADS) stream_read_kernel(const u32x4* __restrict__ src, long long pieces_per_wg,
                                                             int reps, unsigned* __restrict__ sink) {
    const u32x4* p = src + (long long)blockIdx.x * pieces_per_wg;
    u32x4 acc = {0u, 0u, 0u, 0u};
    for (int r = 0; r < reps; ++r)
        for (long long i = threadIdx.x; i + 7 * THREADS < pieces_per_wg; i += 8 * THREADS) {
            u32x4 v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                if constexpr (MODE == 0) v[j] = p[i + j * THREADS];
                if constexpr (MODE == 1) v[j] = __builtin_nontemporal_load(p + i + j * THREADS);
                if constexpr (MODE == 2)
                    asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(v[j]) : "v"(p + i + j * THREADS) : "memory");
            }
            // the assembly loads are the compiler's blind spot: wait for them here, before their registers are read
            if constexpr (MODE == 2) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
            for (int j = 0; j < 8; ++j) acc ^= v[j];
        }
    if (acc[0] == 0x12345u && acc[1] == 77u) sink[threadIdx.x] = acc[2] ^ acc[3];
}

}  // namespace

extern "C" int glm53f_yardstick_update_in_place(void* pool, const int32_t* slots, int64_t slot_bytes, int32_t heads,
                                                int32_t batch, hipStream_t stream) {
    if (!pool || !slots || heads < 1 || batch < 1 || slot_bytes != (int64_t)heads * THREADS * PIECES * 16) return 1;
    update_in_place_kernel<<<dim3(heads, batch), THREADS, 0, stream>>>(reinterpret_cast<u32x4*>(pool), slots,
                                                                      slot_bytes / 16);
    return (int)hipGetLastError();
}

extern "C" int glm53f_yardstick_checkpoints(const void* pool, void* ckpt, int32_t heads, int32_t slots, int32_t rows,
                                            hipStream_t stream) {
    if (!pool || !ckpt || heads < 1 || slots < 1 || rows < 1) return 1;
    checkpoints_kernel<<<dim3(heads, slots), THREADS, 0, stream>>>(reinterpret_cast<const u32x4*>(pool),
                                                                  reinterpret_cast<u32x4*>(ckpt), rows);
    return (int)hipGetLastError();
}

extern "C" int glm53f_yardstick_stream_read(const void* src, int64_t bytes_per_wg, int32_t workgroups, int32_t reps,
                                            int32_t mode, void* sink, hipStream_t stream) {
    if (!src || !sink || bytes_per_wg < 8 * THREADS * 16 || bytes_per_wg % 16 || workgroups < 1 || reps < 1) return 1;
    const size_t lds = 100 * 1024;                        // one workgroup per CU
    const u32x4* s = reinterpret_cast<const u32x4*>(src);
    unsigned* k = reinterpret_cast<unsigned*>(sink);
    hipError_t e = hipSuccess;
    if (mode == 0) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&stream_read_kernel<0>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) stream_read_kernel<0><<<workgroups, THREADS, lds, stream>>>(s, bytes_per_wg / 16, reps, k);
    } else if (mode == 1) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&stream_read_kernel<1>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) stream_read_kernel<1><<<workgroups, THREADS, lds, stream>>>(s, bytes_per_wg / 16, reps, k);
    } else if (mode == 2) {
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&stream_read_kernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e == hipSuccess) stream_read_kernel<2><<<workgroups, THREADS, lds, stream>>>(s, bytes_per_wg / 16, reps, k);
    } else {
        return 1;
    }
    if (e != hipSuccess) return (int)e;
    return (int)hipGetLastError();
}
