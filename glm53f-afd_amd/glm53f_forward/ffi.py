"""Raw bindings of the forward crate's kernels built here, one ctypes prototype per declaration of
include/glm53f_fwd_rows.h (row gather/scatter) and include/glm53f_fwd_gemv.h (the BF16 GEMV and the skinny GEMM): the counterpart of
crates/glm53f-forward/src/ffi.rs:10-40 and :75-96. Pointers are device addresses passed as integers;
the rows' strides and sizes are bytes, the GEMV's strides elements; `stream` is a hipStream_t handle (0: the default stream). The entry points live in the same
shared library as the KDA kernels.
"""
import ctypes as C

from glm53f_kda import ffi as _kda

i32, i64, ptr = C.c_int32, C.c_int64, C.c_void_p

u32 = C.c_uint32

PROTOTYPES = {
    "glm53f_fwd_gemv_bf16": (i32, [ptr, i64, i64, ptr, i64, i64, i32, i32, i32, i32, i32, ptr, ptr, ptr, i32, i64, i64, ptr]),
    "glm53f_fwd_gemv_ksplit": (i32, [i32, i32, i32]),
    "glm53f_fwd_gemv_bf16_static": (i32, [ptr, i64, i64, ptr, i64, i64, i32, i32, i32, i32, i32, ptr, i32, i64, i64, ptr]),
    "glm53f_fwd_gemm_bf16_skinny": (i32, [ptr, i64, i64, ptr, i64, i64, i32, i32, i32, i32, ptr, i32, i64, i64, ptr]),
    "glm53f_fwd_gather_rows": (i32, [ptr, i64, ptr, ptr, i64, i32, i64, ptr]),
    "glm53f_fwd_scatter_rows": (i32, [ptr, i64, ptr, ptr, i64, i32, i64, ptr]),
}

_bound = False


def lib() -> C.CDLL:
    """The loaded library with these prototypes set. Raises if it has not been built."""
    global _bound
    handle = _kda.lib()
    if not _bound:
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _bound = True
    return handle


def __getattr__(name: str):
    if name in PROTOTYPES:
        return getattr(lib(), name)
    raise AttributeError(name)
