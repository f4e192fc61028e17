"""Raw bindings of the C ABI, one ctypes prototype per declaration of include/glm53f_kda.h
(the counterpart of crates/glm53f-kda/src/ffi.rs:16-287). Pointers are device addresses passed as
integers; `stream` is a hipStream_t handle (0: the default stream).
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("GLM53F_KDA_LIB") or os.path.join(os.path.dirname(_HERE), "csrc", "libglm53f_kda.so")

i32, i64, f32, ptr = C.c_int32, C.c_int64, C.c_float, C.c_void_p

_ROWS = [ptr, i64, i64, ptr, i64, ptr, i64]              # p, p_stride, b_off, a, a_stride, g, g_stride
_WEIGHTS = [ptr, ptr, ptr, f32, f32]                     # a_log, dt_bias, norm_w, eps, lower
_SAVES = [ptr, ptr, ptr, ptr]                            # k_save, v_save, g_save, b_save

PROTOTYPES = {
    "glm53f_kda_chain": (C.c_int, [i32, i32] + _ROWS + [ptr, ptr, ptr, ptr] + _WEIGHTS + [ptr, i64] + _SAVES + [ptr]),
    "glm53f_kda_chain_batch": (C.c_int, [i32, i32, ptr] + _ROWS + [ptr, ptr, ptr, ptr, ptr, ptr] + _WEIGHTS
                               + [ptr, i64] + _SAVES + [ptr]),
    "glm53f_kda_chain_batch_bf16state": (C.c_int, [i32, i32, ptr] + _ROWS + [ptr, ptr, ptr, ptr, ptr, ptr] + _WEIGHTS
                                         + [ptr, i64] + _SAVES + [ptr]),
    "glm53f_kda_replay": (C.c_int, [i32, i32, ptr, ptr] + _SAVES + [ptr]),
    "glm53f_kda_replay_layers": (C.c_int, [i32, i32, i32, ptr, ptr, i64] + _SAVES + [i64, i64, ptr]),
    "glm53f_kda_replay_batch": (C.c_int, [i32, i32, i32, ptr, ptr, ptr, ptr, i64, ptr] + _SAVES + [i64, i64, ptr]),
    "glm53f_kda_replay_batch_bf16state": (C.c_int, [i32, i32, i32, ptr, ptr, ptr, ptr, i64, ptr] + _SAVES
                                          + [i64, i64, ptr]),
    "glm53f_kda_conv_shift": (C.c_int, [i32, i32, ptr, ptr, i64, ptr]),
    "glm53f_kda_conv_shift_batch": (C.c_int, [i32, i32, i32, ptr, ptr, ptr, i64, ptr, ptr, i64, i64, ptr]),
    "glm53f_kda_prefill_workspace_bytes": (i64, [i32, i32, i32]),
    "glm53f_kda_prefill": (C.c_int, [i32, i32] + _ROWS + [ptr, ptr, ptr, ptr] + _WEIGHTS
                           + [ptr, i64, i32, ptr, i64, ptr]),
    "glm53f_kda_prefill_batch": (C.c_int, [i32, i32, ptr, i32] + _ROWS + [ptr, ptr, ptr, ptr, ptr, ptr] + _WEIGHTS
                                 + [ptr, i64, i32, ptr, i64, ptr]),
    "glm53f_kda_prefill_batch_bf16state": (C.c_int, [i32, i32, ptr, i32] + _ROWS + [ptr, ptr, ptr, ptr, ptr, ptr]
                                           + _WEIGHTS + [ptr, i64, i32, ptr, i64, ptr]),
    "glm53f_kda_verify_batch_bf16state": (C.c_int, [i32, i32, ptr] + _ROWS + [ptr, ptr, ptr, ptr, ptr] + _WEIGHTS
                                          + [ptr, i64, ptr] + _SAVES + [ptr]),
    "glm53f_kda_select_batch_bf16state": (C.c_int, [i32, i32, i32, ptr, ptr, ptr, i64, ptr, i64, ptr, ptr]),
    "glm53f_kda_chain_shift_batch": (C.c_int, [i32, i32, ptr] + _ROWS + [ptr, ptr, ptr, ptr, ptr, ptr] + _WEIGHTS
                                     + [ptr, i64] + _SAVES + [ptr]),
    "glm53f_kda_chain_shift_batch_bf16state": (C.c_int, [i32, i32, ptr] + _ROWS + [ptr, ptr, ptr, ptr, ptr, ptr]
                                               + _WEIGHTS + [ptr, i64] + _SAVES + [ptr]),
    "glm53f_kda_arch": (C.c_char_p, []),
    "glm53f_kda_init": (C.c_int, []),
}

# The 13 entry points of the reference's ABI (crates/glm53f-kda/tests/provenance.rs:41-69).
REFERENCE_SYMBOLS = [
    "glm53f_kda_chain", "glm53f_kda_chain_batch", "glm53f_kda_chain_batch_bf16state", "glm53f_kda_replay",
    "glm53f_kda_replay_layers", "glm53f_kda_replay_batch", "glm53f_kda_replay_batch_bf16state",
    "glm53f_kda_conv_shift", "glm53f_kda_conv_shift_batch", "glm53f_kda_prefill_workspace_bytes",
    "glm53f_kda_prefill", "glm53f_kda_prefill_batch", "glm53f_kda_prefill_batch_bf16state",
]

_lib = None


def lib() -> C.CDLL:
    """The loaded library. Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP kernels first (python -c 'import __graft_entry__ as g; g.build()')")
        _lib = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(_lib, name)
            fn.restype = res
            fn.argtypes = args
    return _lib


def __getattr__(name: str):
    if name in PROTOTYPES:
        return getattr(lib(), name)
    raise AttributeError(name)
