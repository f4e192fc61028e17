"""glm53f_kda for MI355X: ctypes bindings of the KDA kernels' C ABI (include/glm53f_kda.h).

The module name is the reference crate's (`glm53f_kda`); `ffi` mirrors its raw bindings
(crates/glm53f-kda/src/ffi.rs). There is no CPU fallback: importing `ffi` without the built HIP library
raises.
"""
DK = 128
DV = 128
TAPS = 4
WINDOW = TAPS - 1
HEADS = 64
LAYERS = 34
LOWER_BOUND = -5.0
RMS_EPS = 1e-5
PREFILL_CHUNK = 64


def channels(heads: int) -> int:
    """Conv channels of a layer: q | k | v (crates/glm53f-kda/src/lib.rs:79-81)."""
    return 3 * heads * DK


def state_len(heads: int) -> int:
    """Elements of one layer's recurrent state (crates/glm53f-kda/src/lib.rs:84-86)."""
    return heads * DV * DK
