"""The forward's BF16 weight GEMMs (reference: crates/glm53f-forward/src/gemm.rs:1-291): up to `gemv_max_rows` rows
(8) run the hand-written GEMV of this library, bandwidth-bound and row-independent, so that a verify window of R rows
gives the bits of R serial decode steps; more rows run the vendor GEMM (hipBLASLt through torch.matmul here, cuBLAS
in the reference): BF16 inputs, f32 accumulation. The FP8 and MXFP8 paths of the reference's module are not part of
the KDA layers' BF16 projections and are not built.
"""
from dataclasses import dataclass

import torch

from . import ffi

PARTIAL_FLOATS = 1 << 20      # split-K partial sums (gemm.rs:143)
SYNC_COUNTERS = 1 << 16       # one counter per 8 outputs of a split GEMV (gemm.rs:144)


class GemmError(Exception):
    """An argument the reference rejects as invalid."""


@dataclass(frozen=True)
class Bf16Mat:
    """A BF16 weight [groups][n][k] on the device: row o of group g at ptr + g * gstride + o * ld (gemm.rs:33-43)."""
    ptr: int
    n: int
    k: int
    ld: int
    groups: int = 1
    gstride: int = 0

    def bytes(self) -> int:
        return self.groups * self.n * self.k * 2

    @staticmethod
    def of(t: torch.Tensor) -> "Bf16Mat":
        """A contiguous bf16 tensor [n][k] or [groups][n][k]."""
        assert t.dtype == torch.bfloat16 and t.is_contiguous()
        if t.dim() == 2:
            return Bf16Mat(t.data_ptr(), t.shape[0], t.shape[1], t.shape[1])
        return Bf16Mat(t.data_ptr(), t.shape[1], t.shape[2], t.shape[2], t.shape[0], t.shape[1] * t.shape[2])


@dataclass(frozen=True)
class GemmPolicy:
    gemv_max_rows: int = 8
    # rows from gemv_max_rows + 1 up to this take the library's skinny GEMM where its shape rules allow (0: never,
    # the reference's dispatch: everything above the GEMV goes to the vendor GEMM)
    skinny_max_rows: int = 64


class Gemm:
    """The GEMM engine: the split-K scratch the GEMV launches share (one stream: launches run one after another, and
    the kernel leaves the counters zeroed) (gemm.rs:150-180)."""

    def __init__(self, policy: GemmPolicy = GemmPolicy(), device: str = "cuda:0"):
        if policy.gemv_max_rows > 8:
            raise GemmError("the GEMV takes at most 8 rows")
        self.policy = policy
        self.partials = torch.empty(PARTIAL_FLOATS, dtype=torch.float32, device=device)
        self.sync = torch.zeros(SYNC_COUNTERS, dtype=torch.int32, device=device)

    def bytes(self) -> int:
        return self.partials.numel() * 4 + self.sync.numel() * 4

    @staticmethod
    def gemv_ksplit(w: Bf16Mat) -> int:
        return ffi.glm53f_fwd_gemv_ksplit(w.groups, w.n, w.k)

    def bf16(self, x: int, ldx: int, x_gstride: int, w: Bf16Mat, rows: int, out: int, ldo: int, o_gstride: int,
             out_f32: bool, stream: int = 0) -> None:
        """out[g][m][o] = x[g][m] . w[g][o] for `rows` rows (gemm.rs:203-232). Pointers are device addresses."""
        if rows == 0:
            return
        if rows <= self.policy.gemv_max_rows:
            self.gemv(x, ldx, x_gstride, w, rows, out, ldo, o_gstride, out_f32, stream)
        elif rows <= self.policy.skinny_max_rows and self.skinny_takes(w, ldo, o_gstride, out_f32):
            self.skinny(x, ldx, x_gstride, w, rows, out, ldo, o_gstride, out_f32, stream)
        else:
            self.blas(x, ldx, x_gstride, w, rows, out, ldo, o_gstride, out_f32)

    @staticmethod
    def skinny_takes(w: Bf16Mat, ldo: int, o_gstride: int, out_f32: bool) -> bool:
        """The shapes glm53f_fwd_gemm_bf16_skinny accepts (include/glm53f_fwd_gemv.h); others go to the vendor GEMM."""
        return w.n % 16 == 0 and w.k % 128 == 0 and (out_f32 or (ldo % 2 == 0 and o_gstride % 2 == 0))

    def skinny(self, x: int, ldx: int, x_gstride: int, w: Bf16Mat, rows: int, out: int, ldo: int, o_gstride: int,
               out_f32: bool, stream: int = 0) -> None:
        """The weight-streaming MFMA GEMM for 9 to 64 rows (no counterpart in the reference, which calls cuBLAS
        here: gemm.rs:228-234)."""
        rc = ffi.glm53f_fwd_gemm_bf16_skinny(x, ldx, x_gstride, w.ptr, w.ld, w.gstride, w.groups, rows, w.n, w.k, out,
                                             int(out_f32), ldo, o_gstride, stream)
        if rc != 0:
            raise GemmError("glm53f_fwd_gemm_bf16_skinny rejected its arguments" if rc == 1 else f"glm53f_fwd_gemm_bf16_skinny: hipError {rc}")

    def gemv(self, x: int, ldx: int, x_gstride: int, w: Bf16Mat, rows: int, out: int, ldo: int, o_gstride: int,
             out_f32: bool, stream: int = 0) -> None:
        """The GEMV (1..8 rows), whatever the policy (gemm.rs:238-291)."""
        ksplit = self.gemv_ksplit(w)
        if ksplit > 1 and (w.groups * ksplit * rows * w.n > PARTIAL_FLOATS or w.groups * w.n // 8 > SYNC_COUNTERS):
            raise GemmError(f"GEMV split-K scratch too small for {w}")
        rc = ffi.glm53f_fwd_gemv_bf16(x, ldx, x_gstride, w.ptr, w.ld, w.gstride, w.groups, rows, w.n, w.k, ksplit,
                                      self.partials.data_ptr(), self.sync.data_ptr(), out, int(out_f32), ldo, o_gstride,
                                      stream)
        if rc != 0:
            raise GemmError("glm53f_fwd_gemv_bf16 rejected its arguments" if rc == 1 else f"glm53f_fwd_gemv_bf16: hipError {rc}")

    def blas(self, x: int, ldx: int, x_gstride: int, w: Bf16Mat, rows: int, out: int, ldo: int, o_gstride: int,
             out_f32: bool) -> None:
        """The vendor GEMM, whatever the policy (gemm.rs:293-325): views over the raw pointers, one matmul per group
        on torch's current stream."""
        for g in range(w.groups):
            xv = _view(x + 2 * g * x_gstride, (rows, w.k), (ldx, 1), torch.bfloat16)
            wv = _view(w.ptr + 2 * g * w.gstride, (w.n, w.k), (w.ld, 1), torch.bfloat16)
            es = 4 if out_f32 else 2
            ov = _view(out + es * g * o_gstride, (rows, w.n), (ldo, 1), torch.float32 if out_f32 else torch.bfloat16)
            if out_f32:
                # f32 results of bf16 operands: widened operands through the f32 GEMM (every product exact, f32 sums)
                ov.copy_(torch.matmul(xv.float(), wv.float().t()))
            else:
                ov.copy_(torch.matmul(xv, wv.t()))


def _view(ptr: int, shape, strides, dtype) -> torch.Tensor:
    """A tensor over device memory the caller owns (no copy, no ownership)."""
    es = torch.empty(0, dtype=dtype).element_size()
    span = (shape[0] - 1) * strides[0] + (shape[1] - 1) * strides[1] + 1

    class _Raw:
        __cuda_array_interface__ = {"shape": (span * es,), "typestr": "|u1", "data": (ptr, False), "version": 2}

    raw = torch.as_tensor(_Raw(), device="cuda").view(dtype)
    return raw.as_strided(shape, strides)
