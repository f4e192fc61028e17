"""CPU restatement of the BF16 weight GEMV's numerical contract, in numpy.

TEST INFRASTRUCTURE ONLY: imported by tests, the smoke check and the benchmark's CPU-baseline leg, never by the
product path.

Follows the reference's host model crates/glm53f-forward/src/reference.rs:8-71 (`gemv_ksplit`, `gemv_bf16`) and
crates/glm53f-layers/src/math.rs:76-88 (`warp_sum`): per K split 32 partial sums per output, partial l an fma chain
over k = lo + 8 l + 256 i + j (i outer, j = 0..7), an xor butterfly over offsets 16, 8, 4, 2, 1, splits added in
order. The product of two bf16 values is exact in f32, so `fma(x, w, acc)` is `acc + x * w` in f32 arithmetic
(numpy float32), as long as the product is a normal number.

Pinned by (tests/test_gemv.py): a scalar transcription of the model on small cases (python floats rounded to f32
after every operation), agreement with an f64 dot product within f32 rounding, hand-derived answers of the split
rule, and the fact that a different summation order gives different bits on the same data (the order is what is
being tested).
"""
import numpy as np


def gemv_ksplit(groups: int, n: int, k: int) -> int:
    """reference.rs:8-25."""
    blocks = (n // 8) * groups
    if blocks >= 512:
        return 1
    best, d = 1, 2
    while k // d >= 1024:
        if k % (256 * d) == 0:
            best = d
            if blocks * d >= 512:
                break
        d += 1
    return best


def bf16_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """f32 -> bf16 bits, round to nearest even (finite inputs)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def warp_sum(lanes: np.ndarray) -> np.ndarray:
    """math.rs:76-88 over the last axis (32 lanes); returns lane 0."""
    v = lanes.astype(np.float32)
    idx = np.arange(32)
    for off in (16, 8, 4, 2, 1):
        v = v + v[..., idx ^ off]
    return v[..., 0]


def gemv_bf16(x: np.ndarray, w: np.ndarray, ksplit: int) -> np.ndarray:
    """x bf16 bits [rows][k], w bf16 bits [n][k] -> f32 [rows][n] before the output rounding (reference.rs:27-71)."""
    rows, k = x.shape
    n = w.shape[0]
    assert w.shape[1] == k and k % ksplit == 0 and (k // ksplit) % 8 == 0
    kc = k // ksplit
    xf, wf = bf16_to_f32(x), bf16_to_f32(w)
    steps = -(-kc // 256)
    total = None
    for s in range(ksplit):
        pad = steps * 256 - kc
        xs = np.pad(xf[:, s * kc:(s + 1) * kc], ((0, 0), (0, pad))).reshape(rows, steps, 32, 8)
        ws = np.pad(wf[:, s * kc:(s + 1) * kc], ((0, 0), (0, pad))).reshape(n, steps, 32, 8)
        # lanes past the end of the split do nothing: adding exact zeros (0 * 0) leaves an accumulator as it is
        acc = np.zeros((rows, n, 32), dtype=np.float32)
        for i in range(steps):
            for j in range(8):
                acc = acc + xs[:, None, i, :, j] * ws[None, :, i, :, j]
        part = warp_sum(acc)
        total = part if s == 0 else total + part
    return total.astype(np.float32)
