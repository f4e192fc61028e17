"""CPU tests of the BF16 GEMV's oracle: the split rule against hand-derived answers, the vectorised model against a
scalar transcription of the reference's host model (crates/glm53f-forward/src/reference.rs:27-71) and against an
f64 dot product, the sensitivity of the bits to the summation order, and the C ABI of include/glm53f_fwd_gemv.h as
a boundary (symbols, prototypes, the host-side split rule). No compute call: runs without a GPU."""
import os
import re
import struct

import numpy as np

from glm53f_forward import ffi as fwd
from oracle import gemv_oracle as go

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def f32(x: float) -> float:
    return struct.unpack("f", struct.pack("f", x))[0]


def scalar_model(x, w, ksplit):
    """reference.rs:31-71 line by line on python floats, rounding to f32 after every operation; the exact product of
    two bf16 values needs no rounding of its own inside the fused multiply-add."""
    rows, k = x.shape
    n = w.shape[0]
    kc = k // ksplit
    xf, wf = go.bf16_to_f32(x).astype(np.float64), go.bf16_to_f32(w).astype(np.float64)
    out = np.zeros((rows, n), dtype=np.float32)
    for m in range(rows):
        for o in range(n):
            total = 0.0
            for s in range(ksplit):
                lo, hi = s * kc, (s + 1) * kc
                lanes = [0.0] * 32
                for l in range(32):
                    k0 = lo + 8 * l
                    while k0 < hi:
                        for j in range(8):
                            lanes[l] = f32(xf[m, k0 + j] * wf[o, k0 + j] + lanes[l])
                        k0 += 256
                v = lanes
                for off in (16, 8, 4, 2, 1):
                    v = [f32(v[l] + v[l ^ off]) for l in range(32)]
                total = v[0] if s == 0 else f32(total + v[0])
            out[m, o] = total
    return out


def bf16_normal(rng, shape, sigma):
    return go.bf16_round((rng.standard_normal(shape) * sigma).astype(np.float32))


def test_split_rule_hand_derived():
    # blocks of 8 outputs >= 512: no split
    assert go.gemv_ksplit(1, 4096, 4096) == 1
    assert go.gemv_ksplit(1, 24_640, 4096) == 1
    # 8 blocks, k = 4096: d = 2 (2048 wide), 3 (not a multiple of 768), 4 (1024 wide) -> 4; d = 5 is under 1024
    assert go.gemv_ksplit(1, 64, 4096) == 4
    assert go.gemv_ksplit(1, 288, 4096) == 4
    assert go.gemv_ksplit(1, 256, 4096) == 4
    # k / 2 < 1024: never split
    assert go.gemv_ksplit(1, 1024, 1536) == 1
    assert go.gemv_ksplit(2, 512, 128) == 1
    # k = 8192, 16 blocks: 2, 4, 8 divide with multiples of 256 and stay >= 1024 wide -> 8
    assert go.gemv_ksplit(1, 128, 8192) == 8
    # stops at the first split count that reaches 512 blocks: 128 blocks x 4
    assert go.gemv_ksplit(1, 1024, 8192) == 4
    for args in ((1, 64, 4096), (1, 4096, 4096), (2, 512, 128), (1, 128, 8192), (1, 1024, 8192), (3, 40, 2048)):
        assert fwd.glm53f_fwd_gemv_ksplit(*args) == go.gemv_ksplit(*args), args
    assert fwd.glm53f_fwd_gemv_ksplit(0, 64, 64) == 1 and fwd.glm53f_fwd_gemv_ksplit(1, 4, 64) == 1


def test_model_against_the_scalar_transcription():
    rng = np.random.default_rng(3)
    for rows, n, k, ksplit in ((2, 3, 512, 1), (1, 2, 512, 2), (2, 2, 520, 1), (1, 2, 272, 2), (1, 1, 2048, 2)):
        x, w = bf16_normal(rng, (rows, k), 1.0), bf16_normal(rng, (n, k), 0.05)
        got, want = go.gemv_bf16(x, w, ksplit), scalar_model(x, w, ksplit)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (rows, n, k, ksplit)


def test_model_is_a_dot_product_and_the_order_shows_in_the_bits():
    rng = np.random.default_rng(4)
    x, w = bf16_normal(rng, (3, 4096), 1.0), bf16_normal(rng, (64, 4096), 0.02)
    xf, wf = go.bf16_to_f32(x), go.bf16_to_f32(w)
    exact = xf.astype(np.float64) @ wf.astype(np.float64).T
    for ksplit in (1, 4):
        got = go.gemv_bf16(x, w, ksplit)
        rel = np.sqrt(np.mean((got - exact) ** 2) / np.mean(exact ** 2))
        assert rel < 1e-6, rel
    a, b = go.gemv_bf16(x, w, 1), go.gemv_bf16(x, w, 4)
    assert not np.array_equal(a.view(np.uint32), b.view(np.uint32))      # the split count is part of the result
    plain = (xf[:, None, :] * wf[None, :, :]).astype(np.float32).cumsum(axis=2, dtype=np.float32)[:, :, -1]
    assert not np.array_equal(a.view(np.uint32), plain.view(np.uint32))  # and so is the order inside a split


def test_bf16_rounding_of_the_output():
    x = np.array([1.0, 1.00390625, 1.01171875, -1.00390625, 3.0e38, 1e-40], dtype=np.float32)
    want = np.array([0x3F80, 0x3F80, 0x3F82, 0xBF80, 0x7F62, 0x0001], dtype=np.uint16)   # ties to even; a denormal
    assert np.array_equal(go.bf16_round(x), want)


def declarations():
    text = open(os.path.join(ROOT, "include", "glm53f_fwd_gemv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return {m.group(1): len(m.group(2).split(","))
            for m in re.finditer(r"\bint32_t\s+(glm53f_fwd_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S)}


def test_library_exports_the_declared_gemv_entry_points():
    decl = declarations()
    assert decl == {"glm53f_fwd_gemv_bf16": 18, "glm53f_fwd_gemv_ksplit": 3, "glm53f_fwd_gemv_bf16_static": 16,
                    "glm53f_fwd_gemm_bf16_skinny": 15}
    lib = fwd.lib()
    for name, nargs in decl.items():
        assert hasattr(lib, name) and len(fwd.PROTOTYPES[name][1]) == nargs, name
