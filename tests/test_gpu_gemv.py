"""The BF16 GEMV through the C ABI against its model, bit for bit (after the reference's
crates/glm53f-forward/tests/gemv.rs:97-177): the reference's five shapes (K splits, several splits, no split,
grouped with a small K, an n that is no multiple of 16) with BF16 and f32 outputs; every row count 1..8 and a row's
independence of the rows beside it; padded strides; a split that is no multiple of 256 wide; the argument checks of
kernels/gemv_bf16.cu:158-164; the counters left zeroed; the KDA projection's shape (4096 -> 24,640)."""
import numpy as np
import pytest
import torch

from glm53f_forward import ffi as fwd
from glm53f_forward.gemm import Bf16Mat, Gemm, GemmError, GemmPolicy
from oracle import gemv_oracle as go

import harness as hs

pytestmark = pytest.mark.gpu
DEV = hs.DEV


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


class Scratch:
    """The engine's split-K scratch (crates/glm53f-forward/src/gemm.rs:143-171): 2^20 floats, 2^16 zeroed counters."""

    def __init__(self):
        self.partials = torch.empty(1 << 20, dtype=torch.float32, device=DEV)
        self.sync = torch.zeros(1 << 16, dtype=torch.int32, device=DEV)


def bf16_normal(rng, shape, sigma):
    return go.bf16_round((rng.standard_normal(shape) * sigma).astype(np.float32))


def run(sc, x, w, rows, ksplit, f32_out, *, ldx=None, ldw=None, ldo=None, xg=None, wg=None, og=None):
    """x [groups][rows_total][k] bits, w [groups][n][k] bits -> f32 [groups][rows][n] (bf16 outputs widened)."""
    groups, _, k = x.shape
    n = w.shape[1]
    ldx, ldw, ldo = ldx or k, ldw or k, ldo or n
    xg = xg if xg is not None else x.shape[1] * ldx
    wg = wg if wg is not None else n * ldw
    og = og if og is not None else rows * ldo
    xs = np.full(groups * xg + 8, 0x7FC0, dtype=np.uint16)           # NaN filler: a read outside the rows shows
    ws = np.full(groups * wg + 8, 0x7FC0, dtype=np.uint16)
    for g in range(groups):
        for m in range(x.shape[1]):
            xs[g * xg + m * ldx:g * xg + m * ldx + k] = x[g, m]
        for o in range(n):
            ws[g * wg + o * ldw:g * wg + o * ldw + k] = w[g, o]
    d_x, d_w = dev(xs), dev(ws)
    out = torch.full((groups * og + 8,), -7.0, dtype=torch.float32 if f32_out else torch.bfloat16, device=DEV)
    rc = fwd.glm53f_fwd_gemv_bf16(hs.ptr(d_x), ldx, xg, hs.ptr(d_w), ldw, wg, groups, rows, n, k, ksplit,
                                  hs.ptr(sc.partials), hs.ptr(sc.sync), hs.ptr(out), int(f32_out), ldo, og, None)
    assert rc == 0, rc
    hs.sync()
    o = out.float().cpu().numpy()
    got = np.stack([np.stack([o[g * og + m * ldo:g * og + m * ldo + n] for m in range(rows)]) for g in range(groups)])
    gaps = np.ones(o.size, dtype=bool)
    for g in range(groups):
        for m in range(rows):
            gaps[g * og + m * ldo:g * og + m * ldo + n] = False
    assert (o[gaps] == -7.0).all()                                    # nothing written beside the outputs
    return got


def model(x, w, rows, ksplit, f32_out):
    outs = []
    for g in range(x.shape[0]):
        v = go.gemv_bf16(x[g, :rows], w[g], ksplit)
        outs.append(v if f32_out else go.bf16_to_f32(go.bf16_round(v)))
    return np.stack(outs)


SHAPES = [(1, 64, 4096, False), (1, 288, 4096, True), (1, 1024, 1536, False), (2, 512, 128, False), (1, 4096, 4096, True),
          (1, 24, 520, True), (3, 8, 2048, False)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"g{s[0]}-n{s[1]}-k{s[2]}-{'f32' if s[3] else 'bf16'}")
def test_gemv_matches_its_model_and_is_row_independent(shape):
    groups, n, k, f32_out = shape
    sc = Scratch()
    rng = np.random.default_rng(11 + n + k)
    ksplit = fwd.glm53f_fwd_gemv_ksplit(groups, n, k)
    assert ksplit == go.gemv_ksplit(groups, n, k)
    w = bf16_normal(rng, (groups, n, k), 0.02)
    x = bf16_normal(rng, (groups, 8, k), 1.0)
    got = run(sc, x, w, 8, ksplit, f32_out)
    want = model(x, w, 8, ksplit, f32_out)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"{(got != want).sum()} values differ"
    for rows in range(1, 9):
        part = run(sc, x, w, rows, ksplit, f32_out)
        assert np.array_equal(part.view(np.uint32), got[:, :rows].view(np.uint32)), rows
    assert int(sc.sync.abs().sum()) == 0                              # the counters are left zeroed


def test_gemv_with_padded_strides_and_every_split_count():
    sc = Scratch()
    rng = np.random.default_rng(5)
    groups, n, k = 2, 40, 2048
    w = bf16_normal(rng, (groups, n, k), 0.02)
    x = bf16_normal(rng, (groups, 5, k), 1.0)
    for ksplit in (1, 2, 4, 8):
        for f32_out in (False, True):
            got = run(sc, x, w, 5, ksplit, f32_out, ldx=k + 8, ldw=k + 16, ldo=n + 3, xg=5 * (k + 8) + 64,
                      wg=n * (k + 16) + 8, og=5 * (n + 3) + 1)
            want = model(x, w, 5, ksplit, f32_out)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (ksplit, f32_out)
    assert int(sc.sync.abs().sum()) == 0
    # enough outputs for the eight-outputs-per-half-wave kernel, with K splits (the rule itself would not split here)
    n = 8200
    w = bf16_normal(rng, (1, n, 1024), 0.02)
    x = bf16_normal(rng, (1, 4, 1024), 1.0)
    for ksplit in (1, 2):
        got = run(sc, x, w, 4, ksplit, True, ldo=n + 8)
        assert np.array_equal(got.view(np.uint32), model(x, w, 4, ksplit, True).view(np.uint32)), ksplit
    assert int(sc.sync.abs().sum()) == 0


def test_gemv_kda_projection_shape():
    """The KDA input projection of a decode step: 4096 -> 24,640 (q | k | v and the beta logits), one row and eight."""
    sc = Scratch()
    rng = np.random.default_rng(6)
    n, k = 24_640, 4096
    w = bf16_normal(rng, (1, n, k), 0.02)
    x = bf16_normal(rng, (1, 8, k), 1.0)
    assert fwd.glm53f_fwd_gemv_ksplit(1, n, k) == 1
    got8 = run(sc, x, w, 8, 1, False)
    got1 = run(sc, x, w, 1, 1, False)
    assert np.array_equal(got1.view(np.uint32), got8[:, :1].view(np.uint32))
    for rows in range(2, 8):      # every row count of the eight-outputs kernel, whose K pieces depend on the count
        part = run(sc, x, w, rows, 1, False)
        assert np.array_equal(part.view(np.uint32), got8[:, :rows].view(np.uint32)), rows
    sample = rng.permutation(n)[:2048]
    want = model(x, w[:, sample], 8, 1, False)
    assert np.array_equal(got8[:, :, sample].view(np.uint32), want.view(np.uint32))
    got8f = run(sc, x, w, 8, 1, True)                 # f32 outputs: the same sums before the bf16 rounding
    assert np.array_equal(got8f[:, :, sample].view(np.uint32), model(x, w[:, sample], 8, 1, True).view(np.uint32))


def test_gemv_argument_checks():
    sc = Scratch()
    buf = torch.zeros(1 << 16, dtype=torch.bfloat16, device=DEV)
    out = torch.zeros(1 << 12, dtype=torch.float32, device=DEV)
    x, w, o, pa, sy = hs.ptr(buf), hs.ptr(buf, 8192), hs.ptr(out), hs.ptr(sc.partials), hs.ptr(sc.sync)

    def call(**kw):
        a = dict(x=x, ldx=256, xg=0, w=w, ldw=256, wg=0, groups=1, rows=2, n=16, k=256, ksplit=1, pa=pa, sy=sy, o=o,
                 f32=1, ldo=16, og=0)
        a.update(kw)
        return fwd.glm53f_fwd_gemv_bf16(a["x"], a["ldx"], a["xg"], a["w"], a["ldw"], a["wg"], a["groups"], a["rows"],
                                        a["n"], a["k"], a["ksplit"], a["pa"], a["sy"], a["o"], a["f32"], a["ldo"],
                                        a["og"], None)

    assert call() == 0
    for bad in (dict(groups=0), dict(groups=70000), dict(rows=0), dict(rows=9), dict(n=0), dict(n=12), dict(k=4),
                dict(k=260), dict(ksplit=0), dict(ksplit=3), dict(k=2064, ldx=2064, ldw=2064, ksplit=4),
                dict(x=x + 2), dict(w=w + 6), dict(o=None), dict(ldx=260), dict(ldw=257), dict(xg=4), dict(wg=12),
                dict(ldx=248), dict(ldw=128), dict(ldo=8), dict(k=2048, ldx=2048, ldw=2048, ksplit=2, pa=None),
                dict(k=2048, ldx=2048, ldw=2048, ksplit=2, sy=None), dict(x=None), dict(w=None)):
        assert call(**bad) == 1, bad
    hs.sync()


def test_engine_dispatch_and_the_vendor_gemm_within_rounding():
    """crates/glm53f-forward/tests/gemv.rs:179-254: the GEMV through the engine wrapper, the vendor GEMM for more rows
    than the policy gives the GEMV, and their agreement within f32 rounding (relative RMS < 1e-5)."""
    rng = np.random.default_rng(12)
    n, k = 2048, 4096
    w = dev(bf16_normal(rng, (n, k), 0.02)).view(torch.bfloat16)
    x = dev(bf16_normal(rng, (16, k), 1.0)).view(torch.bfloat16)
    gemm = Gemm()
    mat = Bf16Mat.of(w)
    assert mat.bytes() == n * k * 2 and Gemm.gemv_ksplit(mat) == 2

    def run_f32(rows, blas):
        out = torch.zeros(rows, n, dtype=torch.float32, device=DEV)
        (gemm.blas if blas else gemm.gemv)(x.data_ptr(), k, 0, mat, rows, out.data_ptr(), n, 0, True)
        hs.sync()
        return out.cpu().numpy()

    g8, b8 = run_f32(8, False), run_f32(8, True)
    rel = np.sqrt(np.mean((g8 - b8) ** 2) / np.mean(g8 ** 2))
    assert rel < 1e-5, rel
    want = go.gemv_bf16(x[:8].view(torch.int16).cpu().numpy().view(np.uint16), w.view(torch.int16).cpu().numpy().view(np.uint16), 2)
    assert np.array_equal(g8.view(np.uint32), want.view(np.uint32))
    # the policy: 8 rows and fewer take the GEMV (the model's bits), more the vendor GEMM (bf16 of a close value)
    out = torch.zeros(16, n, dtype=torch.bfloat16, device=DEV)
    gemm.bf16(x.data_ptr(), k, 0, mat, 8, out.data_ptr(), n, 0, False)
    hs.sync()
    got8 = out[:8].float().cpu().numpy()
    assert np.array_equal(got8, go.bf16_to_f32(go.bf16_round(want)))
    gemm.bf16(x.data_ptr(), k, 0, mat, 16, out.data_ptr(), n, 0, False)
    hs.sync()
    got16 = out.float().cpu().numpy()
    assert np.max(np.abs(got16[:8] - got8)) <= np.max(np.abs(got8)) * 2.0 ** -7
    with pytest.raises(GemmError):
        Gemm(GemmPolicy(gemv_max_rows=9))
    with pytest.raises(GemmError):                                    # the launcher's own checks surface as errors
        gemm.gemv(x.data_ptr() + 2, k, 0, mat, 8, out.data_ptr(), n, 0, False)


def test_gemv_output_projection_shape_with_five_to_eight_rows():
    """The output projection under a verify window: 8192 -> 4096 without a K split, five to eight rows (the kernel
    whose wave halves split the rows), against the model on a sample of the outputs."""
    sc = Scratch()
    rng = np.random.default_rng(8)
    n, k = 4096, 8192
    w = bf16_normal(rng, (1, n, k), 0.02)
    x = bf16_normal(rng, (1, 8, k), 1.0)
    assert fwd.glm53f_fwd_gemv_ksplit(1, n, k) == 1
    sample = rng.permutation(n)[:512]
    for f32_out in (False, True):
        want = model(x, w[:, sample], 8, 1, f32_out)
        for rows in (5, 6, 7, 8):
            got = run(sc, x, w, rows, 1, f32_out)
            assert np.array_equal(got[:, :, sample].view(np.uint32), want[:, :rows].view(np.uint32)), (rows, f32_out)
