"""The weight-streaming GEMM for 9 to 64 rows (glm53f_fwd_gemm_bf16_skinny) through the C ABI. The reference has no
kernel here (its engine calls cuBLAS above 8 rows, crates/glm53f-forward/src/gemm.rs:228-234) and no bit-level
contract; its own test holds cuBLAS to the GEMV within f32 rounding (tests/gemv.rs:180-226), and so do these:
against exact arithmetic (f64 over the exact bf16 products) the f32 result may be off by a few roundings of the
terms' absolute sum, a bf16 output by one rounding more; against this library's GEMV (whose bits are the host
model's) the same. Shapes: the KDA layer's four projections with the engine's strides, every row count that changes
the tiling, grouped weights with group strides, padded strides; rows are independent of the rows beside them;
the argument checks."""
import numpy as np
import pytest
import torch

from glm53f_forward import ffi as fwd
from glm53f_forward.gemm import Bf16Mat, Gemm, GemmPolicy
from oracle import gemv_oracle as go

import harness as hs

pytestmark = pytest.mark.gpu
DEV = hs.DEV


def bf16_normal(rng, shape, sigma):
    return go.bf16_to_f32(go.bf16_round((rng.standard_normal(shape) * sigma).astype(np.float32)))


def to_dev_bf16(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV).to(torch.bfloat16)


def exact(x, w):
    """f64 over the exact products of bf16 values, and the absolute sum of the terms (the scale of an f32 sum's error)."""
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    return x64 @ w64.transpose(0, 2, 1), np.abs(x64) @ np.abs(w64).transpose(0, 2, 1)


def run(x, w, rows, f32_out, *, ldx=None, ldo=None, pad_w=0):
    """x [groups][rows][k], w [groups][n][k] as f32 arrays of bf16 values -> f32 [groups][rows][n]."""
    groups, _, k = x.shape
    n = w.shape[1]
    ldx, ldw, ldo = ldx or k, k + pad_w, ldo or n
    xs = torch.full((groups, x.shape[1], ldx), float("nan"), dtype=torch.bfloat16, device=DEV)
    xs[:, :, :k] = to_dev_bf16(x)
    ws = torch.full((groups, n, ldw), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws[:, :, :k] = to_dev_bf16(w)
    out = torch.full((groups, rows, ldo), -7.0, dtype=torch.float32 if f32_out else torch.bfloat16, device=DEV)
    rc = fwd.glm53f_fwd_gemm_bf16_skinny(hs.ptr(xs), ldx, x.shape[1] * ldx, hs.ptr(ws), ldw, n * ldw, groups, rows, n, k,
                                         hs.ptr(out), int(f32_out), ldo, rows * ldo, None)
    assert rc == 0, rc
    hs.sync()
    o = out.float().cpu().numpy()
    assert np.all(o[:, :, n:] == -7.0), "wrote outside the rows"
    return o[:, :, :n]


def check(got, x, w, rows, f32_out, label):
    ref, scale = exact(x[:, :rows], w)
    # f32 accumulation in steps of 32 and eighths of K: a few roundings of the running sum, bounded by the terms'
    # absolute sum; a bf16 output adds half a step of the result
    tol = 8 * 2.0 ** -24 * scale + (0 if f32_out else 2.0 ** -8 * np.abs(ref)) + 1e-30
    err = np.abs(got.astype(np.float64) - ref)
    worst = float(np.max(err / tol))
    print(f"{label}: max |err| {float(err.max()):.3e}, worst err / tolerance {worst:.3f}")
    assert np.all(err <= tol), label


@pytest.mark.parametrize("name,groups,n,k", [("kda_proj", 1, 24640, 4096), ("fga", 1, 256, 4096), ("fgb", 2, 8192, 128),
                                              ("o_proj", 1, 4096, 8192)])
@pytest.mark.parametrize("f32_out", [False, True])
def test_the_kda_layers_projections_with_sixteen_rows(name, groups, n, k, f32_out):
    rng = np.random.default_rng(hash(name) % 1000)
    x, w = bf16_normal(rng, (groups, 16, k), 1.0), bf16_normal(rng, (groups, n, k), 0.02)
    check(run(x, w, 16, f32_out), x, w, 16, f32_out, f"{name}, 16 rows, {'f32' if f32_out else 'bf16'} out")


@pytest.mark.parametrize("rows", [1, 9, 15, 16, 17, 31, 32, 33, 48, 49, 64])
def test_every_tiling_of_the_rows(rows):
    rng = np.random.default_rng(rows)
    x, w = bf16_normal(rng, (1, 64, 1024), 1.0), bf16_normal(rng, (1, 272, 1024), 0.05)
    got = run(x, w, rows, True)
    check(got, x, w, rows, True, f"{rows} rows")
    # a row's result depends neither on how many rows ride along nor on its place among them
    alone = run(x[:, rows - 1:rows], w, 1, True)
    assert np.array_equal(hs.bits(got[:, rows - 1]), hs.bits(alone[:, 0])), rows
    turned = run(x[:, ::-1], w, 64, True)
    assert np.array_equal(hs.bits(got), hs.bits(turned[:, ::-1][:, :rows])), rows


@pytest.mark.parametrize("n,k", [(4112, 128), (4112, 384), (8240, 512), (16432, 1024), (8240, 3072), (16432, 2048), (272, 2048)])
def test_every_shape_of_the_launch(n, k):
    """The launch picks the chunk (256 or 128 k), the K split (1, 4 or 8 waves) and the tiles per workgroup (1, 2,
    4, 8) from n, k and the rows: tile counts one to three past a multiple of the tiles per workgroup (the last
    workgroup owns fewer), one to eight chunks per wave (odd counts too: the load sets swap roles chunk by chunk
    where a chunk has an odd number of items), each with one to four tiles of rows."""
    rng = np.random.default_rng(n + k)
    x, w = bf16_normal(rng, (1, 64, k), 1.0), bf16_normal(rng, (1, n, k), 0.05)
    for rows in (16, 24, 40, 64):
        check(run(x, w, rows, rows == 24), x, w, rows, rows == 24, f"n {n} k {k} rows {rows}")


def test_grouped_weights_and_padded_strides():
    rng = np.random.default_rng(5)
    x, w = bf16_normal(rng, (3, 20, 384), 1.0), bf16_normal(rng, (3, 48, 384), 0.1)
    check(run(x, w, 20, False, ldx=400, ldo=64, pad_w=8), x, w, 20, False, "3 groups, padded strides")


def test_agrees_with_the_gemv_within_f32_rounding():
    """tests/gemv.rs:180-226 holds the vendor GEMM to the GEMV this way: same inputs, 8 rows, f32 outputs."""
    rng = np.random.default_rng(6)
    k, n = 4096, 512
    x, w = bf16_normal(rng, (1, 8, k), 1.0), bf16_normal(rng, (1, n, k), 0.02)
    got = run(x, w, 8, True)
    xs, ws = to_dev_bf16(x[0]), to_dev_bf16(w[0])
    out = torch.zeros(8, n, dtype=torch.float32, device=DEV)
    g = Gemm()
    g.gemv(hs.ptr(xs), k, 0, Bf16Mat.of(ws), 8, hs.ptr(out), n, 0, True)
    hs.sync()
    _, scale = exact(x, w)
    assert np.all(np.abs(got[0] - out.cpu().numpy()) <= 16 * 2.0 ** -24 * scale[0])


def test_the_dispatch_sends_nine_to_sixty_four_rows_here():
    rng = np.random.default_rng(7)
    k, n = 512, 64
    w = to_dev_bf16(bf16_normal(rng, (n, k), 0.1))
    for rows, policy in ((12, GemmPolicy()), (12, GemmPolicy(skinny_max_rows=0)), (70, GemmPolicy())):
        x = to_dev_bf16(bf16_normal(rng, (rows, k), 1.0))
        out = torch.zeros(rows, n, dtype=torch.bfloat16, device=DEV)
        Gemm(policy).bf16(hs.ptr(x), k, 0, Bf16Mat.of(w), rows, hs.ptr(out), n, 0, False)
        hs.sync()
        ref = x.float() @ w.float().t()
        assert torch.allclose(out.float(), ref, rtol=2.0 ** -7, atol=1e-3), (rows, policy)


def test_argument_checks():
    d = torch.zeros(1 << 16, dtype=torch.bfloat16, device=DEV)
    o = torch.zeros(1 << 16, dtype=torch.float32, device=DEV)
    p, q = hs.ptr(d), hs.ptr(o)
    ok = dict(x=p, ldx=256, xg=0, w=p, ldw=256, wg=0, groups=1, rows=16, n=32, k=256, out=q, f32=1, ldo=32, og=0)

    def call(**kw):
        a = {**ok, **kw}
        return fwd.glm53f_fwd_gemm_bf16_skinny(a["x"], a["ldx"], a["xg"], a["w"], a["ldw"], a["wg"], a["groups"], a["rows"],
                                               a["n"], a["k"], a["out"], a["f32"], a["ldo"], a["og"], None)

    assert call() == 0
    for bad in (dict(rows=0), dict(rows=65), dict(n=24), dict(n=0), dict(k=192), dict(k=0), dict(x=None), dict(w=None),
                dict(out=None), dict(ldx=255), dict(ldx=128), dict(ldw=100), dict(ldo=16), dict(groups=0), dict(x=p + 2),
                dict(f32=0, ldo=33), dict(f32=0, out=q + 2)):
        assert call(**bad) == 1, bad
    hs.sync()
