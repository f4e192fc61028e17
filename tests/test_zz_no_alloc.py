"""glm53f_fwd_gemv_bf16_static (the GEMV whose split-K scratch is the library's own per-GPU array) through the C
ABI against glm53f_fwd_gemv_bf16 with caller scratch, bit for bit: two calls in a row on the same GPU, the second
with a smaller input, then a shape without a split and the rejection of shapes beyond the array. Collected last on
purpose (the file name): it shares one array with every call before it in the process."""
import numpy as np
import pytest
import torch

from glm53f_forward import ffi as fwd
from oracle import gemv_oracle as go

import harness as hs

pytestmark = pytest.mark.gpu
DEV = hs.DEV


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def bf16_normal(rng, shape, sigma):
    return go.bf16_round((rng.standard_normal(shape) * sigma).astype(np.float32))


def both_entry_points(rng, groups, rows, n, k, f32_out):
    """The same inputs through the existing entry point (caller scratch) and the new one; outputs as raw bits."""
    ksplit = fwd.glm53f_fwd_gemv_ksplit(groups, n, k)
    x, w = bf16_normal(rng, (groups, rows, k), 1.0), bf16_normal(rng, (groups, n, k), 0.03)
    d_x, d_w = dev(x), dev(w)
    dt = torch.float32 if f32_out else torch.bfloat16
    want = torch.full((groups, rows, n), -7.0, dtype=dt, device=DEV)
    got = torch.full((groups, rows, n), -7.0, dtype=dt, device=DEV)
    partials = torch.empty(groups * ksplit * rows * n, dtype=torch.float32, device=DEV)
    sync = torch.zeros(groups * (n // 8), dtype=torch.int32, device=DEV)
    args = (hs.ptr(d_x), k, rows * k, hs.ptr(d_w), k, n * k, groups, rows, n, k, ksplit)
    tail = (int(f32_out), n, rows * n, None)
    assert fwd.glm53f_fwd_gemv_bf16(*args, hs.ptr(partials), hs.ptr(sync), hs.ptr(want), *tail) == 0
    assert fwd.glm53f_fwd_gemv_bf16_static(*args, hs.ptr(got), *tail) == 0
    hs.sync()
    view = torch.int32 if f32_out else torch.int16
    model = go.gemv_bf16(x[0], w[0], ksplit)
    first = want[0].float().cpu().numpy()
    assert np.array_equal(first, model if f32_out else go.bf16_to_f32(go.bf16_round(model)))   # the checker's bits
    return ksplit, got.view(view).cpu().numpy(), want.view(view).cpu().numpy()


def test_static_scratch_gemv_matches_the_caller_scratch_gemv_twice_in_a_row():
    rng = np.random.default_rng(21)
    # four splits, 8 rows, 288 outputs: 9,216 partial sums, 36 counters
    ksplit, got, want = both_entry_points(rng, 1, 8, 288, 4096, True)
    assert ksplit == 4 and np.array_equal(got, want)
    # right after it, a smaller input over the same array: two groups, 3 rows, 64 outputs, bf16 outputs
    ksplit, got, want = both_entry_points(rng, 2, 3, 64, 4096, False)
    assert ksplit > 1 and np.array_equal(got, want)
    # and a larger one again: eight splits
    ksplit, got, want = both_entry_points(rng, 1, 5, 128, 8192, True)
    assert ksplit == 8 and np.array_equal(got, want)
    # no split: the array is not touched
    ksplit, got, want = both_entry_points(rng, 1, 2, 4096, 1024, False)
    assert ksplit == 1 and np.array_equal(got, want)


def test_static_scratch_gemv_rejects_what_its_array_cannot_hold():
    d = torch.zeros(1 << 16, dtype=torch.int16, device=DEV)
    o = torch.zeros(1 << 16, dtype=torch.float32, device=DEV)
    p = hs.ptr(d)
    # 8 x 2 x 8 x 2,056 = 263,168 partial sums > 262,144 (the argument checks proper come after the size check)
    assert fwd.glm53f_fwd_gemv_bf16_static(p, 2048, 0, p, 2048, 0, 8, 8, 2056, 2048, 2, hs.ptr(o), 1, 2056, 0, None) == 1
    # 33,000 outputs: 4,125 counters > 4,096
    assert fwd.glm53f_fwd_gemv_bf16_static(p, 2048, 0, p, 2048, 0, 1, 1, 33000, 2048, 2, hs.ptr(o), 1, 33000, 0, None) == 1
    # the existing entry point's checks still apply
    assert fwd.glm53f_fwd_gemv_bf16_static(p, 2048, 0, p, 2048, 0, 1, 9, 64, 2048, 2, hs.ptr(o), 1, 64, 0, None) == 1
    assert fwd.glm53f_fwd_gemv_bf16_static(None, 2048, 0, p, 2048, 0, 1, 1, 64, 2048, 1, hs.ptr(o), 1, 64, 0, None) == 1
    hs.sync()
