"""Accuracy over long prompts against exact arithmetic, and drift of chain, prefill and bf16 states.

Follows crates/glm53f-kda/tests/gpu_prefill.rs:413-543 (long_prompt_drift, accuracy_against_exact_arithmetic) and
tests/gpu_bf16_state.rs:704-804 (drift over 8K and 64K rows): final states against an f64 replay of the chain's own
replay inputs (so every path sees the same k, v, decay and beta), with gates across the whole range and with every
channel decaying slowly (multipliers of at least 0.9993, where old rounding is forgotten mostly through the delta
rule itself). The reference's prefill is f32 throughout and is held to 1e-6 there; this one feeds the matrix cores
fp16 hi/lo pairs (22 bits) and is held to 2.5e-4, a quarter of the north-star bound, with the measured figures printed.
"""
import numpy as np
import pytest
import torch

from glm53f_kda import DK, DV
from oracle import kda_oracle as o

import harness as hs

pytestmark = pytest.mark.gpu

H, SEG = 8, 8192
STATE_TOL = 2.5e-4        # measured: 2.7e-6 with gates across the range, 9.7e-5 with slow decay over 8192 rows (the
                         # operands carry 22 bits, not f32's 24, and slow decay forgets no rounding); north-star bar 1e-3


def layer(slow):
    p = o.synth_layer(H, 860)
    if slow:   # exp(A_log) (a + dt_bias) <= -9 for a in [-4, 4]: sigmoid <= 1.2e-4
        p.a_log[:] = 0.0
        p.dt_bias[:] = -13.0
    return p


def rel_exact(got, exact):
    return float(np.max(np.abs(np.asarray(got, np.float64) - exact)) / np.max(np.abs(exact)))


def rel_rms(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return float(np.sqrt(np.sum((got - ref) ** 2) / np.sum(ref ** 2)))


def chain_bf16(p, conv, s0, rows, saves=False):
    """The chain with a bf16 state on one request (through the batch entry point)."""
    pool = hs.Pool(p.heads, 1, True, 1)
    pool.state_host, pool.conv_host = s0, conv
    pool.state, pool.conv = hs.to_bf16(s0), hs.to_bf16(conv)
    out, s_out, sv, _, _ = hs.chain_batch_gpu(p, pool, [0], [rows], write="to", saves=saves)
    return out, pool.device_state(0, s_out), sv


def prefill_bf16(p, conv, s0, rows):
    pool = hs.Pool(p.heads, 1, True, 1)
    pool.state_host, pool.conv_host = s0, conv
    pool.state, pool.conv = hs.to_bf16(s0), hs.to_bf16(conv)
    out, *_ = hs.prefill_batch_gpu(p, pool, [0], [rows])
    return out, pool.device_state(0)


@pytest.mark.parametrize("slow", [False, True])
def test_accuracy_against_exact_arithmetic(slow):
    """gpu_prefill.rs:458-543, gpu_bf16_state.rs:704-764."""
    p = layer(slow)
    rows = o.synth_rows(H, SEG, 895)
    s0 = o.bf16_round(o.synth_state(H, 896, 0.5))
    conv = o.synth_conv_window(H, 897)
    c = hs.chain_gpu(p, conv, s0, rows)
    _, pre, _ = hs.prefill_gpu(p, conv, s0, rows, rows_per_pass=2048)
    exact = o.exact_replay(s0, c.saves, threads=8)
    ce, pe = rel_exact(c.state, exact), rel_exact(pre, exact)
    _, cb, svb = chain_bf16(p, conv, s0, rows, saves=True)
    _, pb = prefill_bf16(p, conv, s0, rows)
    assert np.array_equal(hs.bits(svb.download(SEG).k), hs.bits(c.saves.k)), "the replay inputs do not see the state"
    cbe, pbe = rel_exact(cb, exact), rel_exact(pb, exact)
    name = "slow decay" if slow else "gates across the range"
    print(f"{name}, {SEG} rows, state against exact arithmetic: chain f32 {ce:.2e}, prefill f32 {pe:.2e}, "
          f"chain bf16 state {cbe:.2e}, prefill bf16 state {pbe:.2e}")
    assert ce <= 1e-5
    assert pe <= STATE_TOL
    for st, e in ((cb, cbe), (pb, pbe)):
        assert np.all(np.isfinite(st)) and e < 0.25, "bf16 state far from exact"


@pytest.mark.parametrize("slow", [False, True])
def test_long_prompt_drift(slow):
    """gpu_prefill.rs:413-456: 64K rows in eight segments, prefill and chain each continuing from their own state;
    and gpu_bf16_state.rs:766-804: the bf16-state chain against the f32-state chain over the same rows."""
    p = layer(slow)
    s0 = o.bf16_round(o.synth_state(H, 861, 0.5))
    conv0 = o.synth_conv_window(H, 862)
    sc, sp, sb = s0.copy(), s0.copy(), s0.copy()
    cc = conv0.copy()
    errs, errs_b = [], []
    for k in range(8):
        rows = o.synth_rows(H, SEG, 870 + k)
        c = hs.chain_gpu(p, cc, sc, rows, want_saves=False)
        out_p, st_p, conv_p = hs.prefill_gpu(p, cc, sp, rows, rows_per_pass=2048)
        out_b, st_b, _ = chain_bf16(p, cc, sb, rows)
        conv_c = o.conv_shift(cc, rows, SEG)
        sn = hs.rel_err(st_p, c.state)
        on = hs.rel_err(out_p, c.out)
        sbn = rel_rms(st_b, c.state)
        print(f"{'slow' if slow else 'mixed'} decay, rows {(k + 1) * SEG:6d}: prefill against chain: state {sn:.2e}, "
              f"segment outputs {on:.2e} normwise; bf16 against f32 state: rms {sbn:.2e}")
        errs.append(sn)
        errs_b.append(sbn)
        assert np.array_equal(conv_p, conv_c)
        sc, sp, sb, cc = c.state, st_p, st_b, conv_c
    assert max(errs) <= STATE_TOL, f"state error {max(errs)} after up to 64K rows"
    assert errs[7] <= 4.0 * errs[0] + 1e-7, f"error grows: {errs}"
    assert np.isfinite(max(errs_b)) and max(errs_b) < 0.25
    assert errs_b[7] <= 4.0 * errs_b[0] + 1e-3, f"bf16 error grows: {errs_b}"


def test_one_row_with_a_bf16_state_is_the_f32_chain_rounded_once():
    """gpu_bf16_state.rs:388-396."""
    heads = 64
    p, conv = o.synth_layer(heads, 940), o.synth_conv_window(heads, 940)
    s0 = o.bf16_round(o.synth_state(heads, 940, 0.5))
    rows = o.synth_rows(heads, 1, 940)
    a = hs.chain_gpu(p, conv, s0, rows)
    out_b, st_b, sv_b = chain_bf16(p, conv, s0, rows, saves=True)
    assert np.array_equal(hs.bits(a.out), hs.bits(out_b))
    assert np.array_equal(hs.bits(a.saves.k), hs.bits(sv_b.download(1).k))
    assert np.array_equal(hs.bits(o.bf16_round(a.state)), hs.bits(st_b))
