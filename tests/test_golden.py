"""The committed vectors of tests/golden/kda_vectors.npz (written by tests/golden/make_vectors.py).

On the CPU: the oracle as built today reproduces them bit for bit, so a change of compiler, flags or source that
moves any result shows up here first. On the GPU: the HIP path, fed the fixture's inputs through the C ABI, meets
the fixture's answers to the same bars as the live comparisons in test_gpu_chain.py and test_gpu_prefill.py.
"""
import os

import numpy as np
import pytest

from oracle import kda_oracle as o

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kda_vectors.npz")


@pytest.fixture(scope="module")
def vec():
    z = np.load(FIXTURE)  # numpy's default: no pickled objects
    return {k: z[k] for k in z.files}


def case(vec, prefix):
    heads = int(vec["heads"])
    p = o.LayerParams(heads, vec[f"{prefix}.conv_w"], vec[f"{prefix}.a_log"], vec[f"{prefix}.dt_bias"],
                      vec[f"{prefix}.norm_w"])
    rows = o.Rows(heads, int(vec[f"{prefix}.rows"]), vec[f"{prefix}.qkv"], vec[f"{prefix}.a"], vec[f"{prefix}.b"],
                  vec[f"{prefix}.gate"])
    return p, vec[f"{prefix}.conv"].copy(), vec[f"{prefix}.state"].copy(), rows


def same_bits(a, b):
    return np.array_equal(np.asarray(a, np.float32).view(np.uint32), np.asarray(b, np.float32).view(np.uint32))


def test_oracle_reproduces_the_chain_vectors(vec):
    p, conv, s0, rows = case(vec, "chain")
    keep = int(vec["chain.keep"])
    c = o.chain(p, conv, s0, rows)
    assert same_bits(c.out, vec["chain.out"]) and same_bits(c.state, vec["chain.state_out"])
    assert same_bits(c.saves.k, vec["chain.save_k"]) and same_bits(c.saves.v, vec["chain.save_v"])
    assert same_bits(c.saves.g, vec["chain.save_g"]) and same_bits(c.saves.beta, vec["chain.save_beta"])
    assert same_bits(o.replay(s0, c.saves, keep), vec["chain.replay_state"])
    assert same_bits(o.conv_shift(conv, rows, keep), vec["chain.conv_after"])
    lit = o.literal_chain(p, conv, s0, rows)
    assert same_bits(lit.out, vec["chain.literal_out"]) and same_bits(lit.state, vec["chain.literal_state"])


def test_oracle_reproduces_the_bf16_state_vectors(vec):
    p, conv, s0, rows = case(vec, "chain16")
    c = o.chain_bf16_state(p, conv, s0, rows)
    assert same_bits(c.out, vec["chain16.out"]) and same_bits(c.state, vec["chain16.state_out"])
    assert same_bits(o.replay(s0, c.saves, int(vec["chain16.keep"]), bf16_state=True), vec["chain16.replay_state"])


def test_oracle_reproduces_the_prefill_vectors(vec):
    p, conv, s0, rows = case(vec, "prefill")
    lit = o.literal_chain(p, conv, s0, rows)
    assert same_bits(lit.out, vec["prefill.out"]) and same_bits(lit.state, vec["prefill.state_out"])
    assert same_bits(o.conv_shift(conv, rows, rows.rows), vec["prefill.conv_after"])
    # The chunked form the device kernel follows agrees with the stored recurrence to the reference's bound
    # (crates/glm53f-kda/tests/gpu_prefill.rs:33-36: state 1e-3 of the largest entry).
    ch = o.prefill(p, conv, s0, rows)
    assert np.max(np.abs(ch.state - vec["prefill.state_out"])) <= 1e-3 * np.max(np.abs(vec["prefill.state_out"]))


@pytest.mark.gpu
def test_gpu_chain_meets_the_vectors(vec):
    import torch

    from glm53f_kda import channels, ffi

    import harness as hs

    p, conv, s0, rows = case(vec, "chain")
    heads, keep = p.heads, int(vec["chain.keep"])
    g = hs.chain_gpu(p, conv, s0, rows)
    # tests/gpu.rs:311-368: the tolerances of the reference's CUDA chain against its CPU model.
    assert hs.max_rel(g.saves.g, vec["chain.save_g"]) <= 4e-6
    assert hs.ulps(g.saves.v, vec["chain.save_v"])[0] <= 1 and hs.ulps(g.saves.beta, vec["chain.save_beta"])[0] <= 1
    assert hs.max_abs(g.saves.k, vec["chain.save_k"]) <= 1.0 / 256.0
    assert hs.rel_err(g.state, vec["chain.state_out"]) <= 1e-5
    assert hs.rel_err(g.out, vec["chain.out"]) <= 1.0 / 256.0
    # The north-star bars against the FP32 recurrent reference.
    assert hs.rel_err(g.state, vec["chain.literal_state"]) <= 1e-5
    assert hs.max_abs(g.out, vec["chain.literal_out"]) <= 2e-2
    # Replay of the fixture's saves and the conv shift involve no transcendental function: bitwise.
    sv = hs.Saves(heads, rows.rows)
    sv.upload(o.Saves(heads, rows.rows, vec["chain.save_k"], vec["chain.save_v"], vec["chain.save_g"],
                      vec["chain.save_beta"]))
    s_in = hs.to_f32(s0)
    replayed = torch.zeros_like(s_in)
    hs.check(ffi.glm53f_kda_replay(heads, keep, hs.ptr(s_in), hs.ptr(replayed), *sv.args(), None), "replay")
    conv_d = hs.to_bf16(conv)
    sr = hs.StagedRows(rows)
    hs.check(ffi.glm53f_kda_conv_shift(channels(heads), keep, hs.ptr(conv_d), hs.ptr(sr.p), sr.p_stride, None), "shift")
    hs.sync()
    assert same_bits(hs.back(replayed), vec["chain.replay_state"])
    assert same_bits(hs.back(conv_d), vec["chain.conv_after"])


@pytest.mark.gpu
def test_gpu_bf16_state_chain_meets_the_vectors(vec):
    import harness as hs

    p, conv, s0, rows = case(vec, "chain16")
    pool = hs.Pool(p.heads, 1, True, 1)
    pool.state_host, pool.conv_host = s0, conv
    pool.state, pool.conv = hs.to_bf16(s0), hs.to_bf16(conv)
    out, s_out, sv, _, _ = hs.chain_batch_gpu(p, pool, [0], [rows], write="to", saves=True)
    # The CPU replay of the device's own saves is the device's state bit for bit; against the stored chain the
    # state may differ by a bf16 rounding flip where exp differs in the last place (tests/gpu_bf16_state.rs:385-419).
    got = pool.device_state(0, s_out)
    assert same_bits(o.replay(s0, sv.download(rows.rows), rows.rows, bf16_state=True), got)
    assert hs.bf16_state_close(got, vec["chain16.state_out"])
    assert hs.rel_err(out, vec["chain16.out"]) <= 1.0 / 256.0


@pytest.mark.gpu
def test_gpu_prefill_meets_the_vectors(vec):
    import harness as hs

    p, conv, s0, rows = case(vec, "prefill")
    out, state, conv_after = hs.prefill_gpu(p, conv, s0, rows)
    assert hs.rel_err(state, vec["prefill.state_out"]) <= 1e-5
    # the synthetic layer's outputs reach 7, where one bf16 step is 3e-2: normwise two steps of the largest output,
    # and only a handful of outputs may differ at all
    assert hs.rel_err(out, vec["prefill.out"]) <= 2.0 ** -7
    assert hs.ulps(out, vec["prefill.out"])[1] <= max(4, 0.003 * out.size)
    assert same_bits(conv_after, vec["prefill.conv_after"])
