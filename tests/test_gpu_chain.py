"""The recurrent path on the GPU against the CPU oracle: decode / verify chain, replays, conv shift, and the
checkpointing verify + select. Everything goes through the C ABI.

Follows the reference's GPU tests (crates/glm53f-kda/tests/gpu.rs:311-792, tests/gpu_bf16_state.rs:330-587):
bitwise where no transcendental function is involved (state update, indexing, batching), tolerances where the
device's expf differs from the host's by an ulp or two.
"""
import numpy as np
import pytest
import torch

from glm53f_kda import DK, DV, WINDOW, channels, ffi, state_len
from oracle import kda_oracle as o

import harness as hs

pytestmark = pytest.mark.gpu

H = 64


def case(heads, rows, seed, scale=0.5):
    return (o.synth_layer(heads, seed), o.synth_conv_window(heads, seed), o.synth_state(heads, seed, scale),
            o.synth_rows(heads, rows, seed))


def test_chain_matches_the_cpu_reference():
    """gpu.rs:311-368. The state update has no transcendental function, so the CPU replay of the device's own
    replay inputs gives the device's state bit for bit; the rest differs only through exp."""
    for r in range(1, 9):
        p, conv, s0, rows = case(H, r, 300 + r)
        g = hs.chain_gpu(p, conv, s0, rows)
        assert np.array_equal(hs.bits(o.replay(s0, g.saves, r)), hs.bits(g.state)), f"R={r}: CPU replay of device saves"
        c = o.chain(p, conv, s0, rows)
        eg = hs.max_rel(g.saves.g, c.saves.g)
        uv, nv = hs.ulps(g.saves.v, c.saves.v)
        ub, nb = hs.ulps(g.saves.beta, c.saves.beta)
        ek = hs.max_abs(g.saves.k, c.saves.k)
        es = hs.rel_err(g.state, c.state)
        uo, no = hs.ulps(g.out, c.out)
        eo = hs.rel_err(g.out, c.out)
        print(f"R={r}: exp(g) {eg:.1e} rel; v {nv} differ (max {uv} ulp); beta {nb} (max {ub}); k {ek:.1e} abs; "
              f"state {es:.1e} rel; out {eo:.1e} rel, {no}/{c.out.size} differ (max {uo} bf16 ulp)")
        assert eg <= 4e-6
        assert uv <= 1 and ub <= 1
        assert nv * 1000 <= c.saves.v.size and nb * 100 <= max(c.saves.beta.size, 100)
        assert ek <= 1.0 / 256.0
        assert es <= 1e-5
        assert eo <= 1.0 / 256.0 and no * 1000 <= c.out.size
        # The north-star bars against the FP32 recurrent reference in its literal formulation.
        lit = o.literal_chain(p, conv, s0, rows)
        assert hs.rel_err(g.state, lit.state) <= 1e-5
        assert hs.max_abs(g.out, lit.out) <= max(2e-2, 2.0 ** -7 * np.max(np.abs(lit.out)))


def test_prefixes_and_serial_steps_are_bitwise():
    """gpu.rs:397-474: a replayed prefix has the bits of a chain over that prefix; a window has the bits of
    serial single-row steps with the device conv shift between them."""
    r = 8
    p, conv, s0, rows = case(H, r, 400)
    full = hs.chain_gpu(p, conv, s0, rows)
    sv = hs.Saves(H, r)
    sv.upload(full.saves)
    s_in = hs.to_f32(s0)
    for keep in range(r + 1):
        replayed = torch.zeros_like(s_in)
        hs.check(ffi.glm53f_kda_replay(H, keep, hs.ptr(s_in), hs.ptr(replayed), *sv.args(), None), "replay")
        hs.sync()
        want = s0 if keep == 0 else hs.chain_gpu(p, conv, s0, rows.slice(0, keep)).state
        assert np.array_equal(hs.bits(hs.back(replayed)), hs.bits(want)), keep
    # Serial steps.
    w = hs.Weights(p)
    conv_d = hs.to_bf16(conv)
    s_d = hs.to_f32(s0)
    n = H * DV
    for i in range(r):
        sr = hs.StagedRows(rows.slice(i, 1))
        hs.check(ffi.glm53f_kda_chain(H, 1, *sr.row_args(), hs.ptr(conv_d), hs.ptr(w.conv_w), hs.ptr(s_d), hs.ptr(s_d),
                                      *w.args(), hs.ptr(sr.out), sr.out_stride, *hs.NO_SAVES, None), "chain")
        hs.check(ffi.glm53f_kda_conv_shift(channels(H), 1, hs.ptr(conv_d), hs.ptr(sr.p), sr.p_stride, None), "shift")
        hs.sync()
        assert np.array_equal(hs.bits(sr.out_np()), hs.bits(full.out[i * n:(i + 1) * n])), i
    assert np.array_equal(hs.bits(hs.back(s_d)), hs.bits(full.state))
    assert np.array_equal(hs.back(conv_d), o.conv_shift(conv, rows, r))


def test_strides_negative_b_off_and_in_place():
    """gpu.rs:478-549: padded strides, beta logits in front of q|k|v, in-place state: the dense result's bits."""
    p, conv, s0, rows = case(H, 5, 500)
    dense = hs.chain_gpu(p, conv, s0, rows)
    for kw in ({"pad": 24}, {"b_first": True}, {"pad": 8, "b_first": True, "in_place": True}, {"in_place": True}):
        got = hs.chain_gpu(p, conv, s0, rows, **kw)
        assert np.array_equal(hs.bits(got.out), hs.bits(dense.out)), kw
        assert np.array_equal(hs.bits(got.state), hs.bits(dense.state)), kw
        assert np.array_equal(hs.bits(got.saves.k), hs.bits(dense.saves.k)), kw
    # state_out NULL: outputs only.
    got = hs.chain_gpu(p, conv, s0, rows, want_state=False, want_saves=False)
    assert np.array_equal(hs.bits(got.out), hs.bits(dense.out))


@pytest.mark.parametrize("bf16_state", [False, True])
def test_batch_equals_per_request_bitwise(bf16_state):
    """gpu.rs:553-724, gpu_bf16_state.rs:422-587: a batched launch against one launch per request, states in
    shuffled slots, a zero-row request, a different keep per request; chain, commit replay and conv shift."""
    heads, slots_n = 16, 7
    p = o.synth_layer(heads, 600)
    lens = [3, 0, 8, 1, 5]
    slots = [4, 0, 6, 1, 3]
    keep = [2, 0, 8, 0, 3]
    reqs = [o.synth_rows(heads, n, 610 + i) for i, n in enumerate(lens)]
    pool = hs.Pool(heads, slots_n, bf16_state, 620)
    out, s_out, sv, _, meta = hs.chain_batch_gpu(p, pool, slots, reqs, write="to", saves=True)
    n = heads * DV
    run = o.chain_bf16_state if bf16_state else o.chain
    for i, (slot, rq) in enumerate(zip(slots, reqs)):
        # Per request through the batch entry point with batch 1 (bf16 has no single-request entry point).
        pool1 = hs.Pool(heads, slots_n, bf16_state, 620)
        o1, s1, sv1, _, _ = hs.chain_batch_gpu(p, pool1, [slot], [rq], write="to", saves=True)
        r0 = int(meta.cu_host[i])
        assert np.array_equal(hs.bits(out[r0 * n:(r0 + rq.rows) * n]), hs.bits(o1[:rq.rows * n])), i
        assert np.array_equal(hs.bits(pool.device_state(slot, s_out)), hs.bits(pool1.device_state(slot, s1))), i
        if rq.rows:
            got = sv.download(meta.total)
            one = sv1.download(rq.rows)
            assert np.array_equal(hs.bits(got.k[r0 * heads * DK:(r0 + rq.rows) * heads * DK]), hs.bits(one.k))
            assert np.array_equal(hs.bits(got.beta[r0 * heads:(r0 + rq.rows) * heads]), hs.bits(one.beta))
        else:
            assert np.array_equal(hs.bits(pool.device_state(slot, s_out)), hs.bits(pool.state_of(slot)))
        # Against the oracle: the CPU replay of the device saves is the device state, bit for bit.
        if rq.rows:
            want = o.replay(pool.state_of(slot), sv1.download(rq.rows), rq.rows, bf16_state=bf16_state)
            assert np.array_equal(hs.bits(pool.device_state(slot, s_out)), hs.bits(want)), i
            c = run(p, pool.conv_of(slot), pool.state_of(slot), rq)
            if bf16_state:
                assert hs.bf16_state_close(pool.device_state(slot, s_out), c.state)
            else:
                assert hs.rel_err(pool.device_state(slot, s_out), c.state) <= 1e-5
    # Untouched slots stay zero in the fresh output buffer.
    assert np.all(pool.device_state(2, s_out) == 0.0) and np.all(pool.device_state(5, s_out) == 0.0)

    # The commit: replay_batch with a keep per request, one layer and three layers.
    saves_host = sv.download(meta.total)
    for layers in (1, 3):
        stride = slots_n * state_len(heads)
        big_in = pool.state.repeat(layers)
        big_out = torch.zeros_like(big_in)
        kvs, bs = meta.total * heads * DK, meta.total * heads
        lk, lv, lg, lb = sv.k.repeat(layers), sv.v.repeat(layers), sv.g.repeat(layers), sv.b.repeat(layers)
        m2 = hs.BatchMeta(lens, [pool.conv_off(s) for s in slots], [pool.state_off(s) for s in slots], keep)
        fn = ffi.glm53f_kda_replay_batch_bf16state if bf16_state else ffi.glm53f_kda_replay_batch
        hs.check(fn(heads, layers, m2.batch, hs.ptr(m2.cu_rows), hs.ptr(m2.keep), hs.ptr(big_in), hs.ptr(big_out),
                    stride, hs.ptr(m2.state_off), hs.ptr(lk), hs.ptr(lv), hs.ptr(lg), hs.ptr(lb), kvs, bs, None),
                 "replay_batch")
        hs.sync()
        for l in range(layers):
            for i, slot in enumerate(slots):
                r0 = int(meta.cu_host[i])
                sub = o.Saves(heads, lens[i], saves_host.k[r0 * heads * DK:(r0 + lens[i]) * heads * DK],
                              saves_host.v[r0 * heads * DV:(r0 + lens[i]) * heads * DV],
                              saves_host.g[r0 * heads * DK:(r0 + lens[i]) * heads * DK],
                              saves_host.beta[r0 * heads:(r0 + lens[i]) * heads])
                want = o.replay(pool.state_of(slot), sub, keep[i], bf16_state=bf16_state)
                got = hs.back(big_out[l * stride + pool.state_off(slot):l * stride + pool.state_off(slot) + state_len(heads)])
                assert np.array_equal(hs.bits(got), hs.bits(want)), (layers, l, i)

    # The conv shift of every request, two layers (exact data movement).
    c = channels(heads)
    layers = 2
    conv2 = pool.conv.repeat(layers)
    sr = hs.StagedRows(hs.stack_rows(reqs), pad=8)
    p2 = sr.p.reshape(-1).repeat(layers)
    m2 = hs.BatchMeta(lens, [pool.conv_off(s) for s in slots], [pool.state_off(s) for s in slots], keep)
    hs.check(ffi.glm53f_kda_conv_shift_batch(c, layers, m2.batch, hs.ptr(m2.cu_rows), hs.ptr(m2.keep), hs.ptr(conv2),
                                             pool.conv.numel(), hs.ptr(m2.conv_off), hs.ptr(p2), sr.p.numel(),
                                             sr.p_stride, None), "conv_shift_batch")
    hs.sync()
    for l in range(layers):
        for i, slot in enumerate(slots):
            want = o.conv_shift(pool.conv_of(slot), reqs[i], keep[i])
            at = l * pool.conv.numel() + pool.conv_off(slot)
            assert np.array_equal(hs.back(conv2[at:at + WINDOW * c]), want), (l, i)
    for slot in (2, 5):
        at = pool.conv_off(slot)
        assert np.array_equal(hs.back(conv2[at:at + WINDOW * c]), pool.conv_of(slot))


@pytest.mark.parametrize("seed", range(6))
def test_random_ragged_rounds_against_the_oracle(seed):
    """Seeded sweep: head counts that are no power of two, 0 to 17 rows per request, shuffled slots, either state
    type, in place or to a fresh buffer, with or without the conv window advance in the same launch. The state
    and every output row of every request against the CPU chain run on that request alone: the bf16-stored state
    with the reference's rounding points to a bf16 step (device expf), the f32 state to 1e-3."""
    rng = np.random.default_rng(8000 + seed)
    heads = int(rng.choice([1, 2, 3, 5, 8]))
    batch = int(rng.integers(1, 8))
    lens = [int(rng.choice([0, 1, 1, 1, 2, 3, 7, 8, 16, 17])) for _ in range(batch)]
    slots_n = batch + int(rng.integers(0, 3))
    slots = [int(x) for x in rng.permutation(slots_n)[:batch]]
    bf16_state, shift = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    write = "inplace" if shift else str(rng.choice(["inplace", "to"]))
    label = f"seed {seed}: heads {heads}, lens {lens}, slots {slots} of {slots_n}, bf16 state {bf16_state}, " \
            f"write {write}, window advance {shift}"
    print(label, flush=True)
    p = o.synth_layer(heads, 8100 + seed)
    reqs = [o.synth_rows(heads, n, 8200 + 10 * seed + i) for i, n in enumerate(lens)]
    pool = hs.Pool(heads, slots_n, bf16_state, 8300 + seed)
    before = [(pool.conv_of(s), pool.state_of(s)) for s in range(slots_n)]
    out, s_out, _, _, meta = hs.chain_batch_gpu(p, pool, slots, reqs, write=write, shift=shift)
    n, cw = heads * DV, WINDOW * channels(heads)
    run = o.chain_bf16_state if bf16_state else o.chain
    for i, (slot, rq) in enumerate(zip(slots, reqs)):
        conv0, s0 = before[slot]
        got, r0, at = pool.device_state(slot, s_out), int(meta.cu_host[i]), pool.conv_off(slot)
        want_conv = o.conv_shift(conv0, rq, rq.rows) if shift else conv0
        assert np.array_equal(hs.back(pool.conv[at:at + cw]), want_conv), (label, i)
        if rq.rows == 0:
            assert np.array_equal(hs.bits(got), hs.bits(s0)), (label, i)
            continue
        c = run(p, conv0, s0, rq)
        assert (hs.bf16_state_close(got, c.state) if bf16_state else hs.rel_err(got, c.state) <= 1e-5), (label, i)
        assert hs.rel_err(out[r0 * n:(r0 + rq.rows) * n], c.out) <= 2.0 ** -7, (label, i)
    for slot in set(range(slots_n)) - set(slots):
        at = pool.conv_off(slot)
        assert np.array_equal(hs.back(pool.conv[at:at + cw]), before[slot][0]), (label, slot)
        if write == "inplace":
            assert np.array_equal(hs.bits(pool.device_state(slot, s_out)), hs.bits(before[slot][1])), (label, slot)


def test_bf16_state_window_equals_serial_steps_and_replays():
    """gpu_bf16_state.rs:330-417: an R-row window == R serial single-row steps bitwise (outputs, state, saves),
    verify without a state write leaves the pool untouched, the replay of every prefix == the CPU's
    replay_bf16_state bitwise, one row == the f32 chain rounded once."""
    heads, r = 64, 8
    p = o.synth_layer(heads, 700)
    rows = o.synth_rows(heads, r, 700)
    pool = hs.Pool(heads, 3, True, 701)
    slot = 1
    s0, conv0 = pool.state_of(slot).copy(), pool.conv_of(slot).copy()
    out_w, _, sv, _, _ = hs.chain_batch_gpu(p, pool, [slot], [rows], write="skip", saves=True)
    assert np.array_equal(hs.back(pool.state), pool.state_host), "verify must not write the pool"
    saves = sv.download(r)
    out_w2, s_w, _, _, _ = hs.chain_batch_gpu(p, pool, [slot], [rows], write="to")
    assert np.array_equal(hs.bits(out_w), hs.bits(out_w2))
    state_w = pool.device_state(slot, s_w)
    # Serial steps, in place, conv shift between them.
    pool2 = hs.Pool(heads, 3, True, 701)
    n = heads * DV
    w = hs.Weights(p)
    meta1 = hs.BatchMeta([1], [pool2.conv_off(slot)], [pool2.state_off(slot)])
    for i in range(r):
        sr = hs.StagedRows(rows.slice(i, 1))
        hs.check(ffi.glm53f_kda_chain_batch_bf16state(
            heads, 1, hs.ptr(meta1.cu_rows), *sr.row_args(), hs.ptr(pool2.conv), hs.ptr(meta1.conv_off),
            hs.ptr(w.conv_w), hs.ptr(pool2.state), hs.ptr(pool2.state), hs.ptr(meta1.state_off), *w.args(),
            hs.ptr(sr.out), sr.out_stride, *hs.NO_SAVES, None), "chain")
        hs.check(ffi.glm53f_kda_conv_shift_batch(channels(heads), 1, 1, hs.ptr(meta1.cu_rows), hs.ptr(meta1.keep),
                                                 hs.ptr(pool2.conv), 0, hs.ptr(meta1.conv_off), hs.ptr(sr.p), 0,
                                                 sr.p_stride, None), "shift")
        hs.sync()
        assert np.array_equal(hs.bits(sr.out_np()), hs.bits(out_w[i * n:(i + 1) * n])), i
        # Every prefix: the CPU's bf16 replay of the device saves.
        want = o.replay(s0, saves, i + 1, bf16_state=True)
        assert np.array_equal(hs.bits(pool2.device_state(slot)), hs.bits(want)), i
    assert np.array_equal(hs.bits(pool2.device_state(slot)), hs.bits(state_w))
    at = pool2.conv_off(slot)
    assert np.array_equal(hs.back(pool2.conv[at:at + WINDOW * channels(heads)]), o.conv_shift(conv0, rows, r))
    # Against the CPU model of the bf16 chain.
    c = o.chain_bf16_state(p, conv0, s0, rows)
    assert hs.bf16_state_close(state_w, c.state)
    u, nd = hs.ulps(state_w, c.state)
    print(f"bf16 state vs CPU model: {nd}/{c.state.size} differ, max {u} bf16 ulp")
    assert nd * 1000 <= c.state.size
    eo = hs.rel_err(out_w, c.out)
    assert eo <= 1.0 / 128.0
    # One row: the f32 chain's state rounded once.
    row = rows.slice(0, 1)
    f32 = hs.chain_gpu(p, conv0, s0, row)
    pool3 = hs.Pool(heads, 3, True, 701)
    _, s1, _, _, _ = hs.chain_batch_gpu(p, pool3, [slot], [row], write="to")
    assert np.array_equal(hs.bits(pool3.device_state(slot, s1)), hs.bits(o.bf16_round(f32.state)))


def test_verify_checkpoints_and_select_are_bit_exact():
    """The checkpointing verify: checkpoint k holds the bits of k serial decode steps; select copies the
    accepted one per request and leaves keep == 0 untouched."""
    heads = 64
    lens = [4, 6, 1, 5]
    slots = [5, 2, 0, 3]
    keep = [4, 0, 1, 2]
    p = o.synth_layer(heads, 800)
    reqs = [o.synth_rows(heads, n, 810 + i) for i, n in enumerate(lens)]
    pool = hs.Pool(heads, 6, True, 820)
    out_v, _, sv, ck, meta = hs.chain_batch_gpu(p, pool, slots, reqs, write="skip", saves=True, ckpt=True)
    assert np.array_equal(hs.back(pool.state), pool.state_host)
    n = state_len(heads)
    # Serial decode steps per request on a second pool.
    pool2 = hs.Pool(heads, 6, True, 820)
    w = hs.Weights(p)
    for i, (slot, rq) in enumerate(zip(slots, reqs)):
        m1 = hs.BatchMeta([1], [pool2.conv_off(slot)], [pool2.state_off(slot)])
        for r in range(rq.rows):
            sr = hs.StagedRows(rq.slice(r, 1))
            hs.check(ffi.glm53f_kda_chain_batch_bf16state(
                heads, 1, hs.ptr(m1.cu_rows), *sr.row_args(), hs.ptr(pool2.conv), hs.ptr(m1.conv_off),
                hs.ptr(w.conv_w), hs.ptr(pool2.state), hs.ptr(pool2.state), hs.ptr(m1.state_off), *w.args(),
                hs.ptr(sr.out), sr.out_stride, *hs.NO_SAVES, None), "decode")
            hs.check(ffi.glm53f_kda_conv_shift_batch(channels(heads), 1, 1, hs.ptr(m1.cu_rows), hs.ptr(m1.keep),
                                                     hs.ptr(pool2.conv), 0, hs.ptr(m1.conv_off), hs.ptr(sr.p), 0,
                                                     sr.p_stride, None), "shift")
            hs.sync()
            gr = int(meta.cu_host[i]) + r
            assert torch.equal(ck[gr * n:(gr + 1) * n], pool2.state[slot * n:(slot + 1) * n]), (i, r)
    # The CPU's bf16 replay of the saved rows gives the same checkpoints.
    saves = sv.download(meta.total)
    r0 = int(meta.cu_host[1])
    sub = o.Saves(heads, lens[1], *(x[r0 * heads * w_:(r0 + lens[1]) * heads * w_] for x, w_ in
                                    ((saves.k, DK), (saves.v, DV), (saves.g, DK), (saves.beta, 1))))
    for k in (1, 3, 6):
        want = o.replay(pool.state_of(slots[1]), sub, k, bf16_state=True)
        assert np.array_equal(hs.bits(hs.back(ck[(r0 + k - 1) * n:(r0 + k) * n])), hs.bits(want))
    # Select, two layers sharing one checkpoint layout.
    layers = 2
    ck2 = torch.cat([ck, ck.flip(0)])          # layer 1: different bytes
    st2 = pool.state.repeat(layers)
    m2 = hs.BatchMeta(lens, [pool.conv_off(s) for s in slots], [pool.state_off(s) for s in slots], keep)
    hs.check(ffi.glm53f_kda_select_batch_bf16state(heads, layers, m2.batch, hs.ptr(m2.cu_rows), hs.ptr(m2.keep),
                                                   hs.ptr(ck2), ck.numel(), hs.ptr(st2), pool.state.numel(),
                                                   hs.ptr(m2.state_off), None), "select")
    hs.sync()
    for l in range(layers):
        src = ck2[l * ck.numel():(l + 1) * ck.numel()]
        for i, slot in enumerate(slots):
            got = st2[l * pool.state.numel() + slot * n:l * pool.state.numel() + (slot + 1) * n]
            if keep[i] == 0:
                assert torch.equal(got, pool.state[slot * n:(slot + 1) * n])
            else:
                gr = int(meta.cu_host[i]) + keep[i] - 1
                assert torch.equal(got, src[gr * n:(gr + 1) * n])
        for slot in (1, 4):
            assert torch.equal(st2[l * pool.state.numel() + slot * n:l * pool.state.numel() + (slot + 1) * n],
                               pool.state[slot * n:(slot + 1) * n])


def test_baseline_config1_decode_16_of_48_slots():
    """benchmark configuration 1: 16 slots x 1 token from a 48-slot bf16 pool, H=64; q,k,v ~ N(0,1) before the conv,
    beta = sigmoid(N(0,1)), g = -softplus(N(0,1)) (through A_log = dt_bias = 0 and a = logit(softplus(z)/5)),
    initial states ~ N(0, 0.02), random slot ids without repeats."""
    heads, slots_n, batch = 64, 48, 16
    p, reqs = hs_baseline_layer(heads, 900), None
    rng = np.random.default_rng(901)
    slots = [int(s) for s in rng.permutation(slots_n)[:batch]]
    reqs = [hs_baseline_rows(heads, 1, 910 + i) for i in range(batch)]
    pool = hs.Pool(heads, slots_n, True, 920, scale=0.02, gauss=True)
    out, s_out, _, _, meta = hs.chain_batch_gpu(p, pool, slots, reqs, write="inplace")
    n = heads * DV
    worst_out = worst_state = worst_raw = 0.0
    flips = 0
    for i, slot in enumerate(slots):
        c = o.chain_bf16_state(p, pool.conv_of(slot), pool.state_of(slot), reqs[i])
        lit = o.literal_chain(p, pool.conv_of(slot), pool.state_of(slot), reqs[i])
        got_s = pool.device_state(slot)
        worst_out = max(worst_out, hs.max_abs(out[i * n:(i + 1) * n], lit.out))
        u, nd = hs.ulps(got_s, c.state)
        # Against the CPU model of the same roundings: equal but for isolated rounding flips where the device's
        # exp differs from the host's; a flip is one bf16 ulp of that element.
        assert hs.max_abs(got_s, c.state) <= 2.0 ** -8 * np.max(np.abs(c.state))
        flips += nd
        worst_state = max(worst_state, hs.rel_err(got_s, c.state))
        worst_raw = max(worst_raw, hs.rel_err(got_s, lit.state))
    print(f"config 1: out max-abs {worst_out:.2e}; bf16 state vs rounded model {worst_state:.2e} rel "
          f"({flips} ulp flips); vs unrounded f32 literal {worst_raw:.2e} rel")
    assert worst_out <= 2e-2
    assert worst_state <= 1e-3 or flips * 10000 <= batch * state_len(heads)
    assert worst_raw <= 2.0 ** -8
    untouched = [s for s in range(slots_n) if s not in slots]
    for s in untouched[:4]:
        assert np.array_equal(pool.device_state(s), pool.state_of(s))


def hs_baseline_layer(heads, seed):
    rng = o.Rng(seed)
    conv_w = rng.fill_bf16(channels(heads) * 4, -0.6, 0.6)
    return o.LayerParams(heads, conv_w, np.zeros(heads, np.float32), np.zeros(heads * DK, np.float32),
                         np.ones(DV, np.float32))


def hs_baseline_rows(heads, rows, seed):
    rng = o.Rng(seed)
    qkv = o.bf16_round(rng.normal(rows * channels(heads)))
    z = rng.normal(rows * heads * DK).astype(np.float64)
    sp = np.minimum(np.log1p(np.exp(z)), 4.999)
    a = o.bf16_round(np.log(sp / 5.0) - np.log1p(-sp / 5.0))
    b = o.bf16_round(rng.normal(rows * heads))
    gate = o.bf16_round(rng.normal(rows * heads * DV))
    return o.Rows(heads, rows, qkv, a, b, gate)


def test_bad_arguments_are_rejected():
    """gpu.rs:727-792 at the ABI level: host-side rejections return 1 and launch nothing."""
    p, conv, s0, rows = case(4, 2, 950)
    w = hs.Weights(p)
    sr = hs.StagedRows(rows)
    conv_d, s_d = hs.to_bf16(conv), hs.to_f32(s0)
    sv = hs.Saves(4, 2)
    base = lambda: [4, 2, *sr.row_args(), hs.ptr(conv_d), hs.ptr(w.conv_w), hs.ptr(s_d), hs.ptr(s_d), *w.args(),
                    hs.ptr(sr.out), sr.out_stride, *hs.NO_SAVES, None]
    assert ffi.glm53f_kda_chain(*base()) == 0
    a = base(); a[0] = 0
    assert ffi.glm53f_kda_chain(*a) == 1
    a = base(); a[1] = 0
    assert ffi.glm53f_kda_chain(*a) == 1
    a = base(); a[2] = None
    assert ffi.glm53f_kda_chain(*a) == 1
    a = base(); a[-5] = hs.ptr(sv.k)            # only one of the four saves
    assert ffi.glm53f_kda_chain(*a) == 1
    a = base(); a[11] = hs.ptr(s_d) + 4        # misaligned state
    assert ffi.glm53f_kda_chain(*a) == 1
    assert ffi.glm53f_kda_replay(4, -1, hs.ptr(s_d), hs.ptr(s_d), *sv.args(), None) == 1
    assert ffi.glm53f_kda_replay(4, 0, None, hs.ptr(s_d), *sv.args(), None) == 1
    assert ffi.glm53f_kda_conv_shift(0, 1, hs.ptr(conv_d), hs.ptr(sr.p), sr.p_stride, None) == 1
    assert ffi.glm53f_kda_conv_shift(channels(4), -1, hs.ptr(conv_d), hs.ptr(sr.p), sr.p_stride, None) == 1
    meta = hs.BatchMeta([2], [0], [0])
    assert ffi.glm53f_kda_chain_batch(4, 1, None, *sr.row_args(), hs.ptr(conv_d), hs.ptr(meta.conv_off),
                                      hs.ptr(w.conv_w), hs.ptr(s_d), hs.ptr(s_d), hs.ptr(meta.state_off), *w.args(),
                                      hs.ptr(sr.out), sr.out_stride, *hs.NO_SAVES, None) == 1
    assert ffi.glm53f_kda_replay_batch(4, 1, 1, hs.ptr(meta.cu_rows), None, hs.ptr(s_d), hs.ptr(s_d), 0,
                                       hs.ptr(meta.state_off), *sv.args(), 0, 0, None) == 1
    assert ffi.glm53f_kda_conv_shift_batch(channels(4), 70000, 1, hs.ptr(meta.cu_rows), hs.ptr(meta.keep),
                                           hs.ptr(conv_d), 0, hs.ptr(meta.conv_off), hs.ptr(sr.p), 0, sr.p_stride,
                                           None) == 1
    hs.sync()


def test_conv_shift_wide_and_narrow_paths_agree_with_the_oracle():
    """The shift moves eight channels per lane when every row is 16-byte aligned and one channel per lane
    otherwise (rows starting at an odd element, a channel count that is no multiple of eight): same bits."""
    heads = 4
    c = channels(heads)
    rows = o.synth_rows(heads, 5, 910)
    conv = o.synth_conv_window(heads, 911)
    qkv = rows.qkv.reshape(5, c)
    for keep in (0, 1, 2, 3, 5):
        want = o.conv_shift(conv, rows, keep)
        for shift, stride in ((0, c), (1, c + 8), (3, c + 5)):
            p = torch.zeros(5 * stride + 8, dtype=torch.bfloat16, device=hs.DEV)
            p[shift:shift + 5 * stride].view(5, stride)[:, :c] = hs.to_bf16(qkv)
            conv_d = hs.to_bf16(conv)
            hs.check(ffi.glm53f_kda_conv_shift(c, keep, hs.ptr(conv_d), hs.ptr(p, shift), stride, None), "conv shift")
            hs.sync()
            assert np.array_equal(hs.back(conv_d), want), (keep, shift, stride)
    # a channel count that is not a multiple of eight (the kernel takes any count)
    cc = c - 3
    win = torch.arange(3 * cc, device=hs.DEV).to(torch.bfloat16)
    p = (1000 + torch.arange(2 * cc, device=hs.DEV)).to(torch.bfloat16)
    before = win.clone()
    hs.check(ffi.glm53f_kda_conv_shift(cc, 2, hs.ptr(win), hs.ptr(p), cc, None), "conv shift")
    hs.sync()
    assert torch.equal(win.view(3, cc), torch.cat([before.view(3, cc)[2:], p.view(2, cc)]))


@pytest.mark.parametrize("bf16_state", [False, True], ids=["f32-state", "bf16-state"])
def test_chain_with_the_window_advance_in_one_launch(bf16_state):
    """glm53f_kda_chain_shift_batch[_bf16state] == the chain, then glm53f_kda_conv_shift_batch with keep = rows
    (what a decode round of the engine runs per layer), bit for bit: outputs, states, saves and windows; requests of
    0, 1, 2, 3 and 7 rows in shuffled slots; a slot outside the batch is untouched."""
    heads, slots = 6, [4, 1, 5, 0, 2]
    p = o.synth_layer(heads, 61)
    reqs = [o.synth_rows(heads, n, 70 + n) for n in (1, 0, 3, 7, 2)]
    c = channels(heads)
    two = hs.Pool(heads, 6, bf16_state, 62)
    one = hs.Pool(heads, 6, bf16_state, 62)
    out2, st2, sv2, _, m2 = hs.chain_batch_gpu(p, two, slots, reqs, saves=True)
    sr = hs.StagedRows(hs.stack_rows(reqs))
    hs.check(ffi.glm53f_kda_conv_shift_batch(c, 1, m2.batch, hs.ptr(m2.cu_rows), hs.ptr(m2.keep), hs.ptr(two.conv), 0,
                                             hs.ptr(m2.conv_off), hs.ptr(sr.p), 0, sr.p_stride, None), "conv shift")
    hs.sync()
    out1, st1, sv1, _, _ = hs.chain_batch_gpu(p, one, slots, reqs, saves=True, shift=True)
    assert np.array_equal(hs.bits(out1), hs.bits(out2))
    assert torch.equal(st1, st2)
    for a, b in zip((sv1.k, sv1.v, sv1.g, sv1.b), (sv2.k, sv2.v, sv2.g, sv2.b)):
        assert torch.equal(a, b)
    assert torch.equal(one.conv, two.conv)
    for i, slot in enumerate(slots):
        want = o.conv_shift(one.conv_of(slot), reqs[i], reqs[i].rows)
        at = one.conv_off(slot)
        assert np.array_equal(hs.back(one.conv[at:at + WINDOW * c]), want), slot
    at = one.conv_off(3)
    assert np.array_equal(hs.back(one.conv[at:at + WINDOW * c]), one.conv_of(3))


def test_chain_with_the_window_advance_on_unaligned_windows():
    """A window that starts 2 bytes off a 16-byte boundary is read and written in 16-bit elements."""
    heads = 2
    p = o.synth_layer(heads, 63)
    rows = o.synth_rows(heads, 2, 64)
    c = channels(heads)
    w = hs.Weights(p)
    sr = hs.StagedRows(rows)
    pool = hs.Pool(heads, 1, True, 65)
    conv_host = pool.conv_of(0)
    shifted = torch.zeros(WINDOW * c + 8, dtype=torch.bfloat16, device=hs.DEV)
    shifted[1:1 + WINDOW * c] = pool.conv
    meta = hs.BatchMeta([2], [0], [0])
    hs.check(ffi.glm53f_kda_chain_shift_batch_bf16state(
        heads, 1, hs.ptr(meta.cu_rows), *sr.row_args(), hs.ptr(shifted, 1), hs.ptr(meta.conv_off), hs.ptr(w.conv_w),
        hs.ptr(pool.state), hs.ptr(pool.state), hs.ptr(meta.state_off), *w.args(), hs.ptr(sr.out), sr.out_stride,
        *hs.NO_SAVES, None), "chain + shift")
    hs.sync()
    assert np.array_equal(hs.back(shifted[1:1 + WINDOW * c]), o.conv_shift(conv_host, rows, 2))
    assert float(shifted[0]) == 0.0 and float(shifted[1 + WINDOW * c]) == 0.0
    ref = o.chain_bf16_state(p, conv_host, pool.state_of(0), rows)
    assert hs.bf16_state_close(pool.device_state(0), ref.state)
