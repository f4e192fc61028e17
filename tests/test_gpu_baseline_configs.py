"""The benchmark definition's configurations at their stated sizes, through the C ABI.

Config 1 (decode, 16 of 48 slots) lives in test_gpu_chain.py. Here: config 2 (T = 8192 as four 2048-row calls)
against the FP32 recurrent oracle with the north-star tolerances; config 3 (varlen packed prefill) at a size the
oracle finishes in seconds for all heads and at its full 131072 / 20480 / 4096 / 777 rows: values of four heads
against the oracle from restored snapshots, and properties that do not depend on the size (packed == per request
bit for bit, conv windows exact); config 4 (verify 48 slots x 16
drafts with checkpoints) against serial decode steps, bit for bit.
"""
import numpy as np
import pytest
import torch

from glm53f_kda import DK, DV, WINDOW, channels, ffi, state_len
from oracle import kda_oracle as o

import harness as hs

pytestmark = pytest.mark.gpu


def check_outputs(got, ref, label, flip_fraction=0.003):
    """The north-star bar on bf16 outputs: max-abs <= 2e-2 against the FP32 recurrent oracle. The contract rounds
    twice (the read-out to bf16, then the gated norm's result to bf16), so an output whose read-out lands on the
    other side of a rounding boundary moves one or two representable values, and two values are 3.1e-2 apart from
    |out| = 2 upwards: for any kernel that is not bit-exact the bar holds only while such flips are rare. With every
    operand at f32-class precision 0.055 % of the outputs differ at all (the reference's kernel: 0.013 %, its bar
    0.1 %, gpu_prefill.rs:270-276; this build's f32 chain kernel: 0.024 %), which leaves a two-step event at
    |out| >= 2 about once in 10^8 outputs: none among the 67 million of config 2, one among the 80 million checked of
    config 3. So: every output within 2e-2, except that one output per array (and one more per 30 million) may be
    two representable values away where those are further apart than that; and the share that differs at all is
    bounded."""
    got, ref = np.asarray(got, np.float32), np.asarray(ref, np.float32)
    d = np.abs(got.astype(np.float64) - ref.astype(np.float64))
    steps = hs.bf16_steps(got, ref)
    hist = np.bincount(np.minimum(steps, 4).ravel(), minlength=5)
    differ = int((steps > 0).sum())
    over = d > 2e-2
    print(f"{label}: out max-abs {float(d.max()) if d.size else 0.0:.3e}; outputs 0/1/2/3/4+ bf16 steps apart: "
          f"{hist.tolist()}; {differ} of {got.size} differ ({100.0 * differ / max(got.size, 1):.4f} %); "
          f"{int(over.sum())} by more than 2e-2")
    assert int(over.sum()) <= 1 + got.size // 30_000_000, label
    if over.any():
        assert int(steps[over].max()) <= 2 and float(np.minimum(np.abs(got[over]), np.abs(ref[over])).min()) >= 1.9, label
    assert differ <= max(4, flip_fraction * got.size), label


def baseline_layer(heads, seed):
    """Random-init weights; A_log = dt_bias = 0 so that g = -5 sigmoid(a); norm weight one."""
    rng = np.random.default_rng(seed)
    conv_w = o.bf16_round(rng.uniform(-0.6, 0.6, channels(heads) * 4).astype(np.float32))
    return o.LayerParams(heads, conv_w, np.zeros(heads, np.float32), np.zeros(heads * DK, np.float32),
                         np.ones(DV, np.float32))


def baseline_rows(heads, rows, seed):
    """q, k, v ~ N(0, 1) before the conv, beta logits and output-gate logits ~ N(0, 1), and a such that
    g = -softplus(N(0, 1)) (clamped below 5), all rounded to bf16."""
    rng = np.random.default_rng(seed)
    qkv = o.bf16_round(rng.standard_normal(rows * channels(heads), dtype=np.float32))
    sp = np.minimum(np.log1p(np.exp(rng.standard_normal(rows * heads * DK))), 4.999)
    a = o.bf16_round((np.log(sp / 5.0) - np.log1p(-sp / 5.0)).astype(np.float32))
    b = o.bf16_round(rng.standard_normal(rows * heads, dtype=np.float32))
    gate = o.bf16_round(rng.standard_normal(rows * heads * DV, dtype=np.float32))
    return o.Rows(heads, rows, qkv, a, b, gate)


def test_baseline_config2_prefill_8192_in_four_lanes():
    heads, total, lane = 64, 8192, 2048
    p = baseline_layer(heads, 2000)
    rows = baseline_rows(heads, total, 2001)
    conv0 = o.bf16_round(np.random.default_rng(2002).standard_normal(WINDOW * channels(heads), dtype=np.float32))
    s0 = np.zeros(state_len(heads), np.float32)
    conv, st = conv0, s0
    outs = []
    for first in range(0, total, lane):
        out, st, conv = hs.prefill_gpu(p, conv, st, rows.slice(first, lane), rows_per_pass=lane)
        outs.append(out)
    out = np.concatenate(outs)
    lit = o.literal_chain(p, conv0, s0, rows, threads=16)
    es, ea = hs.rel_err(st, lit.state), hs.max_abs(out, lit.out)
    _, nd = hs.ulps(out, lit.out)
    print(f"config 2: state {es:.2e} rel (north-star bar 1e-3, the reference's own 1e-5); out max-abs {ea:.2e}, "
          f"{nd}/{out.size} differ; max |out| {np.max(np.abs(lit.out)):.2f}")
    assert es <= 1e-5
    check_outputs(out, lit.out, "config 2")
    assert np.array_equal(conv, o.conv_shift(conv0, rows, total))


def test_baseline_config3_varlen_packed_against_the_oracle_reduced():
    """The shape of config 3 at an oracle-sized scale: four prompts of different lengths packed with cu_rows,
    nonzero initial states from a prior-prefix run of the oracle, bf16 final states in the pool; ragged tails of
    9 rows (777 = 12 * 64 + 9)."""
    heads, lens, slots = 8, [2048, 320, 64, 777], [3, 0, 4, 1]
    p = baseline_layer(heads, 3000)
    reqs = [baseline_rows(heads, n, 3010 + i) for i, n in enumerate(lens)]
    pool = hs.Pool(heads, 5, True, 3020)
    # a prior prefix of 100 rows per request gives the snapshot the prompt continues from
    for i, slot in enumerate(slots):
        pre = baseline_rows(heads, 100, 3030 + i)
        c = o.literal_chain(p, pool.conv_of(slot), np.zeros(state_len(heads), np.float32), pre, threads=8)
        n = state_len(heads)
        pool.state_host[slot * n:(slot + 1) * n] = o.bf16_round(c.state)
        cw = WINDOW * channels(heads)
        pool.conv_host[slot * cw:(slot + 1) * cw] = o.conv_shift(pool.conv_of(slot), pre, 100)
    pool.state = hs.to_bf16(pool.state_host)
    pool.conv = hs.to_bf16(pool.conv_host)
    out, s_out, meta = hs.prefill_batch_gpu(p, pool, slots, reqs, write="inplace", rows_per_pass=512)
    assert list(meta.cu_host) == [0, 2048, 2368, 2432, 3209]
    n = heads * DV
    for i, (slot, rq) in enumerate(zip(slots, reqs)):
        lit = o.literal_chain(p, pool.conv_of(slot), pool.state_of(slot), rq, threads=8)
        r0 = int(meta.cu_host[i])
        got = pool.device_state(slot)
        u, nd = hs.ulps(got, o.bf16_round(lit.state))
        raw = hs.rel_err(got, lit.state)
        ea = hs.max_abs(out[r0 * n:(r0 + rq.rows) * n], lit.out)
        print(f"config 3 (reduced), request {i} ({rq.rows} rows): bf16 state vs bf16(f32 oracle) {nd} of {got.size} "
              f"differ (max {u} ulp), raw {raw:.2e} rel; out max-abs {ea:.2e}")
        assert raw <= 2.0 ** -8                      # bf16 storage (2^-9) on top of the 1e-3 bar
        assert hs.rel_err(got, o.bf16_round(lit.state)) <= 2.0 ** -8
        # the state of this entry point is bf16 between chunks, the oracle's is f32 throughout: the read-outs differ
        # by the state's rounding (2^-9), which moves a percent of them across a bf16 boundary
        check_outputs(out[r0 * n:(r0 + rq.rows) * n], lit.out, f"config 3 (reduced), request {i}", flip_fraction=0.03)
        pool1 = hs.Pool(heads, 5, True, 3020)
        pool1.state, pool1.conv = hs.to_bf16(pool.state_host), hs.to_bf16(pool.conv_host)
        o1, _, _ = hs.prefill_batch_gpu(p, pool1, [slot], [rq], write="inplace", rows_per_pass=512)
        assert np.array_equal(hs.bits(o1[:rq.rows * n]), hs.bits(out[r0 * n:(r0 + rq.rows) * n])), i
        assert np.array_equal(hs.bits(pool1.device_state(slot)), hs.bits(got)), i


def test_baseline_config3_varlen_packed_full_size_properties():
    """131072 + 20480 + 4096 + 777 rows, 64 heads, inputs generated on the GPU. Packed == per request, bit for
    bit (outputs, bf16 states, conv windows); conv windows equal the last three input rows; nothing overflows."""
    heads, lens, slots = 64, [131072, 20480, 4096, 777], [2, 0, 3, 1]
    c, n, cw = channels(heads), state_len(heads), WINDOW * channels(heads)
    total = sum(lens)
    gen = torch.Generator(device=hs.DEV).manual_seed(31)
    p = baseline_layer(heads, 3100)
    w = hs.Weights(p)
    ps = c + heads
    P = torch.empty(total, ps, device=hs.DEV, dtype=torch.bfloat16)
    A = torch.empty(total, heads * DK, device=hs.DEV, dtype=torch.bfloat16)
    G = torch.empty(total, heads * DV, device=hs.DEV, dtype=torch.bfloat16)
    step = 16384
    for r0 in range(0, total, step):       # in slices: the f32 temporaries stay small
        r1 = min(total, r0 + step)
        P[r0:r1] = torch.randn(r1 - r0, ps, device=hs.DEV, generator=gen).to(torch.bfloat16)
        sp = torch.clamp(torch.nn.functional.softplus(torch.randn(r1 - r0, heads * DK, device=hs.DEV, generator=gen)), max=4.999)
        A[r0:r1] = (torch.log(sp / 5.0) - torch.log1p(-sp / 5.0)).to(torch.bfloat16)
        G[r0:r1] = torch.randn(r1 - r0, heads * DV, device=hs.DEV, generator=gen).to(torch.bfloat16)
    state0 = (torch.randn(4 * n, device=hs.DEV, generator=gen) * 0.1).to(torch.bfloat16)
    conv0 = torch.randn(4 * cw, device=hs.DEV, generator=gen).to(torch.bfloat16)
    rpp = 2048
    ws_bytes = ffi.glm53f_kda_prefill_workspace_bytes(heads, 4, rpp)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=hs.DEV)

    def run(idx):
        """Prefill requests idx (a list) packed; returns (out rows, states, conv windows)."""
        lens_i = [lens[i] for i in idx]
        cu_full = np.concatenate([[0], np.cumsum(lens)])
        rows_sel = torch.cat([torch.arange(cu_full[i], cu_full[i + 1], device=hs.DEV) for i in idx])
        contiguous = len(idx) == 4
        Pi, Ai, Gi = (P, A, G) if contiguous else (P[rows_sel].contiguous(), A[rows_sel].contiguous(), G[rows_sel].contiguous())
        out = torch.zeros(sum(lens_i), heads * DV, device=hs.DEV, dtype=torch.bfloat16)
        st, cv = state0.clone(), conv0.clone()
        meta = hs.BatchMeta(lens_i, [slots[i] * cw for i in idx], [slots[i] * n for i in idx])
        code = ffi.glm53f_kda_prefill_batch_bf16state(
            heads, meta.batch, hs.ptr(meta.cu_rows), max(lens_i), hs.ptr(Pi), ps, c, hs.ptr(Ai), heads * DK, hs.ptr(Gi),
            heads * DV, hs.ptr(cv), hs.ptr(meta.conv_off), hs.ptr(w.conv_w), hs.ptr(st), hs.ptr(st),
            hs.ptr(meta.state_off), *w.args(), hs.ptr(out), heads * DV, 0, hs.ptr(ws), ws_bytes, None)
        hs.check(code, "prefill_batch_bf16state")
        hs.sync()
        return out, st, cv

    out, st, cv = run([0, 1, 2, 3])
    assert bool(torch.isfinite(out.float()).all()) and bool(torch.isfinite(st.float()).all())
    cu = np.concatenate([[0], np.cumsum(lens)])
    for i in range(4):
        o1, s1, c1 = run([i])
        s = slots[i]
        assert torch.equal(o1, out[cu[i]:cu[i + 1]]), f"request {i}: outputs"
        assert torch.equal(s1[s * n:(s + 1) * n], st[s * n:(s + 1) * n]), f"request {i}: state"
        assert torch.equal(c1[s * cw:(s + 1) * cw], cv[s * cw:(s + 1) * cw]), f"request {i}: conv window"
        # the window is exactly the request's last three q|k|v rows
        assert torch.equal(cv[s * cw:(s + 1) * cw].view(WINDOW, c), P[cu[i + 1] - 3:cu[i + 1], :c]), f"request {i}: window rows"
        del o1, s1, c1


def test_baseline_config3_full_size_values_from_a_restored_snapshot():
    """Config 3 as the benchmark definition states it: 131072 + 20480 + 4096 + 777 rows packed, 64 heads, f32 carried
    state, initial states from a prior-prefix snapshot, bf16 final states written back to the slot pool. The
    snapshot is real: a prefix of every prompt is prefilled into the pool's slots, saved as a mark, the slots are
    overwritten, and the marks are loaded back (the row scatter / gather of the snapshot path) before the prompts
    continue. Values: heads 0, 21, 42 and 63 of every request against the FP32 recurrent oracle run on those heads
    alone (heads are independent), states and every output row, under the north-star bars."""
    from glm53f_forward.kv import KvPool
    from glm53f_forward.kvplan import KvLayout

    heads, lens, prefix, slots = 64, [131072, 20480, 4096, 777], [300, 200, 64, 37], [2, 0, 3, 1]
    sub = [0, 21, 42, 63]
    c, n, cw = channels(heads), state_len(heads), WINDOW * channels(heads)
    total, ps = sum(lens), c + heads
    gen = torch.Generator(device=hs.DEV).manual_seed(33)
    p = baseline_layer(heads, 3300)
    w = hs.Weights(p)

    def draw(rows):
        P = torch.empty(rows, ps, device=hs.DEV, dtype=torch.bfloat16)
        A = torch.empty(rows, heads * DK, device=hs.DEV, dtype=torch.bfloat16)
        G = torch.empty(rows, heads * DV, device=hs.DEV, dtype=torch.bfloat16)
        for r0 in range(0, rows, 16384):       # in slices: the f32 temporaries stay small
            r1 = min(rows, r0 + 16384)
            P[r0:r1] = torch.randn(r1 - r0, ps, device=hs.DEV, generator=gen).to(torch.bfloat16)
            sp = torch.clamp(torch.nn.functional.softplus(torch.randn(r1 - r0, heads * DK, device=hs.DEV, generator=gen)), max=4.999)
            A[r0:r1] = (torch.log(sp / 5.0) - torch.log1p(-sp / 5.0)).to(torch.bfloat16)
            G[r0:r1] = torch.randn(r1 - r0, heads * DV, device=hs.DEV, generator=gen).to(torch.bfloat16)
        return P, A, G

    # the pool: one KDA layer, bf16 states, five slots
    layout = KvLayout(kda_layers=1, dsa_layers=1, kda_state_bf16=True)
    pool = KvPool(layout, slots=5, pages=4 * layout.mark_pages() + 3)
    kvs = [pool.slot() for _ in range(5)]
    state16, conv16 = pool.state.view(torch.bfloat16), pool.conv.view(torch.bfloat16)
    conv16[:] = torch.randn(5 * cw, device=hs.DEV, generator=gen).to(torch.bfloat16)
    conv_start = conv16.clone()
    soff = [kvs[s].state_at() // 2 for s in slots]       # element offsets of the slots' regions
    coff = [kvs[s].conv_at() // 2 for s in slots]
    assert soff == [s * n for s in slots] and coff == [s * cw for s in slots]

    # 1. the prior prefixes, from empty slots, with the bf16 state of the pool
    Pp, Ap, Gp = draw(sum(prefix))
    outp = torch.zeros(sum(prefix), heads * DV, device=hs.DEV, dtype=torch.bfloat16)
    meta_p = hs.BatchMeta(prefix, coff, soff)
    ws_bytes = ffi.glm53f_kda_prefill_workspace_bytes(heads, 4, 1024)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=hs.DEV)
    hs.check(ffi.glm53f_kda_prefill_batch_bf16state(
        heads, 4, hs.ptr(meta_p.cu_rows), max(prefix), hs.ptr(Pp), ps, c, hs.ptr(Ap), heads * DK, hs.ptr(Gp), heads * DV,
        hs.ptr(conv16), hs.ptr(meta_p.conv_off), hs.ptr(w.conv_w), hs.ptr(state16), hs.ptr(state16),
        hs.ptr(meta_p.state_off), *w.args(), hs.ptr(outp), heads * DV, 0, hs.ptr(ws), ws_bytes, None), "prefix prefill")
    hs.sync()
    cup = np.concatenate([[0], np.cumsum(prefix)])
    p4 = hs.subset_params(p, sub)
    for i, s in enumerate(slots):
        pre = hs.subset_rows(heads, sub, Pp, Ap, Gp, int(cup[i]), int(cup[i + 1]))
        lit = o.literal_chain(p4, hs.subset_conv(heads, sub, conv_start[s * cw:(s + 1) * cw]),
                              np.zeros(state_len(4), np.float32), pre, threads=4)
        got = hs.subset_state(heads, sub, state16[s * n:(s + 1) * n])
        # a bf16 state rounded after every chunk against the unrounded oracle: the storage format's bound
        assert hs.rel_err(got, lit.state) <= 2.0 ** -7, f"prefix of request {i}"

    # 2. mark, overwrite, rewind: the prompts continue from restored snapshots
    saved_state, saved_conv = state16.clone(), conv16.clone()
    marks = []
    for i, s in enumerate(slots):
        kvs[s].tokens = prefix[i]
        marks.append(kvs[s].mark())
    state16[:] = torch.randn(5 * n, device=hs.DEV, generator=gen).to(torch.bfloat16)
    conv16[:] = torch.randn(5 * cw, device=hs.DEV, generator=gen).to(torch.bfloat16)
    for i, s in enumerate(slots):
        kvs[s].tokens = prefix[i] + 5
        kvs[s].rewind(prefix[i], marks[i])
    hs.sync()
    for s in slots:
        assert torch.equal(state16[s * n:(s + 1) * n], saved_state[s * n:(s + 1) * n]), f"slot {s}: restored state"
        assert torch.equal(conv16[s * cw:(s + 1) * cw], saved_conv[s * cw:(s + 1) * cw]), f"slot {s}: restored window"
    del Pp, Ap, Gp, outp, saved_state, saved_conv

    # 3. the packed prompts with an f32 carried state, bf16 states back into the pool
    P, A, G = draw(total)
    out = torch.zeros(total, heads * DV, device=hs.DEV, dtype=torch.bfloat16)
    conv_before = conv16.clone()
    state32 = state16.float()
    state_before = state32.clone()
    meta = hs.BatchMeta(lens, coff, soff)
    assert list(meta.cu_host) == [0, 131072, 151552, 155648, 156425]
    ws_bytes = ffi.glm53f_kda_prefill_workspace_bytes(heads, 4, 2048)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=hs.DEV)
    hs.check(ffi.glm53f_kda_prefill_batch(
        heads, 4, hs.ptr(meta.cu_rows), max(lens), hs.ptr(P), ps, c, hs.ptr(A), heads * DK, hs.ptr(G), heads * DV,
        hs.ptr(conv16), hs.ptr(meta.conv_off), hs.ptr(w.conv_w), hs.ptr(state32), hs.ptr(state32),
        hs.ptr(meta.state_off), *w.args(), hs.ptr(out), heads * DV, 0, hs.ptr(ws), ws_bytes, None), "prefill_batch")
    hs.sync()
    state16.copy_(state32.to(torch.bfloat16))              # the write-back to the slot pool
    cu = meta.cu_host
    for i, s in enumerate(slots):
        r0, r1 = int(cu[i]), int(cu[i + 1])
        rq = hs.subset_rows(heads, sub, P, A, G, r0, r1)
        lit = o.literal_chain(p4, hs.subset_conv(heads, sub, conv_before[s * cw:(s + 1) * cw]),
                              hs.subset_state(heads, sub, state_before[s * n:(s + 1) * n]), rq, threads=4)
        got32 = hs.subset_state(heads, sub, state32[s * n:(s + 1) * n])
        got16 = hs.subset_state(heads, sub, state16[s * n:(s + 1) * n])
        es = hs.rel_err(got32, lit.state)
        u, nd = hs.ulps(got16, o.bf16_round(lit.state))
        print(f"config 3, request {i} ({lens[i]} rows, heads {sub}): f32 state {es:.2e} rel (bar 1e-3); pool state vs "
              f"bf16(f32 oracle): {nd} of {got16.size} differ, max {u} ulp; raw {hs.rel_err(got16, lit.state):.2e} rel")
        # Per head. The conv's one bf16 rounding falls the other way on the device than on the host for about one
        # channel value in 10^5 (SiLU through the hardware's exp and reciprocal; the reference notes the same of its
        # kernels, tests/gpu.rs:326-331). Such a value in one of a prompt's last rows, before decay has forgotten it,
        # moves that head's state by up to 2^-9 of a value row times beta: measured 2.2e-4 on one head of the long
        # prompt, 1e-6 on every other. So: the north-star bar on every head, f32-class on the typical one.
        per = [hs.rel_err(got32.reshape(len(sub), -1)[j], lit.state.reshape(len(sub), -1)[j]) for j in range(len(sub))]
        print(f"    per head: {[f'{e:.1e}' for e in per]}")
        assert es <= 1e-3 and float(np.median(per)) <= 1e-5, i
        assert nd <= 2e-3 * got16.size, i                      # roundings that fall the other way
        assert hs.rel_err(got16, lit.state) <= 2.0 ** -8, i    # one rounding to bf16
        got_out = hs.subset_out(heads, sub, out[r0:r1])
        check_outputs(got_out, lit.out, f"config 3, request {i}")
        far = np.flatnonzero(np.abs(got_out.astype(np.float64) - lit.out.astype(np.float64)) > 2e-2)
        if far.size:
            # An output beyond 2e-2 is allowed above only as a two-step event of the contract's double rounding. Whose
            # event it is: the f32 chain kernel (a different kernel, row by row, no chunking, no fp16 anywhere) over
            # the same rows of the same heads, from the same restored snapshot. If the chain's output at that place
            # is off the oracle's as well, the read-out sits on a rounding boundary of the contract itself.
            ch = hs.chain_gpu(p4, hs.subset_conv(heads, sub, conv_before[s * cw:(s + 1) * cw]),
                              hs.subset_state(heads, sub, state_before[s * n:(s + 1) * n]), rq, want_saves=False)
            for j in far:
                row, col = divmod(int(j), len(sub) * DV)
                print(f"    output beyond 2e-2 at row {row}, head {sub[col // DV]}, value {col % DV}: oracle "
                      f"{lit.out.reshape(-1)[j]:.6f} (read-out {lit.y.reshape(-1)[j]:.6f}), prefill {got_out.reshape(-1)[j]:.6f}, "
                      f"chain kernel {ch.out.reshape(-1)[j]:.6f}; the chain kernel differs from the oracle in "
                      f"{int((hs.bf16_steps(ch.out, lit.out).reshape(-1, DV)[j // DV] > 0).sum())} of that row-head's 128 outputs, "
                      f"the prefill in {int((hs.bf16_steps(got_out, lit.out).reshape(-1, DV)[j // DV] > 0).sum())}")
                assert hs.bf16_steps(ch.out, lit.out).reshape(-1)[j] >= 1, "the chain kernel agrees with the oracle there: the event is the prefill's own"
        # the window a request leaves is its last three q | k | v rows
        assert torch.equal(conv16[s * cw:(s + 1) * cw].view(WINDOW, c), P[r1 - 3:r1, :c]), i
    # the slot no request lives in is untouched
    free = (set(range(5)) - set(slots)).pop()
    assert torch.equal(state32[free * n:(free + 1) * n], state_before[free * n:(free + 1) * n])


def test_baseline_config0_shape_through_the_prefill():
    """Config 0's shape (one sequence, T = 256, 64 heads, zero initial state, g = -softplus(N(0, 1)) through the
    lower-bound gate) through the prefill kernels against the literal recurrence; config 0 itself (core-level
    inputs, chunked against recurrent on the CPU) is in test_oracle.py."""
    heads, t = 64, 256
    p = baseline_layer(heads, 100)
    rows = baseline_rows(heads, t, 101)
    conv0 = o.bf16_round(np.random.default_rng(102).standard_normal(WINDOW * channels(heads), dtype=np.float32))
    s0 = np.zeros(state_len(heads), np.float32)
    out, st, conv = hs.prefill_gpu(p, conv0, s0, rows, rows_per_pass=256)
    lit = o.literal_chain(p, conv0, s0, rows, threads=16)
    es = hs.rel_err(st, lit.state)
    print(f"config 0 shape: state {es:.2e} rel")
    assert es <= 1e-5
    check_outputs(out, lit.out, "config 0 shape")
    assert np.array_equal(conv, o.conv_shift(conv0, rows, t))


def test_baseline_config4_verify_checkpoints_and_rollback():
    """48 slots x 16 drafts, 64 heads, bf16 state: every checkpoint equals the pool after that many serial decode
    steps (with the conv shift between them), and the selected state for an accepted length drawn uniformly from
    [0, 16] is that checkpoint, bit for bit; slots that accept nothing keep their state."""
    heads, slots_n, drafts = 64, 48, 16
    c, n, cw = channels(heads), state_len(heads), WINDOW * channels(heads)
    gen = torch.Generator(device=hs.DEV).manual_seed(41)
    p = baseline_layer(heads, 4000)
    w = hs.Weights(p)
    ps = c + heads
    total = slots_n * drafts
    P = torch.randn(total, ps, device=hs.DEV, generator=gen).to(torch.bfloat16)
    sp = torch.clamp(torch.nn.functional.softplus(torch.randn(total, heads * DK, device=hs.DEV, generator=gen)), max=4.999)
    A = (torch.log(sp / 5.0) - torch.log1p(-sp / 5.0)).to(torch.bfloat16)
    G = torch.randn(total, heads * DV, device=hs.DEV, generator=gen).to(torch.bfloat16)
    pool = (torch.randn(slots_n * n, device=hs.DEV, generator=gen) * 0.02).to(torch.bfloat16)
    conv = torch.randn(slots_n * cw, device=hs.DEV, generator=gen).to(torch.bfloat16)
    keep_host = torch.randint(0, drafts + 1, (slots_n,), generator=torch.Generator().manual_seed(42)).tolist()
    keep_host[0], keep_host[1] = 0, drafts
    meta = hs.BatchMeta([drafts] * slots_n, [s * cw for s in range(slots_n)], [s * n for s in range(slots_n)], keep_host)
    out_v = torch.zeros(total, heads * DV, device=hs.DEV, dtype=torch.bfloat16)
    ck = torch.empty(total * n, device=hs.DEV, dtype=torch.bfloat16)
    pool0 = pool.clone()
    hs.check(ffi.glm53f_kda_verify_batch_bf16state(
        heads, slots_n, hs.ptr(meta.cu_rows), hs.ptr(P), ps, c, hs.ptr(A), heads * DK, hs.ptr(G), heads * DV, hs.ptr(conv),
        hs.ptr(meta.conv_off), hs.ptr(w.conv_w), hs.ptr(pool), hs.ptr(meta.state_off), *w.args(), hs.ptr(out_v),
        heads * DV, hs.ptr(ck), None, None, None, None, None), "verify")
    hs.sync()
    assert torch.equal(pool, pool0), "verify leaves the pool untouched"
    # serial decode: step r runs row r of every slot; rows of a step are strided through the packed buffers
    pool_s, conv_s = pool0.clone(), conv.clone()
    one = hs.BatchMeta([1] * slots_n, [s * cw for s in range(slots_n)], [s * n for s in range(slots_n)])
    ckv = ck.view(slots_n, drafts, n)
    for r in range(drafts):
        idx = torch.arange(slots_n, device=hs.DEV) * drafts + r
        Pr, Ar, Gr = P[idx].contiguous(), A[idx].contiguous(), G[idx].contiguous()
        out_r = torch.zeros(slots_n, heads * DV, device=hs.DEV, dtype=torch.bfloat16)
        hs.check(ffi.glm53f_kda_chain_batch_bf16state(
            heads, slots_n, hs.ptr(one.cu_rows), hs.ptr(Pr), ps, c, hs.ptr(Ar), heads * DK, hs.ptr(Gr), heads * DV,
            hs.ptr(conv_s), hs.ptr(one.conv_off), hs.ptr(w.conv_w), hs.ptr(pool_s), hs.ptr(pool_s), hs.ptr(one.state_off),
            *w.args(), hs.ptr(out_r), heads * DV, None, None, None, None, None), "decode")
        hs.check(ffi.glm53f_kda_conv_shift_batch(c, 1, slots_n, hs.ptr(one.cu_rows), hs.ptr(one.keep), hs.ptr(conv_s), 0,
                                                 hs.ptr(one.conv_off), hs.ptr(Pr), 0, ps, None), "shift")
        hs.sync()
        assert torch.equal(ckv[:, r], pool_s.view(slots_n, n)), f"checkpoint after row {r}"
        assert torch.equal(out_r, out_v[idx]), f"outputs of row {r}"
    # the commit by selection
    hs.check(ffi.glm53f_kda_select_batch_bf16state(heads, 1, slots_n, hs.ptr(meta.cu_rows), hs.ptr(meta.keep), hs.ptr(ck), 0,
                                                   hs.ptr(pool), 0, hs.ptr(meta.state_off), None), "select")
    hs.sync()
    pv = pool.view(slots_n, n)
    for s, k in enumerate(keep_host):
        want = pool0.view(slots_n, n)[s] if k == 0 else ckv[s, k - 1]
        assert torch.equal(pv[s], want), (s, k)
