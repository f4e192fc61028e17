"""The kernels driven with the reference engine's buffers and strides, as glm53f-forward packs them
(crates/glm53f-forward/src/forward.rs:3476-3767 for a layer, :1936-2040 for the commit; kv.rs:10-12 for the arenas):

* state arena `[slots][layers][64][128][128]` bf16 and conv arena `[slots][layers][3][24576]`: a layer's base is
  `arena + j * per_layer`, a slot's offset `slot * layers * per_layer`, so a layer's slots lie `layers` states apart;
* projection rows `p` of 24,640 columns with the beta logits behind q|k|v (`b_off = 24,576`);
* `a` and the output gate interleaved in one buffer `ag` of 16,384 columns (`g = ag + 8192`, both strides 16,384);
* a verify round keeps every layer's `p` rows and replay saves (`[layers][verify rows][...]`) for the commit, which
  replays all layers in one launch with per-layer strides and shifts all conv windows in another.

Each engine-layout call is held, bit for bit, to the same work done one layer and one request at a time on dense
buffers (which the other GPU tests hold to the oracle), and the bf16 states to the oracle directly.
"""
import numpy as np
import pytest
import torch

from glm53f_kda import DK, DV, WINDOW, channels, ffi, state_len
from oracle import kda_oracle as o

import harness as hs

pytestmark = pytest.mark.gpu

H, L, SLOTS = 64, 3, 5
C, N, CW = channels(H), state_len(H), WINDOW * channels(H)
P_COLS, WIDTH = C + H, H * DK
DEV = hs.DEV


class Engine:
    """The arenas, the per-layer weights and the row buffers of a small engine."""

    def __init__(self, seed):
        g = torch.Generator(device=DEV).manual_seed(seed)
        self.g = g
        self.state = (torch.randn(SLOTS * L * N, device=DEV, generator=g) * 0.05).to(torch.bfloat16)
        self.conv = torch.randn(SLOTS * L * CW, device=DEV, generator=g).to(torch.bfloat16)
        self.layers = [o.synth_layer(H, seed + 10 * j) for j in range(L)]
        self.w = [hs.Weights(p) for p in self.layers]

    def rows(self, total):
        """One layer's input rows in the engine's packing: (p, ag, out)."""
        g = self.g
        p = torch.randn(total, P_COLS, device=DEV, generator=g).to(torch.bfloat16)
        ag = torch.randn(total, 2 * WIDTH, device=DEV, generator=g).to(torch.bfloat16)
        out = torch.zeros(total, WIDTH, device=DEV, dtype=torch.bfloat16)
        return p, ag, out

    def meta(self, slots, lens, keep=None):
        return hs.BatchMeta(lens, [s * L * CW for s in slots], [s * L * N for s in slots], keep)

    def slot_state(self, arena, slot, j):
        return arena[(slot * L + j) * N:(slot * L + j + 1) * N]

    def slot_conv(self, arena, slot, j):
        return arena[(slot * L + j) * CW:(slot * L + j + 1) * CW]


def row_args(p, ag, first=0):
    return [hs.ptr(p, first * P_COLS), P_COLS, C, hs.ptr(ag, first * 2 * WIDTH), 2 * WIDTH,
            hs.ptr(ag, first * 2 * WIDTH + WIDTH), 2 * WIDTH]


def dense_request(eng, j, p, ag, r0, n, state, conv):
    """The same rows on dense, separate buffers, one request, through the batch entry point with batch 1.
    Returns (out, state after, saves) with the state/conv given as 1-D bf16 tensors (not modified)."""
    pd = p[r0:r0 + n].contiguous()
    a = ag[r0:r0 + n, :WIDTH].contiguous()
    gt = ag[r0:r0 + n, WIDTH:].contiguous()
    out = torch.zeros(n, WIDTH, device=DEV, dtype=torch.bfloat16)
    st = state.clone()
    cu = torch.tensor([0, n], dtype=torch.int32, device=DEV)
    zero = torch.zeros(1, dtype=torch.int64, device=DEV)
    sv = hs.Saves(H, max(n, 1))
    w = eng.w[j]
    code = ffi.glm53f_kda_chain_batch_bf16state(
        H, 1, hs.ptr(cu), hs.ptr(pd), P_COLS, C, hs.ptr(a), WIDTH, hs.ptr(gt), WIDTH, hs.ptr(conv), hs.ptr(zero),
        hs.ptr(w.conv_w), hs.ptr(st), hs.ptr(st), hs.ptr(zero), *w.args(), hs.ptr(out), WIDTH, *sv.args(), None)
    hs.check(code, "dense chain")
    hs.sync()
    return out, st, sv


def test_decode_round_in_the_engine_arenas():
    """forward.rs:3669-3760 with mode Decode: chain in place on the arena, then the conv shift with keep = rows."""
    eng = Engine(100)
    slots, lens = [3, 0, 4], [1, 1, 1]
    meta = eng.meta(slots, lens)
    state0, conv0 = eng.state.clone(), eng.conv.clone()
    for j in range(L):
        p, ag, out = eng.rows(meta.total)
        w = eng.w[j]
        st_l, cv_l = hs.ptr(eng.state, j * N), hs.ptr(eng.conv, j * CW)
        hs.check(ffi.glm53f_kda_chain_batch_bf16state(
            H, meta.batch, hs.ptr(meta.cu_rows), *row_args(p, ag), cv_l, hs.ptr(meta.conv_off), hs.ptr(w.conv_w),
            st_l, st_l, hs.ptr(meta.state_off), *w.args(), hs.ptr(out), WIDTH, None, None, None, None, None), "chain")
        hs.check(ffi.glm53f_kda_conv_shift_batch(C, 1, meta.batch, hs.ptr(meta.cu_rows), hs.ptr(meta.keep), cv_l, 0,
                                                 hs.ptr(meta.conv_off), hs.ptr(p), 0, P_COLS, None), "conv shift")
        hs.sync()
        for i, s in enumerate(slots):
            r0 = int(meta.cu_host[i])
            o1, s1, _ = dense_request(eng, j, p, ag, r0, 1, eng.slot_state(state0, s, j), eng.slot_conv(conv0, s, j))
            assert torch.equal(out[r0:r0 + 1], o1), (j, s)
            assert torch.equal(eng.slot_state(eng.state, s, j), s1), (j, s)
            want_conv = torch.cat([eng.slot_conv(conv0, s, j).view(WINDOW, C)[1:], p[r0:r0 + 1, :C]])
            assert torch.equal(eng.slot_conv(eng.conv, s, j).view(WINDOW, C), want_conv), (j, s)
    # Slots outside the batch are untouched, in every layer.
    for s in (1, 2):
        assert torch.equal(eng.state[s * L * N:(s + 1) * L * N], state0[s * L * N:(s + 1) * L * N])
        assert torch.equal(eng.conv[s * L * CW:(s + 1) * L * CW], conv0[s * L * CW:(s + 1) * L * CW])


def test_verify_round_and_commit_over_all_layers():
    """forward.rs:3669-3716 with mode Verify (state_out NULL, saves and p kept per layer), then the commit of
    forward.rs:1980-2040: replay_batch_bf16state over all layers and conv_shift_batch over all layers, with a keep
    per request. Held to serial single-row decode steps of the kept prefix, and to the checkpoint + select path."""
    eng = Engine(200)
    slots, lens, keep = [2, 4, 0, 1], [8, 5, 8, 3], [3, 0, 8, 1]
    meta = eng.meta(slots, lens, keep)
    vr = meta.total
    state0, conv0 = eng.state.clone(), eng.conv.clone()
    vp = torch.zeros(L, vr, P_COLS, device=DEV, dtype=torch.bfloat16)
    vk = torch.zeros(L, vr, WIDTH, device=DEV)
    vv = torch.zeros(L, vr, WIDTH, device=DEV, dtype=torch.bfloat16)
    vg = torch.zeros(L, vr, WIDTH, device=DEV)
    vb = torch.zeros(L, vr, H, device=DEV)
    ckpt = torch.zeros(L, vr, N, device=DEV, dtype=torch.bfloat16)
    ags, outs, outs_ck = [], [], []
    for j in range(L):
        p, ag, out = eng.rows(vr)
        vp[j] = p
        ags.append(ag)
        w = eng.w[j]
        common = [H, meta.batch, hs.ptr(meta.cu_rows), *row_args(vp[j], ag), hs.ptr(eng.conv, j * CW),
                  hs.ptr(meta.conv_off), hs.ptr(w.conv_w), hs.ptr(eng.state, j * N)]
        hs.check(ffi.glm53f_kda_chain_batch_bf16state(
            *common, None, hs.ptr(meta.state_off), *w.args(), hs.ptr(out), WIDTH, hs.ptr(vk[j]), hs.ptr(vv[j]),
            hs.ptr(vg[j]), hs.ptr(vb[j]), None), "verify chain")
        out_ck = torch.zeros_like(out)
        hs.check(ffi.glm53f_kda_verify_batch_bf16state(
            *common, hs.ptr(meta.state_off), *w.args(), hs.ptr(out_ck), WIDTH, hs.ptr(ckpt[j]), None, None, None,
            None, None), "verify with checkpoints")
        outs.append(out)
        outs_ck.append(out_ck)
    hs.sync()
    # A verify round writes neither arena.
    assert torch.equal(eng.state, state0) and torch.equal(eng.conv, conv0)
    for j in range(L):
        assert torch.equal(outs[j], outs_ck[j]), j

    # The commit, all layers in two launches.
    by_select = eng.state.clone()
    hs.check(ffi.glm53f_kda_replay_batch_bf16state(
        H, L, meta.batch, hs.ptr(meta.cu_rows), hs.ptr(meta.keep), hs.ptr(eng.state), hs.ptr(eng.state), N,
        hs.ptr(meta.state_off), hs.ptr(vk), hs.ptr(vv), hs.ptr(vg), hs.ptr(vb), vr * WIDTH, vr * H, None), "replay")
    hs.check(ffi.glm53f_kda_conv_shift_batch(C, L, meta.batch, hs.ptr(meta.cu_rows), hs.ptr(meta.keep),
                                             hs.ptr(eng.conv), CW, hs.ptr(meta.conv_off), hs.ptr(vp), vr * P_COLS,
                                             P_COLS, None), "conv shift")
    hs.check(ffi.glm53f_kda_select_batch_bf16state(H, L, meta.batch, hs.ptr(meta.cu_rows), hs.ptr(meta.keep),
                                                   hs.ptr(ckpt), vr * N, hs.ptr(by_select), N, hs.ptr(meta.state_off),
                                                   None), "select")
    hs.sync()
    assert torch.equal(by_select, eng.state), "commit by selection == commit by replay"

    for j in range(L):
        for i, s in enumerate(slots):
            r0, k = int(meta.cu_host[i]), keep[i]
            st, cv = eng.slot_state(state0, s, j).clone(), eng.slot_conv(conv0, s, j).clone()
            for r in range(k):      # serial decode steps over the kept prefix
                o1, st, _ = dense_request(eng, j, vp[j], ags[j], r0 + r, 1, st, cv)
                assert torch.equal(outs[j][r0 + r:r0 + r + 1], o1), (j, s, r)
                cv = torch.cat([cv.view(WINDOW, C)[1:], vp[j][r0 + r:r0 + r + 1, :C]]).reshape(-1)
            assert torch.equal(eng.slot_state(eng.state, s, j), st), (j, s)
            assert torch.equal(eng.slot_conv(eng.conv, s, j), cv), (j, s)
    # The oracle on one (layer, request): the replay of the device's saves from the arena state.
    j, i = 1, 0
    s, r0, k = slots[i], int(meta.cu_host[i]), keep[i]
    sv = o.Saves(H, lens[i], hs.back(vk[j][r0:r0 + lens[i]]), hs.back(vv[j][r0:r0 + lens[i]]),
                 hs.back(vg[j][r0:r0 + lens[i]]), hs.back(vb[j][r0:r0 + lens[i]]))
    want = o.replay(hs.back(eng.slot_state(state0, s, j)), sv, k, bf16_state=True)
    assert np.array_equal(hs.bits(want), hs.bits(hs.back(eng.slot_state(eng.state, s, j))))


def test_prefill_round_in_the_engine_arenas():
    """forward.rs:3577-3666: the chunked prefill of a batch, bf16 states in the arena, windows advanced in place."""
    eng = Engine(300)
    slots, lens = [4, 1], [150, 37]
    meta = eng.meta(slots, lens)
    state0, conv0 = eng.state.clone(), eng.conv.clone()
    per = 64
    ws_bytes = ffi.glm53f_kda_prefill_workspace_bytes(H, meta.batch, per)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=DEV)
    for j in range(L):
        p, ag, out = eng.rows(meta.total)
        w = eng.w[j]
        st_l, cv_l = hs.ptr(eng.state, j * N), hs.ptr(eng.conv, j * CW)
        hs.check(ffi.glm53f_kda_prefill_batch_bf16state(
            H, meta.batch, hs.ptr(meta.cu_rows), max(lens), *row_args(p, ag), cv_l, hs.ptr(meta.conv_off),
            hs.ptr(w.conv_w), st_l, st_l, hs.ptr(meta.state_off), *w.args(), hs.ptr(out), WIDTH, 0, hs.ptr(ws),
            ws_bytes, None), "prefill")
        hs.sync()
        for i, s in enumerate(slots):
            r0, n = int(meta.cu_host[i]), lens[i]
            # the same request alone, on dense buffers
            pd, a = p[r0:r0 + n].contiguous(), ag[r0:r0 + n, :WIDTH].contiguous()
            gt = ag[r0:r0 + n, WIDTH:].contiguous()
            o1 = torch.zeros(n, WIDTH, device=DEV, dtype=torch.bfloat16)
            s1, c1 = eng.slot_state(state0, s, j).clone(), eng.slot_conv(conv0, s, j).clone()
            cu = torch.tensor([0, n], dtype=torch.int32, device=DEV)
            zero = torch.zeros(1, dtype=torch.int64, device=DEV)
            hs.check(ffi.glm53f_kda_prefill_batch_bf16state(
                H, 1, hs.ptr(cu), n, hs.ptr(pd), P_COLS, C, hs.ptr(a), WIDTH, hs.ptr(gt), WIDTH, hs.ptr(c1),
                hs.ptr(zero), hs.ptr(w.conv_w), hs.ptr(s1), hs.ptr(s1), hs.ptr(zero), *w.args(), hs.ptr(o1), WIDTH, 0,
                hs.ptr(ws), ws_bytes, None), "dense prefill")
            hs.sync()
            assert torch.equal(out[r0:r0 + n], o1), (j, s)
            assert torch.equal(eng.slot_state(eng.state, s, j), s1), (j, s)
            assert torch.equal(eng.slot_conv(eng.conv, s, j), c1), (j, s)
            assert torch.equal(c1.view(WINDOW, C), p[r0 + n - 3:r0 + n, :C]), (j, s)
        if j == 0:
            # against the oracle: the FP32 recurrence from the arena's state, final state rounded to bf16
            i, s = 1, slots[1]
            r0, n = int(meta.cu_host[i]), lens[i]
            rows = o.Rows(H, n, hs.back(p[r0:r0 + n, :C]), hs.back(ag[r0:r0 + n, :WIDTH]), hs.back(p[r0:r0 + n, C:]),
                          hs.back(ag[r0:r0 + n, WIDTH:]))
            lit = o.literal_chain(eng.layers[j], hs.back(eng.slot_conv(conv0, s, j)),
                                  hs.back(eng.slot_state(state0, s, j)), rows)
            assert hs.rel_err(hs.back(eng.slot_state(eng.state, s, j)), lit.state) <= 1e-2
            assert hs.rel_err(hs.back(out[r0:r0 + n]), lit.out) <= 2.0 ** -7
    for s in (0, 2, 3):
        assert torch.equal(eng.state[s * L * N:(s + 1) * L * N], state0[s * L * N:(s + 1) * L * N])
