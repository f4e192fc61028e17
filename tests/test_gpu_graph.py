"""The entry points under HIP graph capture: they allocate nothing and clear nothing with memsets, so a decode
round and a prefill call can be recorded once and replayed. Every replay is checked against the same calls made
eagerly, bit for bit, with eager work and synchronisations between the replays.

(The reference has no graph path; its engine launches eagerly on one stream. This is what a caller that captures
its step gets from this library.)
"""
import numpy as np
import pytest
import torch

from glm53f_kda import WINDOW, channels, ffi, state_len
from oracle import kda_oracle as o

import harness as hs
from harness import ptr

pytestmark = pytest.mark.gpu

NO_SAVES = (None, None, None, None)


def decode_call(p, w, pool, slots, sr, meta, stream):
    """One decode round in place: chain and conv window advance in one launch per call."""
    fn = ffi.glm53f_kda_chain_shift_batch_bf16state if pool.bf16 else ffi.glm53f_kda_chain_shift_batch
    hs.check(fn(p.heads, meta.batch, ptr(meta.cu_rows), *sr.row_args(), ptr(pool.conv), ptr(meta.conv_off),
                ptr(w.conv_w), ptr(pool.state), ptr(pool.state), ptr(meta.state_off), *w.args(), ptr(sr.out),
                sr.out_stride, *NO_SAVES, stream), "chain_shift_batch")


@pytest.mark.parametrize("bf16_state", [True, False])
def test_a_captured_decode_round_replays_like_eager_rounds(bf16_state):
    heads, slots_n, slots = 8, 5, [3, 0, 4]
    p = o.synth_layer(heads, 1500)
    w = hs.Weights(p)
    reqs = [o.synth_rows(heads, 1, 1510 + i) for i in range(len(slots))]
    sr = hs.StagedRows(hs.stack_rows(reqs))
    pool_g, pool_e = hs.Pool(heads, slots_n, bf16_state, 1520), hs.Pool(heads, slots_n, bf16_state, 1520)
    meta = hs.BatchMeta([1] * len(slots), [pool_g.conv_off(s) for s in slots], [pool_g.state_off(s) for s in slots])
    sr_e = hs.StagedRows(hs.stack_rows(reqs))           # the eager rounds write their own output rows

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        decode_call(p, w, pool_g, slots, sr, meta, torch.cuda.current_stream().cuda_stream)
    for replay in range(1, 4):
        graph.replay()
        # eager work between the replays, on the default stream, and a synchronisation
        decode_call(p, w, pool_e, slots, sr_e, meta, None)
        junk = torch.randn(1 << 16, device=hs.DEV).sum().item()
        hs.sync()
        assert np.isfinite(junk)
        assert torch.equal(pool_g.state, pool_e.state), f"state after replay {replay}"
        assert torch.equal(pool_g.conv, pool_e.conv), f"conv windows after replay {replay}"
        assert np.array_equal(hs.bits(sr.out_np()), hs.bits(sr_e.out_np())), f"outputs of replay {replay}"


def test_a_captured_prefill_call_replays_like_eager_calls():
    heads, t = 4, 150
    p = o.synth_layer(heads, 1600)
    w = hs.Weights(p)
    rows = o.synth_rows(heads, t, 1610)
    n, cw = state_len(heads), WINDOW * channels(heads)
    conv0, s0 = o.synth_conv_window(heads, 1620), o.synth_state(heads, 1620, 0.5)
    ws_bytes = ffi.glm53f_kda_prefill_workspace_bytes(heads, 1, 128)        # two passes over the 150 rows
    assert ws_bytes > 0

    def buffers():
        return dict(sr=hs.StagedRows(rows), conv=hs.to_bf16(conv0), state=hs.to_f32(s0),
                    ws=torch.empty(ws_bytes // 4, dtype=torch.float32, device=hs.DEV))

    def call(b, stream):
        # the state is carried in place and the conv window advances, so every call starts where the last ended
        hs.check(ffi.glm53f_kda_prefill(heads, t, *b["sr"].row_args(), ptr(b["conv"]), ptr(w.conv_w), ptr(b["state"]),
                                        ptr(b["state"]), *w.args(), ptr(b["sr"].out), b["sr"].out_stride, 0, ptr(b["ws"]),
                                        ws_bytes, stream), "prefill")

    hs.check(ffi.glm53f_kda_init(), "init")             # the per-device set-up, so that the capture holds launches only
    hs.check(ffi.glm53f_kda_init(), "init again")
    g, e = buffers(), buffers()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(g, torch.cuda.current_stream().cuda_stream)
    for replay in range(1, 4):
        graph.replay()
        call(e, None)
        junk = torch.randn(1 << 16, device=hs.DEV).sum().item()
        hs.sync()
        assert np.isfinite(junk)
        assert torch.equal(g["state"], e["state"]), f"state after replay {replay}"
        assert torch.equal(g["conv"], e["conv"]), f"conv window after replay {replay}"
        assert np.array_equal(hs.bits(g["sr"].out_np()), hs.bits(e["sr"].out_np())), f"outputs of replay {replay}"
    assert len(g["conv"]) == cw and len(g["state"]) == n


def test_a_captured_verify_and_select_round_replays_like_eager_rounds():
    """The speculative round as a caller would capture it: the checkpointing verify of every request's drafts, then
    the select that commits each request's accepted prefix into the pool. The accepted lengths are device data, so
    one recorded graph serves rounds with different outcomes: `keep` is rewritten between the replays."""
    heads, slots_n, slots, lens = 8, 5, [3, 0, 4], [4, 1, 6]
    keeps = [[4, 0, 3], [1, 1, 6], [0, 0, 0]]
    p = o.synth_layer(heads, 1700)
    w = hs.Weights(p)
    reqs = [o.synth_rows(heads, n, 1710 + i) for i, n in enumerate(lens)]
    n = state_len(heads)

    def buffers():
        pool = hs.Pool(heads, slots_n, True, 1720)
        sr = hs.StagedRows(hs.stack_rows(reqs))
        meta = hs.BatchMeta(lens, [pool.conv_off(s) for s in slots], [pool.state_off(s) for s in slots], keeps[0])
        ck = torch.zeros(meta.total * n, dtype=torch.bfloat16, device=hs.DEV)
        return dict(pool=pool, sr=sr, meta=meta, ck=ck)

    def call(b, stream):
        pool, sr, meta, ck = b["pool"], b["sr"], b["meta"], b["ck"]
        hs.check(ffi.glm53f_kda_verify_batch_bf16state(
            heads, meta.batch, ptr(meta.cu_rows), *sr.row_args(), ptr(pool.conv), ptr(meta.conv_off), ptr(w.conv_w),
            ptr(pool.state), ptr(meta.state_off), *w.args(), ptr(sr.out), sr.out_stride, ptr(ck), *NO_SAVES, stream),
            "verify")
        hs.check(ffi.glm53f_kda_select_batch_bf16state(heads, 1, meta.batch, ptr(meta.cu_rows), ptr(meta.keep), ptr(ck),
                                                       ck.numel(), ptr(pool.state), pool.state.numel(),
                                                       ptr(meta.state_off), stream), "select")

    g, e = buffers(), buffers()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(g, torch.cuda.current_stream().cuda_stream)
    for replay, keep in enumerate(keeps, 1):
        for b in (g, e):                                # this round's outcome, written where the graph reads it
            b["meta"].keep.copy_(torch.tensor(keep, dtype=torch.int32))
        graph.replay()
        call(e, None)
        junk = torch.randn(1 << 16, device=hs.DEV).sum().item()
        hs.sync()
        assert np.isfinite(junk)
        assert torch.equal(g["pool"].state, e["pool"].state), f"pool after replay {replay}"
        assert torch.equal(g["ck"], e["ck"]), f"checkpoints of replay {replay}"
        assert np.array_equal(hs.bits(g["sr"].out_np()), hs.bits(e["sr"].out_np())), f"outputs of replay {replay}"
    # the rounds did commit something: the pool has moved from where it started
    assert not torch.equal(g["pool"].state, hs.Pool(heads, slots_n, True, 1720).state)
