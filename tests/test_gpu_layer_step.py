"""A KDA layer's step from the normed hidden rows to the attention output, as the reference's engine issues it
(crates/glm53f-forward/src/forward.rs:3494-3542 the projections, :3672-3705 the core's arguments, :3772-3789 the
output projection), through the GEMM engine's dispatch (glm53f_forward.gemm) and the KDA entry points, with the
engine's packing: p rows with the beta logits behind q|k|v, the gates' two halves interleaved in one buffer `ag`
written by a grouped GEMM, `a` and `g` read out of it with its row stride.

What is held: a verify window of 16 slots x 4 draft rows (64 rows through the projections: the GEMM for 9 to 64 rows,
four row tiles; the core with a checkpoint after every row) gives, bit for bit, what four decode rounds of 16 rows give
(the same GEMM with one row tile; the core as chain + conv window advance): attention outputs, checkpoints against
states. The reference has this property up to 8 rows through its GEMV (gemm.rs:1-8); the GEMM for 9 to 64 rows keeps
a row's bits independent of the rows beside it, which carries it to 64. The projections themselves are held to exact
arithmetic in test_gpu_gemm_skinny.py, the core to the oracle in test_gpu_chain.py.
"""
import pytest
import torch

from glm53f_kda import DK, WINDOW, channels, ffi, state_len
from glm53f_forward.gemm import Bf16Mat, Gemm, GemmPolicy
from oracle import kda_oracle as o

import harness as hs

pytestmark = pytest.mark.gpu
DEV = hs.DEV
H, HIDDEN, POOL = 16, 512, 20
WIDTH, C = H * DK, channels(H)
P_COLS, N, CW = C + H, state_len(H), WINDOW * channels(H)


class Layer:
    def __init__(self, seed):
        g = torch.Generator(device=DEV).manual_seed(seed)
        rnd = lambda *s, scale: (torch.randn(*s, device=DEV, generator=g) * scale).to(torch.bfloat16)
        self.qkvb, self.fga = rnd(P_COLS, HIDDEN, scale=0.05), rnd(2 * DK, HIDDEN, scale=0.05)
        self.fgb, self.o = rnd(2, WIDTH, DK, scale=0.1), rnd(HIDDEN, WIDTH, scale=0.02)
        self.kda = hs.Weights(o.synth_layer(H, seed))
        self.state = rnd(POOL * N, scale=0.05)
        self.conv = rnd(POOL * CW, scale=1.0)

    @staticmethod
    def buffers(rows):
        z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)
        return dict(p=z(rows, P_COLS), fga=z(rows, 2 * DK), ag=z(rows, 2 * WIDTH), kda_out=z(rows, WIDTH), out=z(rows, HIDDEN))

    def launch(self, gemm, x, meta, state, conv, b, ckpt=None, stream=None):
        """The step's five launches on `stream` into the row buffers b (no allocation, no synchronisation)."""
        rows = x.shape[0]
        p, fga, ag, kda_out, out = b["p"], b["fga"], b["ag"], b["kda_out"], b["out"]
        gemm.bf16(hs.ptr(x), HIDDEN, 0, Bf16Mat.of(self.qkvb), rows, hs.ptr(p), P_COLS, 0, False, stream)
        gemm.bf16(hs.ptr(x), HIDDEN, 0, Bf16Mat.of(self.fga), rows, hs.ptr(fga), 2 * DK, 0, False, stream)
        gemm.bf16(hs.ptr(fga), 2 * DK, DK, Bf16Mat.of(self.fgb), rows, hs.ptr(ag), 2 * WIDTH, WIDTH, False, stream)
        w = self.kda
        head = [H, meta.batch, hs.ptr(meta.cu_rows), hs.ptr(p), P_COLS, C, hs.ptr(ag), 2 * WIDTH, hs.ptr(ag, WIDTH), 2 * WIDTH,
                hs.ptr(conv), hs.ptr(meta.conv_off), hs.ptr(w.conv_w), hs.ptr(state)]
        if ckpt is None:
            hs.check(ffi.glm53f_kda_chain_shift_batch_bf16state(*head, hs.ptr(state), hs.ptr(meta.state_off), *w.args(),
                                                                hs.ptr(kda_out), WIDTH, None, None, None, None, stream), "decode")
        else:
            hs.check(ffi.glm53f_kda_verify_batch_bf16state(*head, hs.ptr(meta.state_off), *w.args(), hs.ptr(kda_out), WIDTH,
                                                           hs.ptr(ckpt), None, None, None, None, stream), "verify")
        gemm.bf16(hs.ptr(kda_out), WIDTH, 0, Bf16Mat.of(self.o), rows, hs.ptr(out), HIDDEN, 0, False, stream)

    def step(self, gemm, x, meta, state, conv, ckpt=None):
        """x [rows][HIDDEN] bf16 -> attention output [rows][HIDDEN]; ckpt None: a decode round in place (chain + conv
        window advance), else a verify window that leaves state and conv alone and writes a checkpoint per row."""
        b = self.buffers(x.shape[0])
        self.launch(gemm, x, meta, state, conv, b, ckpt)
        hs.sync()
        return b["out"], b["p"]


@pytest.mark.parametrize("slots_n,drafts", [(16, 4), (5, 3), (3, 16)])
def test_a_verify_window_gives_the_bits_of_serial_decode_rounds(slots_n, drafts):
    layer = Layer(31 + slots_n)
    gemm = Gemm(GemmPolicy(gemv_max_rows=0))       # every row count through the GEMM for 9 to 64 rows
    g = torch.Generator(device=DEV).manual_seed(7)
    slots = torch.randperm(POOL, generator=torch.Generator().manual_seed(3))[:slots_n].tolist()
    rows = slots_n * drafts
    x = torch.randn(rows, HIDDEN, device=DEV, generator=g).to(torch.bfloat16)          # row = slot index * drafts + t
    window = hs.BatchMeta([drafts] * slots_n, [s * CW for s in slots], [s * N for s in slots])
    ckpt = torch.zeros(rows, N, dtype=torch.bfloat16, device=DEV)
    state0, conv0 = layer.state.clone(), layer.conv.clone()
    out_v, p_v = layer.step(gemm, x, window, layer.state, layer.conv, ckpt)
    assert torch.equal(layer.state, state0) and torch.equal(layer.conv, conv0), "a verify window writes neither"

    one = hs.BatchMeta([1] * slots_n, [s * CW for s in slots], [s * N for s in slots])
    state, conv = state0.clone(), conv0.clone()
    for t in range(drafts):
        xt = x.view(slots_n, drafts, HIDDEN)[:, t].contiguous()
        out_d, p_d = layer.step(gemm, xt, one, state, conv)
        assert torch.equal(p_d, p_v.view(slots_n, drafts, P_COLS)[:, t]), f"projection rows of step {t}"
        assert torch.equal(out_d, out_v.view(slots_n, drafts, HIDDEN)[:, t]), f"attention output of step {t}"
        for i, s in enumerate(slots):
            assert torch.equal(state[s * N:(s + 1) * N], ckpt[i * drafts + t]), f"checkpoint {t} of slot {s}"
    # the commit by selection of every draft leaves the pool where the decode rounds left it
    by_select = state0.clone()
    hs.check(ffi.glm53f_kda_select_batch_bf16state(H, 1, slots_n, hs.ptr(window.cu_rows), hs.ptr(window.keep), hs.ptr(ckpt), 0,
                                                   hs.ptr(by_select), 0, hs.ptr(window.state_off), None), "select")
    hs.sync()
    assert torch.equal(by_select, state)
    untouched = [s for s in range(POOL) if s not in slots]
    for s in untouched:
        assert torch.equal(state[s * N:(s + 1) * N], state0[s * N:(s + 1) * N])


def test_the_default_dispatch_agrees_with_the_reference_dispatch_within_bf16_rounding():
    """Sixteen rows: the GEMM for 9 to 64 rows (default) against the vendor GEMM (the reference's dispatch above 8
    rows). No bit-level contract between the two; the layer's attention outputs agree within the bf16 roundings on
    the way (projection rows, core outputs, output projection)."""
    layer = Layer(77)
    g = torch.Generator(device=DEV).manual_seed(8)
    slots = list(range(16))
    x = torch.randn(16, HIDDEN, device=DEV, generator=g).to(torch.bfloat16)
    one = hs.BatchMeta([1] * 16, [s * CW for s in slots], [s * N for s in slots])
    outs = []
    for policy in (GemmPolicy(), GemmPolicy(skinny_max_rows=0)):
        state, conv = layer.state.clone(), layer.conv.clone()
        outs.append(layer.step(Gemm(policy), x, one, state, conv)[0].float())
    scale = float(outs[1].abs().max())
    worst = float((outs[0] - outs[1]).abs().max())
    print(f"layer output, skinny against vendor GEMM: max |diff| {worst:.3e} at max |out| {scale:.3e}")
    assert worst <= 2.0 ** -5 * scale


@pytest.mark.parametrize("rows", [8, 16])
def test_a_captured_layer_step_replays_like_eager_steps(rows):
    """The step's five launches recorded once (8 rows: the GEMV, whose split projection uses the engine's counters;
    16 rows: the GEMM for 9 to 64 rows) and replayed: nothing on the path allocates or clears with a memset. Every
    replay advances the slots' states and windows, and is held to the same step made eagerly, bit for bit, with eager
    work and synchronisations between the replays."""
    layer_g, layer_e = Layer(91), Layer(91)
    assert torch.equal(layer_g.state, layer_e.state)
    gemm = Gemm()
    g = torch.Generator(device=DEV).manual_seed(9)
    slots = list(range(2, 2 + rows))
    x = torch.randn(rows, HIDDEN, device=DEV, generator=g).to(torch.bfloat16)
    one = hs.BatchMeta([1] * rows, [s * CW for s in slots], [s * N for s in slots])
    bg, be = Layer.buffers(rows), Layer.buffers(rows)
    stream = torch.cuda.Stream()                       # default priority; the legacy default stream cannot be captured
    hs.sync()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            layer_g.launch(gemm, x, one, layer_g.state, layer_g.conv, bg, stream=stream.cuda_stream)
        for replay in range(1, 4):
            graph.replay()
            stream.synchronize()
            layer_e.launch(gemm, x, one, layer_e.state, layer_e.conv, be, stream=stream.cuda_stream)
            junk = torch.randn(1 << 16, device=DEV).sum().item()
            hs.sync()
            assert junk == junk
            assert torch.equal(bg["out"], be["out"]), f"attention outputs of replay {replay}"
            assert torch.equal(layer_g.state, layer_e.state), f"states after replay {replay}"
            assert torch.equal(layer_g.conv, layer_e.conv), f"conv windows after replay {replay}"
    assert not torch.equal(layer_g.state, Layer(91).state)
