#!/usr/bin/env python3
"""Benchmark of the KDA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only decode|prefill|verify|mark|gemv|layer|copy]

Prints ONE JSON line. The headline `value` is the decode step's state traffic in GB/s in the 16-slot decode configuration
(16 slots x 1 token out of a 48-slot bf16 pool, 64 heads, 34 layers each with its own pool so the working set
exceeds the last-level cache); a "step" is one decode step over the 34 KDA layers: per layer the chain and the
conv window advance, in one launch (the reference engine's two launches per layer are timed beside it as
`decode_two_launches`). The same line carries the chunked prefill (T = 8192 as four sequential 2048-row calls on one
slot) and the checkpointing verify (48 slots x 16 drafts) under `prefill` and `verify`, each with its
own roofline object, and the CPU oracle timed on this host's cores as `cpu_baseline`.

Inputs are synthetic with the distributions of the benchmark definition, generated on the GPU; all buffers are resident in HBM
before the timed region. Kernel durations are measured with events on the stream the kernels are launched on.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "glm53f-afd_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import numpy as np
import torch

from glm53f_kda import DK, DV, HEADS, LAYERS, WINDOW, channels, ffi, state_len

# HBM bytes per launch from the FETCH_SIZE and WRITE_SIZE counters (one rocprofv3 --pmc run each over this
# script's legs, scaled by the same counters over the 1 GiB copy of --only copy: x2.00 and x1.00). Measured
# offline; the summaries are kept in profiles/.
TRAFFIC_BYTES = {
    "decode_chain": (36_798 + 33_024) * 1024,            # per plain chain launch, 16 slots x 1 row
    "verify_chain": (167_884 + 1_585_673) * 1024,        # per chain launch, 48 slots x 16 rows with checkpoints
    # two passes of 1024 rows (intra read + written, inter read + written) and one norm launch
    "prefill_2048_rows": (2 * (74_010 + 141_329 + 144_138 + 20_482) + 65_755 + 32_912) * 1024,
    "mark_state_pages": (69_928 + 70_854) * 1024,
    "gemv_kda_proj_1row": (197_941 + 48) * 1024,         # per launch: the weights once, the activations, the outputs
    "skinny_kda_proj_16rows": (198_481 + 770) * 1024,    # per launch: the weights once, sixteen rows' activations per workgroup (L2), the outputs
}
HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16/fp16 MFMA, published
DEV = "cuda:0"

METRIC = "KDA prefill tok/s per layer at T=8K (MFMA %); decode state GB/s at 16 slots"
PREFILL_DTYPE = "fp16 hi/lo operand pairs on the MFMA (f32-class products), f32 accumulate"


def ptr(t, off=0):
    return None if t is None else t.data_ptr() + off * t.element_size()


class Layer:
    """Random-init weights of one KDA layer with the gate mapping of the benchmark definition: A_log = 0, dt_bias = 0, so
    g = -5 * sigmoid(a) and a = logit(softplus(z) / 5) gives g = -softplus(z)."""

    def __init__(self, heads, gen):
        c = channels(heads)
        self.heads = heads
        self.conv_w = ((torch.rand(c * 4, device=DEV, generator=gen) - 0.5) * 1.2).to(torch.bfloat16)
        self.a_log = torch.zeros(heads, device=DEV)
        self.dt_bias = torch.zeros(heads * DK, device=DEV)
        self.norm_w = torch.ones(DV, device=DEV, dtype=torch.bfloat16)
        self.eps, self.lower = 1e-5, -5.0

    def args(self):
        return [ptr(self.a_log), ptr(self.dt_bias), ptr(self.norm_w), self.eps, self.lower]


class RowBuffers:
    """Projection rows in the engine's layout: p rows of C + H columns (beta logits behind q|k|v), dense a, g,
    out (reference call site: crates/glm53f-forward/src/forward.rs:3672-3705)."""

    def __init__(self, heads, rows, gen):
        c = channels(heads)
        self.heads, self.rows = heads, rows
        self.p_stride = c + heads
        self.p = torch.randn(rows, self.p_stride, device=DEV, generator=gen).to(torch.bfloat16)
        z = torch.randn(rows, heads * DK, device=DEV, generator=gen, dtype=torch.float64)
        sp = torch.clamp(torch.nn.functional.softplus(z), max=4.999)
        self.a = (torch.log(sp / 5.0) - torch.log1p(-sp / 5.0)).to(torch.bfloat16)
        self.g = torch.randn(rows, heads * DV, device=DEV, generator=gen).to(torch.bfloat16)
        self.out = torch.zeros(rows, heads * DV, device=DEV, dtype=torch.bfloat16)

    def row_args(self, first=0):
        c = channels(self.heads)
        return [ptr(self.p, first * self.p_stride), self.p_stride, c, ptr(self.a, first * self.heads * DK),
                self.heads * DK, ptr(self.g, first * self.heads * DV), self.heads * DV]

    def out_args(self, first=0):
        return [ptr(self.out, first * self.heads * DV), self.heads * DV]

    def to_oracle(self, o, first, n):
        c, h = channels(self.heads), self.heads
        f = lambda t: t.float().cpu().numpy().reshape(-1)
        return o.Rows(h, n, f(self.p[first:first + n, :c]), f(self.a[first:first + n]),
                      f(self.p[first:first + n, c:c + h]), f(self.g[first:first + n]))


PREWARM_S = 0.1


def timed(fn, steps, warmup, stream):
    """W untimed calls, then exactly K timed ones between events on `stream`; returns ms per call. Before the W
    calls the same work runs untimed for a tenth of a second: a leg that starts on an idle GPU otherwise measures
    the clocks ramping up (the decode step read 5 % slower as the first leg than as a later one)."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < PREWARM_S:
        fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(steps):
        fn()
    e1.record(stream)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def check(code, what):
    if code != 0:
        raise RuntimeError(f"{what} returned {code}")


# ------------------------------------------------------------------------------------------------ decode

def bench_decode(steps, warmup, stream, cpu=True):
    heads, slots_n, batch, layers = HEADS, 48, 16, LAYERS
    gen = torch.Generator(device=DEV).manual_seed(1)
    layer = Layer(heads, gen)
    n, cw = state_len(heads), WINDOW * channels(heads)
    # One pool per layer, as the engine lays them out: 34 x 48 x 2 MiB of bf16 state.
    pools = (torch.randn(layers, slots_n * n, device=DEV, generator=gen) * 0.02).to(torch.bfloat16)
    convs = torch.randn(layers, slots_n * cw, device=DEV, generator=gen).to(torch.bfloat16)
    rows = RowBuffers(heads, batch, gen)
    perm = torch.randperm(slots_n, generator=torch.Generator().manual_seed(2))[:batch]
    cu = torch.arange(batch + 1, dtype=torch.int32, device=DEV)
    keep = torch.ones(batch, dtype=torch.int32, device=DEV)
    soff = (perm.to(torch.int64) * n).to(DEV)
    coff = (perm.to(torch.int64) * cw).to(DEV)
    st = stream.cuda_stream
    c = channels(heads)

    # Argument lists are built once: the timed loops only make the C calls.
    chain_fn, shift_fn = ffi.glm53f_kda_chain_batch_bf16state, ffi.glm53f_kda_conv_shift_batch
    chain_args = [(heads, batch, ptr(cu), *rows.row_args(), ptr(convs[l]), ptr(coff),
                   ptr(layer.conv_w), ptr(pools[l]), ptr(pools[l]), ptr(soff),
                   *layer.args(), *rows.out_args(), None, None, None, None, st) for l in range(layers)]
    shift_args = [(c, 1, batch, ptr(cu), ptr(keep), ptr(convs[l]), 0, ptr(coff), ptr(rows.p), 0, rows.p_stride, st)
                  for l in range(layers)]

    def chain(l):
        check(chain_fn(*chain_args[l]), "chain")

    def shift(l):
        check(shift_fn(*shift_args[l]), "conv_shift")

    fused_fn = ffi.glm53f_kda_chain_shift_batch_bf16state

    def step():                                          # a decode round as one launch per layer
        for l in range(layers):
            check(fused_fn(*chain_args[l]), "chain + shift")

    def step_two_launches():                             # the reference engine's two launches per layer
        for l in range(layers):
            chain(l)
            shift(l)

    def chains_only():
        for l in range(layers):
            chain(l)

    ms_step = timed(step, steps, warmup, stream)
    ms_two = timed(step_two_launches, steps, max(1, warmup // 2), stream)
    ms_chain = timed(chains_only, steps, max(1, warmup // 2), stream) / layers
    state_bytes = 2 * batch * n * 2                      # read + write of 16 bf16 states: 67,108,864 B
    # What this box moves for the same traffic with no arithmetic behind it: the same entry point with requests of
    # zero rows copies every slot's state to `state_out` (here the next layer's pool), same workgroups, same
    # nontemporal accesses, 32 MiB read and 32 MiB written per launch.
    cu0 = torch.zeros(batch + 1, dtype=torch.int32, device=DEV)
    copy_args = [(heads, batch, ptr(cu0), *rows.row_args(), ptr(convs[l]), ptr(coff), ptr(layer.conv_w), ptr(pools[l]),
                  ptr(pools[(l + 1) % layers]), ptr(soff), *layer.args(), *rows.out_args(), None, None, None, None, st)
                 for l in range(layers)]

    def copies_only():
        for l in range(layers):
            check(chain_fn(*copy_args[l]), "chain (zero rows)")

    ms_copy = timed(copies_only, steps, max(1, warmup // 2), stream) / layers
    res = {
        "ms_per_step": ms_step,
        "state_GBps": layers * state_bytes / (ms_step * 1e-3) / 1e9,
        "two_launches": {"ms_per_step": ms_two, "state_GBps": layers * state_bytes / (ms_two * 1e-3) / 1e9,
                         "what": "glm53f_kda_chain_batch_bf16state then glm53f_kda_conv_shift_batch per layer"},
        "roofline": {"bound": "hbm", "achieved": state_bytes / (ms_chain * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": state_bytes / (ms_chain * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                     "traffic": TRAFFIC_BYTES["decode_chain"],
                     "kernel": "chain_kernel<bf16>", "bytes_per_launch": state_bytes,
                     "us_per_launch": ms_chain * 1e3,
                     "same_traffic_copy": {"us_per_launch": ms_copy * 1e3, "GBps": state_bytes / (ms_copy * 1e-3) / 1e9,
                                           "what": "zero-row requests: each slot's state copied to another pool"}},
    }
    if cpu:
        from oracle import kda_oracle as o
        threads = min(16, os.cpu_count() or 1)
        p = o.LayerParams(heads, layer.conv_w.float().cpu().numpy(), layer.a_log.cpu().numpy(),
                          layer.dt_bias.cpu().numpy(), layer.norm_w.float().cpu().numpy())
        reqs = [rows.to_oracle(o, i, 1) for i in range(batch)]
        pool0 = pools[0].float().cpu().numpy()
        conv0 = convs[0].float().cpu().numpy()
        slots = perm.tolist()

        def one_layer_step(nthreads):
            for i, s in enumerate(slots):
                o.chain_bf16_state(p, conv0[s * cw:(s + 1) * cw], pool0[s * n:(s + 1) * n], reqs[i], threads=nthreads)

        def seconds_per_step(nthreads, budget):
            one_layer_step(nthreads)
            t0, reps = time.perf_counter(), 0
            while reps < 1 or time.perf_counter() - t0 < budget:
                one_layer_step(nthreads)
                reps += 1
            return (time.perf_counter() - t0) / reps, reps

        dt, reps = seconds_per_step(threads, 2.0)
        dt1, reps1 = seconds_per_step(1, 2.0)
        res["cpu_baseline"] = {"value": state_bytes / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                               "sample": f"config 1 in full for one layer (16 slots x 64 heads x 1 row, bf16-rounded "
                                         f"state), {reps} repetitions of the C oracle chain_bf16_state, "
                                         f"{dt * 1e3:.2f} ms per layer-step",
                               "single_thread": {"value": state_bytes / dt1 / 1e9, "unit": "GB/s", "cores": 1,
                                                 "sample": f"the same layer-step on one thread, {reps1} repetitions, "
                                                           f"{dt1 * 1e3:.2f} ms"}}
    return res


# ------------------------------------------------------------------------------------------------ prefill

def bench_prefill(steps, warmup, stream, cpu=True):
    """benchmark configuration 2: one prompt of 8192 rows as four sequential calls of 2048 rows on one slot (the
    engine's lanes), 64 heads, f32 carried state, conv and output gate included."""
    heads, total, lane_rows = HEADS, 8192, 2048
    gen = torch.Generator(device=DEV).manual_seed(3)
    layer = Layer(heads, gen)
    n, cw = state_len(heads), WINDOW * channels(heads)
    rows = RowBuffers(heads, total, gen)
    state = torch.zeros(n, device=DEV)
    conv = torch.randn(cw, device=DEV, generator=gen).to(torch.bfloat16)
    ws_bytes = ffi.glm53f_kda_prefill_workspace_bytes(heads, 1, lane_rows)
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=DEV)
    st = stream.cuda_stream
    fn = ffi.glm53f_kda_prefill
    calls = [(heads, lane_rows, *rows.row_args(first), ptr(conv), ptr(layer.conv_w), ptr(state), ptr(state),
              *layer.args(), *rows.out_args(first), 0, ptr(ws), ws_bytes, st) for first in range(0, total, lane_rows)]

    def step():
        for a in calls:
            check(fn(*a), "prefill")

    ms = timed(step, steps, warmup, stream)
    flops = total * 11_709_099 / 64 * heads        # dense MFMA count of the chunk-64 form: 11.71 MFLOP per token
    io_bytes = total * 98_432                       # compulsory row traffic: p, a, g in, out
    res = {
        "tok_per_s_per_layer": total / (ms * 1e-3), "ms_per_8192_tokens": ms,
        "roofline": {"bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12, "peak": MFMA_BF16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": TRAFFIC_BYTES["prefill_2048_rows"], "traffic_unit": "B per 2048-row call (2 intra + 2 inter launches of 1024 rows, 1 norm launch)",
                     "kernel": "prefill (intra + inter + norm with the conv window advance, whole call)",
                     "flops_per_token": 11_709_099, "hbm_GBps_compulsory": io_bytes / (ms * 1e-3) / 1e9,
                     "hbm_frac": io_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS},
        "config": {"workload": "benchmark configuration 2: T=8192 as 4 calls of 2048 rows on one slot, H=64, chunk 64, "
                               "bf16 rows, f32 state, conv + output gate", "workspace_MB": ws_bytes / 1e6},
        "dtype": PREFILL_DTYPE,
    }
    if cpu:
        from oracle import kda_oracle as o
        threads = min(16, os.cpu_count() or 1)
        sample = 2048
        p = o.LayerParams(heads, layer.conv_w.float().cpu().numpy(), layer.a_log.cpu().numpy(),
                          layer.dt_bias.cpu().numpy(), layer.norm_w.float().cpu().numpy())
        rq = rows.to_oracle(o, 0, sample)
        conv0 = conv.float().cpu().numpy()
        s0 = np.zeros(n, np.float32)
        t0 = time.perf_counter()
        o.literal_chain(p, conv0, s0, rq, threads=threads)
        dt = time.perf_counter() - t0
        t0 = time.perf_counter()
        o.prefill(p, conv0, s0, rq, threads=threads)
        dt_chunked = time.perf_counter() - t0
        sample1 = 256
        rq1 = rows.to_oracle(o, 0, sample1)
        t0 = time.perf_counter()
        o.literal_chain(p, conv0, s0, rq1, threads=1)
        dt1 = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": sample / dt, "unit": "tok/s per layer", "cores": threads, "kind": "port",
                               "sample": f"the first {sample}-row lane of the prompt, 64 heads, the C oracle's literal "
                                         f"recurrent chain (conv, gates, delta rule, gated norm), {dt:.2f} s wall; "
                                         f"its chunked form takes {dt_chunked:.2f} s "
                                         f"({sample / dt_chunked:.0f} tok/s per layer)",
                               "single_thread": {"value": sample1 / dt1, "unit": "tok/s per layer", "cores": 1,
                                                 "sample": f"the first {sample1} rows, 64 heads, the literal chain on one "
                                                           f"thread, {dt1:.2f} s wall"}}
    return res


# ------------------------------------------------------------------------------------------------ verify

def bench_verify(steps, warmup, stream, saves_form=True, cpu=True):
    """benchmark configuration 4: 48 slots x 16 draft rows, bf16 state, a checkpoint after every row, then the commit by
    selection with an accepted length per slot drawn uniformly from [0, 16]."""
    heads, slots_n, drafts, layers = HEADS, 48, 16, 2
    gen = torch.Generator(device=DEV).manual_seed(4)
    layer = Layer(heads, gen)
    n, cw = state_len(heads), WINDOW * channels(heads)
    pools = (torch.randn(layers, slots_n * n, device=DEV, generator=gen) * 0.02).to(torch.bfloat16)
    convs = torch.randn(layers, slots_n * cw, device=DEV, generator=gen).to(torch.bfloat16)
    rows = RowBuffers(heads, slots_n * drafts, gen)
    ck = torch.empty(layers, slots_n * drafts * n, dtype=torch.bfloat16, device=DEV)
    cu = (torch.arange(slots_n + 1, dtype=torch.int32) * drafts).to(DEV)
    keep = torch.randint(0, drafts + 1, (slots_n,), generator=torch.Generator().manual_seed(5)).to(torch.int32).to(DEV)
    soff = (torch.arange(slots_n, dtype=torch.int64) * n).to(DEV)
    coff = (torch.arange(slots_n, dtype=torch.int64) * cw).to(DEV)
    st = stream.cuda_stream
    vfn, sfn = ffi.glm53f_kda_verify_batch_bf16state, ffi.glm53f_kda_select_batch_bf16state
    vargs = [(heads, slots_n, ptr(cu), *rows.row_args(), ptr(convs[l]), ptr(coff), ptr(layer.conv_w), ptr(pools[l]),
              ptr(soff), *layer.args(), *rows.out_args(), ptr(ck[l]), None, None, None, None, st)
             for l in range(layers)]
    sargs = [(heads, 1, slots_n, ptr(cu), ptr(keep), ptr(ck[l]), 0, ptr(pools[l]), 0, ptr(soff), st)
             for l in range(layers)]
    it = [0]

    def verify():
        check(vfn(*vargs[it[0] % layers]), "verify")
        it[0] += 1

    def select():
        check(sfn(*sargs[it[0] % layers]), "select")
        it[0] += 1

    ms_v = timed(verify, steps, warmup, stream)
    ms_s = timed(select, steps, warmup, stream)
    vbytes = slots_n * n * 2 + slots_n * drafts * n * 2          # read 48 states + write 48 x 16 checkpoints
    kept = int((keep > 0).sum().item())
    sbytes = 2 * kept * n * 2

    res = {
        "verify_ms_per_layer": ms_v, "select_ms_per_layer": ms_s,
        "roofline": {"bound": "hbm", "achieved": vbytes / (ms_v * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": vbytes / (ms_v * 1e-3) / 1e9 / HBM_PEAK_GBPS, "traffic": TRAFFIC_BYTES["verify_chain"],
                     "kernel": "chain_kernel<bf16> with checkpoints", "bytes_per_launch": vbytes},
        "select_GBps": sbytes / (ms_s * 1e-3) / 1e9,
        "config": {"workload": "benchmark configuration 4: verify 48 slots x 16 drafts, bf16 state, per-row checkpoints; "
                               "select with keep ~ U{0..16}", "kept_slots": kept},
    }
    res["dtype"] = "f32 arithmetic, bf16-stored state"
    if cpu:
        # The CPU path of the same step on a bounded sample: 4 of the 48 slots, all 16 drafts, 64 heads, the state
        # rounded to bf16 after every row (the checkpoints are those states).
        from oracle import kda_oracle as o
        threads = min(16, os.cpu_count() or 1)
        p = o.LayerParams(heads, layer.conv_w.float().cpu().numpy(), layer.a_log.cpu().numpy(),
                          layer.dt_bias.cpu().numpy(), layer.norm_w.float().cpu().numpy())
        sample_slots = 4
        pool0, conv0 = pools[0].float().cpu().numpy(), convs[0].float().cpu().numpy()
        reqs = [rows.to_oracle(o, s * drafts, drafts) for s in range(sample_slots)]

        def sample(nthreads):
            for s in range(sample_slots):
                o.chain_bf16_state(p, conv0[s * cw:(s + 1) * cw], pool0[s * n:(s + 1) * n], reqs[s], threads=nthreads)

        def seconds(nthreads):
            sample(nthreads)
            t0, reps = time.perf_counter(), 0
            while reps < 1 or time.perf_counter() - t0 < 2.0:
                sample(nthreads)
                reps += 1
            return (time.perf_counter() - t0) / reps

        sbytes_cpu = vbytes * sample_slots / slots_n
        dt, dt1 = seconds(threads), seconds(1)
        res["cpu_baseline"] = {"value": sbytes_cpu / dt / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
                               "sample": f"{sample_slots} of the 48 slots x 16 drafts x 64 heads, the C oracle's "
                                         f"chain_bf16_state, counted with the verify pass's bytes for those slots "
                                         f"({sbytes_cpu / 1e6:.0f} MB), {dt * 1e3:.1f} ms",
                               "single_thread": {"value": sbytes_cpu / dt1 / 1e9, "unit": "GB/s", "cores": 1,
                                                 "sample": f"the same sample on one thread, {dt1 * 1e3:.1f} ms"}}
    if not saves_form:
        return res

    # The reference's form of the same round, for comparison: the verify pass saves every row's replay inputs
    # (1,284 B per row and head) and leaves the state alone; the commit replays the kept prefix from the saves.
    total = slots_n * drafts
    sk = torch.empty(layers, total * heads * DK, device=DEV)
    sv = torch.empty(layers, total * heads * DV, device=DEV, dtype=torch.bfloat16)
    sg = torch.empty(layers, total * heads * DK, device=DEV)
    sb = torch.empty(layers, total * heads, device=DEV)
    cfn, rfn = ffi.glm53f_kda_chain_batch_bf16state, ffi.glm53f_kda_replay_batch_bf16state
    cargs = [(heads, slots_n, ptr(cu), *rows.row_args(), ptr(convs[l]), ptr(coff), ptr(layer.conv_w), ptr(pools[l]),
              None, ptr(soff), *layer.args(), *rows.out_args(), ptr(sk[l]), ptr(sv[l]), ptr(sg[l]), ptr(sb[l]), st)
             for l in range(layers)]
    rargs = [(heads, 1, slots_n, ptr(cu), ptr(keep), ptr(pools[l]), ptr(pools[l]), 0, ptr(soff), ptr(sk[l]), ptr(sv[l]),
              ptr(sg[l]), ptr(sb[l]), 0, 0, st) for l in range(layers)]

    def verify_saves():
        check(cfn(*cargs[it[0] % layers]), "chain with saves")
        it[0] += 1

    def replay():
        check(rfn(*rargs[it[0] % layers]), "replay")
        it[0] += 1

    ms_vs = timed(verify_saves, steps, warmup, stream)
    ms_r = timed(replay, steps, warmup, stream)
    res["saves_form"] = {"verify_ms_per_layer": ms_vs, "replay_commit_ms_per_layer": ms_r,
                         "bytes_saved_per_layer": total * heads * 1284}
    return res


# ------------------------------------------------------------------------------------------------ mark

def bench_mark(steps, warmup, stream, cpu=True):
    """A snapshot mark of one slot's positional state in the full model's layout with bf16 KDA states (195 pool
    pages of 394,944 B; crates/glm53f-forward/src/kv.rs:412-478): the scatter of the state's 180 whole pages
    alone, and the whole save and load as the engine runs them (page list upload, two launches, three copies of
    partial pages)."""
    from glm53f_forward import ffi as rf
    from glm53f_forward.kv import KvPool
    from glm53f_forward.kvplan import KvLayout
    l = KvLayout().with_kda_state_bf16(True)
    # Four slots and four marks in turn: 8 x 73 MiB, so that no call finds its source in the 256 MB Infinity Cache
    # because the call before it left it there.
    nslots = 4
    pool = KvPool(l, slots=nslots, pages=2 * nslots * l.mark_pages() + 16)
    gen = torch.Generator(device=DEV).manual_seed(6)
    pool.state[:] = torch.randint(0, 256, (pool.state.numel(),), device=DEV, generator=gen, dtype=torch.uint8)
    # every other page of the pool, so that a mark's pages are no contiguous run
    held = [pool.alloc.alloc() for _ in range(2 * nslots * l.mark_pages())]
    for pg in held[1::2]:
        pool.alloc.release(pg)
    kvs = [pool.slot() for _ in range(nslots)]
    marks = [kv.mark() for kv in kvs]
    torch.cuda.synchronize()
    pb, full = l.page_bytes, l.kda_state_bytes() // l.page_bytes
    lists = [torch.tensor(m.page_list(), dtype=torch.int32, device=DEV) for m in marks]
    calls = [[ptr(pool.state, kv.state_at()), pb, ptr(ix), ptr(pool.pages), pb, full, pb, None]
             for kv, ix in zip(kvs, lists)]
    turn = [0]

    def scatter():
        turn[0] += 1
        check(rf.glm53f_fwd_scatter_rows(*calls[turn[0] % nslots]), "scatter rows")

    def save():
        turn[0] += 1
        kvs[turn[0] % nslots].copy_mark(marks[turn[0] % nslots], True)

    def load():
        turn[0] += 1
        kvs[turn[0] % nslots].copy_mark(marks[turn[0] % nslots], False)

    ms_scatter = timed(scatter, steps, warmup, stream)
    ms_save = timed(save, steps, warmup, stream)
    ms_load = timed(load, steps, warmup, stream)
    m = marks[0]
    moved = 2 * full * pb
    res = {"config": {"workload": "snapshot mark of one slot, full model layout with bf16 KDA states: 195 pages "
                                  "of 394,944 B (181 state, 13 conv, 1 tails), pages not contiguous; four slots and marks in turn",
                      "mark_bytes": l.mark_bytes(), "pages": l.mark_pages()},
           "scatter_state_pages_ms": ms_scatter, "save_ms": ms_save, "load_ms": ms_load,
           "save_GBps": 2 * l.mark_bytes() / (ms_save * 1e-3) / 1e9,
           "load_GBps": 2 * l.mark_bytes() / (ms_load * 1e-3) / 1e9,
           "roofline": {"bound": "hbm", "kernel": "long_rows_kernel", "achieved": moved / (ms_scatter * 1e-3) / 1e9,
                        "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                        "frac": moved / (ms_scatter * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                        "traffic": TRAFFIC_BYTES["mark_state_pages"],
                        "algorithmic_bytes": moved}}
    if cpu:
        from oracle import rows_oracle as ro
        image = np.random.default_rng(3).integers(0, 256, l.mark_bytes(), dtype=np.uint8)
        s, c = l.kda_state_bytes(), l.conv_bytes()
        arenas = [(image[:s], 0), (image[s:s + c], 0), (image[s + c:], 0)]
        host_pages = np.zeros(pool.pages.numel(), dtype=np.uint8)
        reps, t0 = 0, time.perf_counter()
        while reps < 3 or time.perf_counter() - t0 < 2.0:
            ro.copy_mark(l.mark_regions(), pb, m.page_list(), host_pages, arenas, True)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = {"value": 2 * l.mark_bytes() / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"{reps} saves of the same mark by the numpy restatement (page-sized memcpys)"}
    return res


# ------------------------------------------------------------------------------------------------ gemv

def bench_gemv(steps, warmup, stream, cpu=True):
    """The BF16 projections next to the KDA core in a decode or verify step (crates/glm53f-forward/src/forward.rs:
    3494-3542, :3772-3789): the input projection 4096 -> 24,640 with 1 and 8 rows, and the output projection
    8192 -> 4096. Weights streamed from HBM once per call; four copies of each weight in turn, so that no call finds
    its weight in the 256 MB Infinity Cache."""
    from glm53f_forward import ffi as fwd
    gen = torch.Generator(device=DEV).manual_seed(8)
    partials = torch.empty(1 << 20, dtype=torch.float32, device=DEV)
    sync = torch.zeros(1 << 16, dtype=torch.int32, device=DEV)
    res = {"config": {"workload": "BF16 GEMV, weights [n][k] streamed once: kda_proj 4096 -> 24,640 and o_proj "
                                  "8192 -> 4096 with 1 to 8 rows; four weight copies in turn"}}
    copies = 4
    for name, n, k, rows in (("kda_proj_1row", 24_640, 4096, 1), ("kda_proj_4rows", 24_640, 4096, 4),
                             ("kda_proj_8rows", 24_640, 4096, 8), ("o_proj_1row", 4096, 8192, 1),
                             ("o_proj_8rows", 4096, 8192, 8)):
        w = (torch.randn(copies, n, k, device=DEV, generator=gen) * 0.02).to(torch.bfloat16)
        x = torch.randn(8, k, device=DEV, generator=gen).to(torch.bfloat16)
        out = torch.zeros(8, n, dtype=torch.bfloat16, device=DEV)
        ksplit = fwd.glm53f_fwd_gemv_ksplit(1, n, k)
        calls = [(ptr(x), k, 0, ptr(w[c]), k, 0, 1, rows, n, k, ksplit, ptr(partials), ptr(sync), ptr(out), 0, n, 0,
                  stream.cuda_stream) for c in range(copies)]
        turn = [0]

        def one():
            turn[0] += 1
            check(fwd.glm53f_fwd_gemv_bf16(*calls[turn[0] % copies]), "gemv")

        ms = timed(one, steps, warmup, stream)
        wbytes = n * k * 2
        res[name] = {"us": ms * 1e3, "weight_GBps": wbytes / (ms * 1e-3) / 1e9, "ksplit": ksplit,
                     "frac_of_hbm_peak": wbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
        del w
    # the same projections over a 2048-row prefill segment: the vendor GEMM (hipBLASLt through torch.matmul), which the
    # reference's engine takes above 8 rows (cuBLAS there); reported, not built here
    for name, n, k in (("kda_proj_2048rows_vendor_gemm", 24_640, 4096), ("o_proj_2048rows_vendor_gemm", 4096, 8192)):
        w = (torch.randn(n, k, device=DEV, generator=gen) * 0.02).to(torch.bfloat16)
        xr = torch.randn(2048, k, device=DEV, generator=gen).to(torch.bfloat16)
        o2 = torch.empty(2048, n, dtype=torch.bfloat16, device=DEV)
        ms = timed(lambda: torch.matmul(xr, w.t(), out=o2), max(2, steps // 4), 2, stream)
        flops = 2.0 * 2048 * n * k
        res[name] = {"us": ms * 1e3, "TFLOPs": flops / (ms * 1e-3) / 1e12,
                     "frac_of_mfma_peak": flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS}
        del w, xr, o2
    r = res["kda_proj_1row"]
    res["roofline"] = {"bound": "hbm", "kernel": "gemv_kernel<1, bf16 out>", "achieved": r["weight_GBps"],
                       "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": r["frac_of_hbm_peak"],
                       "traffic": TRAFFIC_BYTES.get("gemv_kda_proj_1row"), "algorithmic_bytes": 24_640 * 4096 * 2}
    if cpu:
        from oracle import gemv_oracle as go
        rng = np.random.default_rng(2)
        n_s, k = 512, 4096
        wh = go.bf16_round((rng.standard_normal((n_s, k)) * 0.02).astype(np.float32))
        xh = go.bf16_round(rng.standard_normal((1, k)).astype(np.float32))
        reps, t0 = 0, time.perf_counter()
        while reps < 2 or time.perf_counter() - t0 < 2.0:
            go.gemv_bf16(xh, wh, 1)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        res["cpu_baseline"] = {"value": n_s * k * 2 / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"{reps} runs of the numpy model on 512 of the 24,640 outputs, one row"}
    return res


# ------------------------------------------------------------------------------------------------ skinny GEMM

def bench_skinny(steps, warmup, stream):
    """The same projections with 9 to 64 rows (a decode step of more than 8 slots, a verify window): this library's
    weight-streaming GEMM (glm53f_fwd_gemm_bf16_skinny) and, beside it, the vendor GEMM that the reference's dispatch
    takes there (crates/glm53f-forward/src/gemm.rs:228-234). The KDA layer's four projections with the engine's
    strides; four copies of each weight in turn, so that no call finds its weight in the 256 MB Infinity Cache."""
    from glm53f_forward import ffi as fwd
    gen = torch.Generator(device=DEV).manual_seed(9)
    res = {"config": {"workload": "BF16 GEMM with 16 to 64 rows, weights [n][k] streamed once: kda_proj 4096 -> 24,640, "
                                  "o_proj 8192 -> 4096, the gates' 4096 -> 256 and 2 x (128 -> 8192), the LM head "
                                  "4096 -> 151,936; four weight copies in turn (two of the LM head)"}}
    for name, g, n, k, ldx, xgs, ldo, ogs, rows_list in (("kda_proj", 1, 24_640, 4096, 4096, 0, 24_640, 0, (16, 32, 64)),
                                                         ("o_proj", 1, 4096, 8192, 8192, 0, 4096, 0, (16, 64)),
                                                         ("fga", 1, 256, 4096, 4096, 0, 256, 0, (16,)),
                                                         ("fgb", 2, 8192, 128, 256, 128, 16_384, 8192, (16,)),
                                                         # the LM head, which the reference's engine sends through the
                                                         # same BF16 dispatch (gemm.rs:3): 1.24 GB of weights
                                                         ("lm_head", 1, 151_936, 4096, 4096, 0, 151_936, 0, (16,))):
        copies = 4 if n * k < (1 << 28) else 2
        w = torch.empty(copies, g, n, k, dtype=torch.bfloat16, device=DEV)
        flat = w.view(-1)
        for i in range(0, flat.numel(), 1 << 26):               # in slices: the f32 temporaries stay small
            j = min(flat.numel(), i + (1 << 26))
            flat[i:j] = (torch.randn(j - i, device=DEV, generator=gen) * 0.02).to(torch.bfloat16)
        x = torch.randn(64, ldx, device=DEV, generator=gen).to(torch.bfloat16)
        out = torch.zeros(64, ldo, dtype=torch.bfloat16, device=DEV)
        wbytes = g * n * k * 2
        for rows in rows_list:
            calls = [(ptr(x), ldx, xgs, ptr(w[c]), k, n * k, g, rows, n, k, ptr(out), 0, ldo, ogs, stream.cuda_stream)
                     for c in range(copies)]
            turn = [0]

            def one():
                turn[0] += 1
                check(fwd.glm53f_fwd_gemm_bf16_skinny(*calls[turn[0] % copies]), "skinny GEMM")

            ms = timed(one, steps, warmup, stream)
            res[f"{name}_{rows}rows"] = {"us": ms * 1e3, "weight_GBps": wbytes / (ms * 1e-3) / 1e9,
                                         "frac_of_hbm_peak": wbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
            if g == 1:
                def vendor():
                    turn[0] += 1
                    torch.mm(x[:rows, :k], w[turn[0] % copies, 0].t(), out=out[:rows, :n])
                ms = timed(vendor, steps, warmup, stream)
                res[f"{name}_{rows}rows"]["vendor_gemm_us"] = ms * 1e3
        del w
    r = res["kda_proj_16rows"]
    res["roofline"] = {"bound": "hbm", "kernel": "stream_kernel<256 k per chunk, 1 row tile, 8 weight tiles, 4 waves>",
                       "achieved": r["weight_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": r["frac_of_hbm_peak"],
                       "traffic": TRAFFIC_BYTES.get("skinny_kda_proj_16rows"), "algorithmic_bytes": 24_640 * 4096 * 2}
    return res


# ------------------------------------------------------------------------------------------------ decode layer

def bench_layer_decode(steps, warmup, stream):
    """A KDA layer's decode step end to end as the engine issues it (crates/glm53f-forward/src/forward.rs:3494-3542
    the projections, :3672-3705 the core's arguments, :3772-3789 the output projection), over all 34 layers with
    their own weights, states and conv windows (12.8 GB: nothing is found in a cache): per layer
        p   = normed x qkvb^T   [rows][24,640]   (q | k | v | beta logits; b_off = 24,576)
        fga = normed x fga^T    [rows][256]      (the gates' low-rank halves; split K, so it needs scratch)
        ag  = fga x fgb^T       [rows][2 x 8192] (two groups: forget-gate input | output-gate logits, interleaved rows)
        core: chain + conv window advance in one launch on the slots' states (glm53f_kda_chain_shift_batch_bf16state)
        out = kda_out x o^T     [rows][4096]
    Up to 8 rows the projections are this library's GEMV (the split one through glm53f_fwd_gemv_bf16_static, which
    holds its scratch itself); above that the reference's dispatch calls the vendor GEMM (gemm.rs:228-234), and this
    library has its weight-streaming GEMM for 9 to 64 rows (glm53f_fwd_gemm_bf16_skinny). Benchmark configuration
    1's 16 slots are measured with both, and 8 slots beside them for the GEMV path (and with the GEMM for 9 to 64
    rows, which accepts fewer: the reference's bit-level contract with its host model is then given up, a row's
    independence of the rows beside it is not). Each both ways: launched eagerly, and as one captured graph
    replayed."""
    from glm53f_forward import ffi as fwd
    heads, layers, slots_n, hidden = HEADS, LAYERS, 48, 4096
    width, dim = heads * DK, DK                            # 8192, 128
    pcols = 3 * width + heads                              # 24,640
    gen = torch.Generator(device=DEV).manual_seed(11)
    n, cw = state_len(heads), WINDOW * channels(heads)

    def weight(*shape):
        w = torch.empty(*shape, dtype=torch.bfloat16, device=DEV)
        flat = w.view(-1)
        for i in range(0, flat.numel(), 1 << 26):           # in slices: the f32 temporaries stay small
            j = min(flat.numel(), i + (1 << 26))
            flat[i:j] = (torch.randn(j - i, device=DEV, generator=gen) * 0.02).to(torch.bfloat16)
        return w

    w_qkvb, w_fga = weight(layers, pcols, hidden), weight(layers, 2 * dim, hidden)
    w_fgb, w_o = weight(layers, 2, width, dim), weight(layers, hidden, width)
    layer = Layer(heads, gen)
    pools = (torch.randn(layers, slots_n * n, device=DEV, generator=gen) * 0.02).to(torch.bfloat16)
    convs = torch.randn(layers, slots_n * cw, device=DEV, generator=gen).to(torch.bfloat16)
    weight_bytes = (pcols * hidden + 2 * dim * hidden + 2 * width * dim + hidden * width) * 2
    # on a stream of its own (default priority): the legacy default stream cannot be captured
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    st = stream.cuda_stream
    res = {"config": {"workload": "a KDA layer's decode step end to end, 34 layers in turn: kda_proj, the two gate "
                                  "projections, chain + conv window advance, o_proj; engine strides",
                      "weight_bytes_per_layer": weight_bytes}}
    ck = None
    # (slots, rows per slot, who runs the projections, key): one row per slot is a decode step; four rows per slot a
    # verify window (the core is then glm53f_kda_verify_batch_bf16state with a checkpoint after every row, which
    # leaves the slots' states and windows as they are: the commit is the select of the verify leg)
    for slots, per, kind, key in ((16, 1, "skinny", "slots16"), (16, 1, "vendor", "slots16_vendor_gemm"), (8, 1, "gemv", "slots8"),
                                  (8, 1, "skinny", "slots8_skinny_gemm"), (16, 4, "skinny", "verify_16slots_x4"),
                                  (16, 4, "vendor", "verify_16slots_x4_vendor_gemm")):
        batch = slots * per
        normed = torch.randn(batch, hidden, device=DEV, generator=gen).to(torch.bfloat16)
        pbuf = torch.zeros(batch, pcols, dtype=torch.bfloat16, device=DEV)
        fga = torch.zeros(batch, 2 * dim, dtype=torch.bfloat16, device=DEV)
        ag = torch.zeros(batch, 2 * width, dtype=torch.bfloat16, device=DEV)
        kda_out = torch.zeros(batch, width, dtype=torch.bfloat16, device=DEV)
        attn_out = torch.zeros(batch, hidden, dtype=torch.bfloat16, device=DEV)
        perm = torch.randperm(slots_n, generator=torch.Generator().manual_seed(12))[:slots]
        cu = (torch.arange(slots + 1, dtype=torch.int32) * per).to(DEV)
        soff, coff = (perm.to(torch.int64) * n).to(DEV), (perm.to(torch.int64) * cw).to(DEV)
        if per == 1:
            core = ffi.glm53f_kda_chain_shift_batch_bf16state
            core_args = [(heads, slots, ptr(cu), ptr(pbuf), pcols, 3 * width, ptr(ag), 2 * width, ptr(ag, width), 2 * width,
                          ptr(convs[l]), ptr(coff), ptr(layer.conv_w), ptr(pools[l]), ptr(pools[l]), ptr(soff),
                          *layer.args(), ptr(kda_out), width, None, None, None, None, st) for l in range(layers)]
        else:
            if ck is None:
                ck = torch.empty(layers, batch * n, dtype=torch.bfloat16, device=DEV)   # a checkpoint per row and layer
            core = ffi.glm53f_kda_verify_batch_bf16state
            core_args = [(heads, slots, ptr(cu), ptr(pbuf), pcols, 3 * width, ptr(ag), 2 * width, ptr(ag, width), 2 * width,
                          ptr(convs[l]), ptr(coff), ptr(layer.conv_w), ptr(pools[l]), ptr(soff),
                          *layer.args(), ptr(kda_out), width, ptr(ck[l]), None, None, None, None, st) for l in range(layers)]
        gemv = kind != "vendor"
        if kind == "gemv":
            ks = {name: fwd.glm53f_fwd_gemv_ksplit(g, nn, kk) for name, g, nn, kk in
                  (("qkvb", 1, pcols, hidden), ("fga", 1, 2 * dim, hidden), ("fgb", 2, width, dim), ("o", 1, hidden, width))}
            gv = fwd.glm53f_fwd_gemv_bf16_static
            gemv_args = [[
                (ptr(normed), hidden, 0, ptr(w_qkvb[l]), hidden, 0, 1, batch, pcols, hidden, ks["qkvb"], ptr(pbuf), 0, pcols, 0, st),
                (ptr(normed), hidden, 0, ptr(w_fga[l]), hidden, 0, 1, batch, 2 * dim, hidden, ks["fga"], ptr(fga), 0, 2 * dim, 0, st),
                (ptr(fga), 2 * dim, dim, ptr(w_fgb[l]), dim, width * dim, 2, batch, width, dim, ks["fgb"], ptr(ag), 0, 2 * width, width, st),
                (ptr(kda_out), width, 0, ptr(w_o[l]), width, 0, 1, batch, hidden, width, ks["o"], ptr(attn_out), 0, hidden, 0, st),
            ] for l in range(layers)]
        elif kind == "skinny":
            gv = fwd.glm53f_fwd_gemm_bf16_skinny
            gemv_args = [[
                (ptr(normed), hidden, 0, ptr(w_qkvb[l]), hidden, 0, 1, batch, pcols, hidden, ptr(pbuf), 0, pcols, 0, st),
                (ptr(normed), hidden, 0, ptr(w_fga[l]), hidden, 0, 1, batch, 2 * dim, hidden, ptr(fga), 0, 2 * dim, 0, st),
                (ptr(fga), 2 * dim, dim, ptr(w_fgb[l]), dim, width * dim, 2, batch, width, dim, ptr(ag), 0, 2 * width, width, st),
                (ptr(kda_out), width, 0, ptr(w_o[l]), width, 0, 1, batch, hidden, width, ptr(attn_out), 0, hidden, 0, st),
            ] for l in range(layers)]
        ag_f, ag_g = ag[:, :width], ag[:, width:]

        def step():
            for l in range(layers):
                if gemv:
                    a = gemv_args[l]
                    check(gv(*a[0]), "kda_proj")
                    check(gv(*a[1]), "fga")
                    check(gv(*a[2]), "fgb")
                else:
                    torch.mm(normed, w_qkvb[l].t(), out=pbuf)
                    torch.mm(normed, w_fga[l].t(), out=fga)
                    torch.mm(fga[:, :dim], w_fgb[l, 0].t(), out=ag_f)
                    torch.mm(fga[:, dim:], w_fgb[l, 1].t(), out=ag_g)
                check(core(*core_args[l]), "chain + shift")
                if gemv:
                    check(gv(*gemv_args[l][3]), "o_proj")
                else:
                    torch.mm(kda_out, w_o[l].t(), out=attn_out)

        with torch.cuda.stream(stream):
            ms_eager = timed(step, steps, warmup, stream)
            graph = torch.cuda.CUDAGraph()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                step()
            ms_graph = timed(graph.replay, steps, warmup, stream)
        state_bytes = (2 * slots if per == 1 else slots + batch) * n * 2     # read + written | read + checkpoints
        per_layer = weight_bytes + state_bytes
        res[key] = {"projections": {"gemv": "this library's GEMV (glm53f_fwd_gemv_bf16_static)",
                                    "skinny": "this library's GEMM for 9 to 64 rows (glm53f_fwd_gemm_bf16_skinny)",
                                    "vendor": "vendor GEMM (hipBLASLt through torch.mm)"}[kind],
                    "eager_us_per_layer": ms_eager * 1e3 / layers, "graph_us_per_layer": ms_graph * 1e3 / layers,
                    "bytes_per_layer": per_layer, "state_bytes_per_layer": state_bytes,
                    "eager_GBps": per_layer / (ms_eager * 1e-3 / layers) / 1e9,
                    "graph_GBps": per_layer / (ms_graph * 1e-3 / layers) / 1e9}
        best = min(ms_eager, ms_graph)
        res[key]["roofline"] = {"bound": "hbm", "achieved": per_layer / (best * 1e-3 / layers) / 1e9, "peak": HBM_PEAK_GBPS,
                                "unit": "GB/s", "frac": per_layer / (best * 1e-3 / layers) / 1e9 / HBM_PEAK_GBPS,
                                "traffic": None, "what": "weights of the four projections + state read and written (a verify "
                                                         "window: read, and a checkpoint written per row), "
                                                         "over the faster of the eager and the graph time"}
        del graph
    return res

# ------------------------------------------------------------------------------------------------ main

# ------------------------------------------------------------------------------------------------ copy

def bench_copy(steps, warmup, stream):
    """A plain device-to-device copy of known size: the yardstick that FETCH_SIZE / WRITE_SIZE counter readings
    of the kernels above are scaled by, and the copy bandwidth this box reaches."""
    n = 1 << 29                                          # 512 Mi bf16 elements = 1 GiB read + 1 GiB written
    src = torch.ones(n, dtype=torch.bfloat16, device=DEV)
    dst = torch.empty_like(src)
    ms = timed(lambda: dst.copy_(src), steps, warmup, stream)
    return {"bytes_read": 2 * n, "bytes_written": 2 * n, "ms": ms, "GBps": 4 * n / (ms * 1e-3) / 1e9}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--only", choices=["decode", "prefill", "verify", "mark", "gemv", "skinny", "layer", "copy"], default=None)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; the KDA path shards by heads or slots with no exchange step, "
              "and no multi-GPU figure is produced. Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    ffi.lib()
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream()
    line = {"metric": METRIC, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "f32 (decode and verify: f32 arithmetic on a bf16-stored state; the prefill leg states its own)",
            "data": "synthetic"}
    dec = None
    if args.only in (None, "decode"):
        dec = bench_decode(args.steps, args.warmup, stream, cpu=not args.no_cpu)
        line.update({"value": dec["state_GBps"], "ms_per_step": dec["ms_per_step"], "roofline": dec["roofline"],
                     "config": {"workload": "configs[1]: decode, 16 slots x 1 token of a 48-slot bf16 pool, "
                                            "H=64, dk=dv=128, 34 layers (one pool each), per layer the chain and "
                                            "the conv window advance in one launch "
                                            "(glm53f_kda_chain_shift_batch_bf16state)",
                                "slots": 16, "pool_slots": 48, "heads": 64, "layers": 34}})
        line["decode_two_launches"] = dec["two_launches"]
        if "cpu_baseline" in dec:
            line["cpu_baseline"] = dec["cpu_baseline"]
    if args.only in (None, "prefill"):
        pre = bench_prefill(max(2, args.steps // 4), max(1, args.warmup // 2), stream, cpu=not args.no_cpu)
        line["prefill"] = pre
        if args.only == "prefill":
            line.update({"value": pre["tok_per_s_per_layer"], "unit": "tok/s per layer",
                         "ms_per_step": pre["ms_per_8192_tokens"], "roofline": pre["roofline"],
                         "config": pre["config"], "dtype": pre["dtype"]})
    if args.only in (None, "verify"):
        # alone (--only verify) the leg runs the checkpoint form only, so that a profile of it holds one kind of launch
        ver = bench_verify(max(2, args.steps // 4), max(1, args.warmup // 2), stream, saves_form=args.only is None,
                           cpu=not args.no_cpu)
        line["verify"] = ver
        if args.only == "verify":
            line.update({"value": ver["roofline"]["achieved"], "ms_per_step": ver["verify_ms_per_layer"],
                         "roofline": ver["roofline"], "config": ver["config"]})
    if args.only in (None, "mark"):
        mk = bench_mark(args.steps, args.warmup, stream, cpu=not args.no_cpu)
        line["mark"] = mk
        if args.only == "mark":
            line.update({"value": mk["roofline"]["achieved"], "ms_per_step": mk["scatter_state_pages_ms"],
                         "roofline": mk["roofline"], "config": mk["config"]})
    if args.only in (None, "gemv"):
        gv = bench_gemv(args.steps, args.warmup, stream, cpu=not args.no_cpu)
        line["gemv"] = gv
        if args.only == "gemv":
            line.update({"value": gv["roofline"]["achieved"], "ms_per_step": gv["kda_proj_1row"]["us"] / 1e3,
                         "roofline": gv["roofline"], "config": gv["config"]})
    if args.only in (None, "skinny"):
        sk = bench_skinny(args.steps, args.warmup, stream)
        line["skinny_gemm"] = sk
        if args.only == "skinny":
            line.update({"value": sk["roofline"]["achieved"], "ms_per_step": sk["kda_proj_16rows"]["us"] / 1e3,
                         "roofline": sk["roofline"], "config": sk["config"]})
    if args.only in (None, "layer"):
        ly = bench_layer_decode(max(2, args.steps // 4), max(1, args.warmup // 2), stream)
        line["layer_decode"] = ly
        if args.only == "layer":
            line.update({"value": ly["slots16"]["roofline"]["achieved"], "ms_per_step": ly["slots16"]["eager_us_per_layer"] * LAYERS / 1e3,
                         "roofline": ly["slots16"]["roofline"], "config": ly["config"]})
    if args.only == "copy":
        cp = bench_copy(args.steps, args.warmup, stream)
        line.update({"copy": cp, "value": cp["GBps"], "ms_per_step": cp["ms"],
                     "config": {"workload": "1 GiB device-to-device copy (counter yardstick)"}})
    print(json.dumps(line))


if __name__ == "__main__":
    main()
