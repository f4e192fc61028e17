"""Device staging for the GPU parity tests: oracle-side tensors (float32 numpy holding bfloat16-exact values)
go to HBM in the ABI's layouts, the kernels run through the C ABI (ctypes), results come back as float32.

Mirrors the reference's test stagers (crates/glm53f-kda/tests/gpu.rs:36-89, tests/gpu_prefill.rs:32-108):
padded strides, junk between rows, optional beta logits in front of q|k|v (negative b_off).
"""
from __future__ import annotations

import numpy as np
import torch

from glm53f_kda import DK, DV, WINDOW, channels, ffi, state_len
from oracle import kda_oracle as o

DEV = "cuda:0"


def to_bf16(x: np.ndarray) -> torch.Tensor:
    """float32 numpy (bf16-exact or not: rounds to nearest even) -> bf16 tensor on the GPU."""
    return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(torch.bfloat16).to(DEV)


def to_f32(x: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(DEV)


def back(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy().reshape(-1)


def ptr(t: torch.Tensor | None, offset: int = 0) -> int | None:
    if t is None:
        return None
    return t.data_ptr() + offset * t.element_size()


class Weights:
    """One layer's weights on the device (reference: kernel.rs:14-52)."""

    def __init__(self, p: o.LayerParams):
        self.heads = p.heads
        self.conv_w = to_bf16(p.conv_w)
        self.a_log = to_f32(p.a_log)
        self.dt_bias = to_f32(p.dt_bias)
        self.norm_w = to_bf16(p.norm_w)
        self.eps = p.eps
        self.lower = p.lower

    def args(self):
        return [ptr(self.a_log), ptr(self.dt_bias), ptr(self.norm_w), self.eps, self.lower]


class StagedRows:
    """Projection rows in device buffers with the engine's layout by default: p rows of C + H columns with
    the beta logits behind q|k|v (b_off = C), dense a/g/out rows. `pad` widens every stride and fills the gaps
    with junk; `b_first` puts the beta logits in front (negative b_off)."""

    def __init__(self, rows: o.Rows, pad: int = 0, b_first: bool = False, junk_seed: int = 1):
        h, n = rows.heads, rows.rows
        c = channels(h)
        self.heads, self.rows, self.c = h, n, c
        rng = np.random.default_rng(junk_seed)
        self.p_stride = c + h + pad
        p = rng.uniform(-3, 3, (max(n, 1), self.p_stride)).astype(np.float32)
        if b_first:
            self.p_base, self.b_off = h, -h
            p[:n, :h] = rows.b.reshape(n, h)
            p[:n, h:h + c] = rows.qkv.reshape(n, c)
        else:
            self.p_base, self.b_off = 0, c
            p[:n, :c] = rows.qkv.reshape(n, c)
            p[:n, c:c + h] = rows.b.reshape(n, h)
        self.p = to_bf16(p)
        self.a_stride = h * DK + pad
        a = rng.uniform(-3, 3, (max(n, 1), self.a_stride)).astype(np.float32)
        a[:n, :h * DK] = rows.a.reshape(n, h * DK)
        self.a = to_bf16(a)
        self.g_stride = h * DV + pad
        g = rng.uniform(-3, 3, (max(n, 1), self.g_stride)).astype(np.float32)
        g[:n, :h * DV] = rows.gate.reshape(n, h * DV)
        self.g = to_bf16(g)
        self.out_stride = h * DV + pad
        self.out = torch.full((max(n, 1), self.out_stride), 7.0, dtype=torch.bfloat16, device=DEV)

    def row_args(self):
        return [ptr(self.p, self.p_base), self.p_stride, self.b_off, ptr(self.a), self.a_stride, ptr(self.g),
                self.g_stride]

    def out_np(self) -> np.ndarray:
        return back(self.out[:self.rows, :self.heads * DV])


class Saves:
    """Replay inputs on the device for up to `rows` rows (reference: kernel.rs:137-179)."""

    def __init__(self, heads: int, rows: int):
        self.heads, self.rows = heads, rows
        n = max(rows, 1)
        self.k = torch.zeros(n * heads * DK, dtype=torch.float32, device=DEV)
        self.v = torch.zeros(n * heads * DV, dtype=torch.bfloat16, device=DEV)
        self.g = torch.zeros(n * heads * DK, dtype=torch.float32, device=DEV)
        self.b = torch.zeros(n * heads, dtype=torch.float32, device=DEV)

    def args(self):
        return [ptr(self.k), ptr(self.v), ptr(self.g), ptr(self.b)]

    def download(self, rows: int) -> o.Saves:
        h = self.heads
        return o.Saves(h, rows, back(self.k[:rows * h * DK]), back(self.v[:rows * h * DV]),
                       back(self.g[:rows * h * DK]), back(self.b[:rows * h]))

    def upload(self, s: o.Saves):
        self.k[:s.k.size] = to_f32(s.k)
        self.v[:s.v.size] = to_bf16(s.v)
        self.g[:s.g.size] = to_f32(s.g)
        self.b[:s.beta.size] = to_f32(s.beta)


NO_SAVES = [None, None, None, None]


class BatchMeta:
    """cu_rows / keep / conv_off / state_off on the device (reference: kernel.rs:407-487)."""

    def __init__(self, rows: list[int], conv_off: list[int], state_off: list[int], keep: list[int] | None = None):
        self.rows = list(rows)
        self.batch = len(rows)
        cu = np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)
        self.cu_host = cu
        self.cu_rows = torch.from_numpy(cu).to(DEV)
        self.keep_host = list(rows) if keep is None else list(keep)
        self.keep = torch.tensor(self.keep_host, dtype=torch.int32, device=DEV)
        self.conv_off = torch.tensor(conv_off, dtype=torch.int64, device=DEV)
        self.state_off = torch.tensor(state_off, dtype=torch.int64, device=DEV)

    @property
    def total(self) -> int:
        return int(self.cu_host[-1])


def sync():
    torch.cuda.synchronize()


def check(code: int, what: str):
    assert code == 0, f"{what} returned {code}"


def chain_gpu(p: o.LayerParams, conv: np.ndarray, state: np.ndarray, rows: o.Rows, *, pad=0, b_first=False,
              in_place=False, want_state=True, want_saves=True) -> o.ChainOut:
    """glm53f_kda_chain on one request, f32 state (reference helper: tests/gpu.rs chain_gpu)."""
    w = Weights(p)
    sr = StagedRows(rows, pad=pad, b_first=b_first)
    conv_d = to_bf16(conv)
    s_in = to_f32(state)
    s_out = s_in if in_place else torch.zeros_like(s_in)
    sv = Saves(p.heads, rows.rows) if want_saves else None
    code = ffi.glm53f_kda_chain(p.heads, rows.rows, *sr.row_args(), ptr(conv_d), ptr(w.conv_w), ptr(s_in),
                                ptr(s_out) if want_state else None, *w.args(), ptr(sr.out), sr.out_stride,
                                *(sv.args() if sv else NO_SAVES), None)
    check(code, "glm53f_kda_chain")
    sync()
    return o.ChainOut(sr.out_np(), None, back(s_out) if want_state else None,
                      sv.download(rows.rows) if sv else None)


def stack_rows(parts: list[o.Rows]) -> o.Rows:
    h = parts[0].heads
    cat = lambda xs: np.concatenate([np.asarray(x, np.float32).reshape(-1) for x in xs]) if xs else np.zeros(0, np.float32)
    return o.Rows(h, sum(r.rows for r in parts), cat([r.qkv for r in parts]), cat([r.a for r in parts]),
                  cat([r.b for r in parts]), cat([r.gate for r in parts]))


class Pool:
    """A slot pool of one layer: `slots` states [H][128][128] and conv windows [3][C], in f32 or bf16."""

    def __init__(self, heads: int, slots: int, bf16_state: bool, seed: int, scale: float = 0.5, gauss: bool = False):
        self.heads, self.slots, self.bf16 = heads, slots, bf16_state
        n = state_len(heads)
        rng = o.Rng(seed)
        st = (rng.normal(slots * n) * np.float32(scale)) if gauss else rng.fill(slots * n, -scale, scale)
        self.state_host = o.bf16_round(st) if bf16_state else st
        self.state = to_bf16(self.state_host) if bf16_state else to_f32(self.state_host)
        self.conv_host = rng.fill_bf16(slots * WINDOW * channels(heads), -2.0, 2.0)
        self.conv = to_bf16(self.conv_host)

    def state_of(self, slot: int) -> np.ndarray:
        n = state_len(self.heads)
        return self.state_host[slot * n:(slot + 1) * n]

    def conv_of(self, slot: int) -> np.ndarray:
        n = WINDOW * channels(self.heads)
        return self.conv_host[slot * n:(slot + 1) * n]

    def state_off(self, slot: int) -> int:
        return slot * state_len(self.heads)

    def conv_off(self, slot: int) -> int:
        return slot * WINDOW * channels(self.heads)

    def device_state(self, slot: int, t: torch.Tensor | None = None) -> np.ndarray:
        n = state_len(self.heads)
        return back((self.state if t is None else t)[slot * n:(slot + 1) * n])


def chain_batch_gpu(p: o.LayerParams, pool: Pool, slots: list[int], reqs: list[o.Rows], *, write="inplace",
                    saves=False, ckpt=False, pad=0, shift=False):
    """glm53f_kda_chain_batch[_bf16state] / verify over requests living in `slots` of `pool`.
    write: "inplace", "skip" or "to" (a fresh buffer). shift: the entry points that also advance the conv windows
    of the pool. Returns (out rows, state tensor or None, Saves, ckpt)."""
    w = Weights(p)
    sr = StagedRows(stack_rows(reqs), pad=pad)
    meta = BatchMeta([r.rows for r in reqs], [pool.conv_off(s) for s in slots], [pool.state_off(s) for s in slots])
    sv = Saves(p.heads, meta.total) if saves else None
    if write == "inplace":
        s_out = pool.state
    elif write == "to":
        s_out = torch.zeros_like(pool.state)
    else:
        s_out = None
    ck = None
    common = [p.heads, meta.batch, ptr(meta.cu_rows), *sr.row_args(), ptr(pool.conv), ptr(meta.conv_off),
              ptr(w.conv_w), ptr(pool.state)]
    tail = [*w.args(), ptr(sr.out), sr.out_stride]
    if ckpt:
        assert pool.bf16
        ck = torch.zeros(max(meta.total, 1) * state_len(p.heads), dtype=torch.bfloat16, device=DEV)
        code = ffi.glm53f_kda_verify_batch_bf16state(*common, ptr(meta.state_off), *tail, ptr(ck),
                                                     *(sv.args() if sv else NO_SAVES), None)
    else:
        if shift:
            fn = ffi.glm53f_kda_chain_shift_batch_bf16state if pool.bf16 else ffi.glm53f_kda_chain_shift_batch
        else:
            fn = ffi.glm53f_kda_chain_batch_bf16state if pool.bf16 else ffi.glm53f_kda_chain_batch
        code = fn(*common, ptr(s_out), ptr(meta.state_off), *tail, *(sv.args() if sv else NO_SAVES), None)
    check(code, "chain_batch")
    sync()
    return sr.out_np(), s_out, sv, ck, meta


def max_abs(a, b):
    return float(np.max(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)))) if len(a) else 0.0


def rel_err(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    if a.size == 0:
        return 0.0
    return float(np.max(np.abs(a - b)) / max(np.max(np.abs(b)), 1e-30))


def max_rel(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.max(np.abs(a - b) / np.maximum(np.abs(b), 1e-30)))


def ulps(a, b):
    d = o.ulp_distance(o.bf16_from_f32(a), o.bf16_from_f32(b))
    return int(d.max()) if d.size else 0, int((d > 0).sum())


def bf16_state_close(got, ref, share=1e-3):
    """A bf16-stored state against the CPU model with the same rounding points: the device's exp, division and square
    root differ from the host's in the last place, which flips an isolated bf16 rounding now and then. So: within one
    bf16 step of the largest entry everywhere, and at most `share` of the entries differ at all."""
    got, ref = np.asarray(got, np.float32), np.asarray(ref, np.float32)
    differ = int((bits(got) != bits(ref)).sum())
    return rel_err(got, ref) <= 2.0 ** -8 and differ <= max(2, share * got.size)


def bf16_steps(a, b):
    """How many representable bf16 values apart two arrays of bf16-valued floats are."""
    def key(x):
        u = np.asarray(x, np.float32).view(np.uint32).astype(np.int64) >> 16
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(key(a) - key(b))


def bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)


def prefill_batch_gpu(p: o.LayerParams, pool: Pool, slots: list[int], reqs: list[o.Rows], *, rows_per_pass=1024,
                      value_blocks=0, write="inplace", pad=0, ws_batch=None):
    """glm53f_kda_prefill_batch[_bf16state] over requests living in `slots` of `pool` (states and conv windows;
    the windows are advanced in place). Returns (out rows, state tensor, meta)."""
    w = Weights(p)
    sr = StagedRows(stack_rows(reqs), pad=pad)
    meta = BatchMeta([r.rows for r in reqs], [pool.conv_off(s) for s in slots], [pool.state_off(s) for s in slots])
    nb = ws_batch or meta.batch
    ws_bytes = ffi.glm53f_kda_prefill_workspace_bytes(p.heads, nb, rows_per_pass)
    assert ws_bytes > 0
    ws = torch.empty(ws_bytes // 4, dtype=torch.float32, device=DEV)
    s_out = pool.state if write == "inplace" else torch.zeros_like(pool.state)
    fn = ffi.glm53f_kda_prefill_batch_bf16state if pool.bf16 else ffi.glm53f_kda_prefill_batch
    code = fn(p.heads, meta.batch, ptr(meta.cu_rows), max(meta.rows), *sr.row_args(), ptr(pool.conv),
              ptr(meta.conv_off), ptr(w.conv_w), ptr(pool.state), ptr(s_out), ptr(meta.state_off), *w.args(),
              ptr(sr.out), sr.out_stride, value_blocks, ptr(ws), ws_bytes, None)
    check(code, "prefill_batch")
    sync()
    return sr.out_np(), s_out, meta


def prefill_gpu(p: o.LayerParams, conv: np.ndarray, state: np.ndarray, rows: o.Rows, *, rows_per_pass=1024,
                value_blocks=0, in_place=False, pad=0, b_first=False):
    """glm53f_kda_prefill on one request, f32 state. Returns (out, state, conv window after)."""
    w = Weights(p)
    sr = StagedRows(rows, pad=pad, b_first=b_first)
    conv_d = to_bf16(conv)
    s_in = to_f32(state)
    s_out = s_in if in_place else torch.zeros_like(s_in)
    ws_bytes = ffi.glm53f_kda_prefill_workspace_bytes(p.heads, 1, rows_per_pass)
    ws = torch.empty(max(ws_bytes, 16) // 4, dtype=torch.float32, device=DEV)
    code = ffi.glm53f_kda_prefill(p.heads, rows.rows, *sr.row_args(), ptr(conv_d), ptr(w.conv_w), ptr(s_in),
                                  ptr(s_out), *w.args(), ptr(sr.out), sr.out_stride, value_blocks, ptr(ws), ws_bytes,
                                  None)
    check(code, "prefill")
    sync()
    return sr.out_np(), back(s_out), back(conv_d)


# --------------------------------------------------------------------------------------- head subsets
# Heads are independent (state, conv channels, norms and gates are per head), so a run over H heads restricted to a
# few of them equals a run of the oracle over just those: what makes the full-size configurations checkable on the
# host in seconds.

def subset_params(p: o.LayerParams, heads: list[int]) -> o.LayerParams:
    h = p.heads
    cw = np.asarray(p.conv_w, np.float32).reshape(3, h, DK, 4)[:, heads].reshape(-1)
    return o.LayerParams(len(heads), cw, np.asarray(p.a_log, np.float32)[heads],
                         np.asarray(p.dt_bias, np.float32).reshape(h, DK)[heads].reshape(-1), p.norm_w, p.eps, p.lower)


def subset_rows(h: int, heads: list[int], P: torch.Tensor, A: torch.Tensor, G: torch.Tensor, r0: int, r1: int) -> o.Rows:
    """Rows r0..r1 of device buffers in the engine's layout (p rows of C + H columns, dense a and g), the chosen
    heads only, as oracle rows on the host."""
    c, n = channels(h), r1 - r0
    idx = torch.tensor(heads, device=P.device)
    qkv = P[r0:r1, :c].reshape(n, 3, h, DK).index_select(2, idx).float().cpu().numpy().reshape(-1)
    b = P[r0:r1, c:c + h].index_select(1, idx).float().cpu().numpy().reshape(-1)
    a = A[r0:r1].reshape(n, h, DK).index_select(1, idx).float().cpu().numpy().reshape(-1)
    g = G[r0:r1].reshape(n, h, DV).index_select(1, idx).float().cpu().numpy().reshape(-1)
    return o.Rows(len(heads), n, qkv, a, b, g)


def subset_conv(h: int, heads: list[int], window: torch.Tensor) -> np.ndarray:
    idx = torch.tensor(heads, device=window.device)
    return window.reshape(WINDOW, 3, h, DK).index_select(2, idx).float().cpu().numpy().reshape(-1)


def subset_state(h: int, heads: list[int], state: torch.Tensor) -> np.ndarray:
    idx = torch.tensor(heads, device=state.device)
    return state.reshape(h, DV * DK).index_select(0, idx).float().cpu().numpy().reshape(-1)


def subset_out(h: int, heads: list[int], out: torch.Tensor) -> np.ndarray:
    idx = torch.tensor(heads, device=out.device)
    return out.reshape(out.shape[0], h, DV).index_select(1, idx).float().cpu().numpy().reshape(-1)
