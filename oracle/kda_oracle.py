"""TEST INFRASTRUCTURE ONLY: numpy bindings of the CPU oracle (oracle/kda_ref.c).

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this module. The shipped
library never does: it fails loudly when its HIP code is missing instead of falling back to this.

The classes mirror the reference's CPU types: `LayerParams` and `Rows` (crates/glm53f-kda/src/cpu.rs:82-159),
`Saves` and `ChainOut` (cpu.rs:161-200), and the `synth` generators (src/synth.rs:49-83). bfloat16 tensors
are float32 arrays of bfloat16-exact values, as in the reference.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass, field

import numpy as np

DK = 128
DV = 128
TAPS = 4
WINDOW = 3
HEADS = 64
LAYERS = 34
LOWER_BOUND = -5.0
RMS_EPS = 1e-5
FUSED, UNFUSED, F32 = 0, 1, 2

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkda_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (oracle/Makefile)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE, "libkda_oracle.so"], check=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


class _Layer(C.Structure):
    _fields_ = [("heads", C.c_int32), ("conv_w", C.c_void_p), ("a_log", C.c_void_p), ("dt_bias", C.c_void_p),
                ("norm_w", C.c_void_p), ("eps", C.c_float), ("lower", C.c_float)]


class _Rows(C.Structure):
    _fields_ = [("heads", C.c_int32), ("rows", C.c_int32), ("qkv", C.c_void_p), ("a", C.c_void_p),
                ("b", C.c_void_p), ("gate", C.c_void_p)]


class _Rng(C.Structure):
    _fields_ = [("s", C.c_uint64)]


def _declare(l: C.CDLL) -> None:
    f32, i32, i64, u16, u32, u64, vp = C.c_float, C.c_int32, C.c_int64, C.c_uint16, C.c_uint32, C.c_uint64, C.c_void_p
    sig = {
        "kda_bf16_from_f32": (u16, [f32]), "kda_bf16_to_f32": (f32, [u16]), "kda_bf16_round": (f32, [f32]),
        "kda_bf16_ulp_distance": (u32, [u16, u16]),
        "kda_bf16_encode": (None, [vp, vp, i64]), "kda_bf16_decode": (None, [vp, vp, i64]),
        "kda_rng_new": (None, [vp, u64]), "kda_rng_next_u64": (u64, [vp]),
        "kda_rng_uniform": (f32, [vp, f32, f32]), "kda_rng_uniform_bf16": (f32, [vp, f32, f32]),
        "kda_rng_fill": (None, [vp, vp, i64, f32, f32]), "kda_rng_fill_bf16": (None, [vp, vp, i64, f32, f32]),
        "kda_rng_normal": (f32, [vp]), "kda_rng_fill_normal": (None, [vp, vp, i64]),
        "kda_synth_layer": (None, [i32, u64, vp, vp, vp, vp]),
        "kda_synth_rows": (None, [i32, i32, u64, vp, vp, vp, vp]),
        "kda_synth_conv_window": (None, [i32, u64, vp]),
        "kda_synth_state": (None, [i32, u64, f32, vp]),
        "kda_sigmoid": (f32, [f32]), "kda_silu": (f32, [f32]), "kda_warp_sum": (f32, [vp]),
        "kda_dot128": (f32, [vp, vp]), "kda_log_decay": (f32, [f32, f32, f32, f32]),
        "kda_decay": (f32, [f32, f32, f32, f32]), "kda_beta": (f32, [f32]), "kda_q_scale": (f32, []),
        "kda_conv_channel": (f32, [vp, vp, vp, i32, i32, C.c_int]),
        "kda_conv_qkv": (None, [vp, vp, vp, i32, i32, C.c_int, vp, vp, vp]),
        "kda_l2norm": (None, [vp, f32, vp]), "kda_update": (None, [vp, vp, vp, vp, f32]),
        "kda_read_out": (None, [vp, vp, vp]),
        "kda_gated_rmsnorm_as": (None, [vp, vp, vp, f32, C.c_int, vp]),
        "kda_chain_with": (None, [vp, vp, vp, vp, C.c_int, C.c_int, vp, vp, vp, vp, vp, vp, vp, C.c_int]),
        "kda_replay_with": (None, [i32, vp, vp, vp, vp, vp, i32, C.c_int, vp]),
        "kda_exact_replay": (None, [i32, vp, vp, vp, vp, vp, i32, vp, C.c_int]),
        "kda_conv_shift": (None, [i32, vp, vp, i32, i32, vp]),
        "kda_transpose_state": (None, [vp, vp, i64]),
        "kda_literal_l2norm": (None, [vp, vp]),
        "kda_literal_step": (None, [vp, vp, vp, vp, vp, f32, vp]),
        "kda_literal_gated_rmsnorm_as": (None, [vp, vp, vp, f32, C.c_int, vp]),
        "kda_literal_chain": (None, [vp, vp, vp, vp, C.c_int, vp, vp, vp, vp, vp, vp, vp, C.c_int]),
        "kda_chunked_head": (None, [vp, vp, vp, vp, vp, i32, vp, i32, vp]),
        "kda_chunked_layer": (None, [i32, vp, vp, vp, vp, vp, i32, vp, i32, vp, C.c_int]),
        "kda_recurrent_layer": (None, [i32, vp, vp, vp, vp, vp, i32, vp, vp, C.c_int]),
        "kda_prefill_head": (None, [vp, vp, vp, vp, vp, i32, vp, vp]),
        "kda_prefill": (None, [vp, vp, vp, vp, C.c_int, vp, vp, vp, C.c_int]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(l, name)
        fn.restype = res
        fn.argtypes = args


EXPORTS = [
    "kda_bf16_from_f32", "kda_bf16_to_f32", "kda_bf16_round", "kda_bf16_ulp_distance", "kda_bf16_encode",
    "kda_bf16_decode", "kda_rng_new", "kda_rng_next_u64", "kda_rng_uniform", "kda_rng_uniform_bf16",
    "kda_rng_fill", "kda_rng_fill_bf16", "kda_rng_normal", "kda_rng_fill_normal", "kda_synth_layer",
    "kda_synth_rows", "kda_synth_conv_window", "kda_synth_state", "kda_sigmoid", "kda_silu", "kda_warp_sum",
    "kda_dot128", "kda_log_decay", "kda_decay", "kda_beta", "kda_q_scale", "kda_conv_channel", "kda_conv_qkv",
    "kda_l2norm", "kda_update", "kda_read_out", "kda_gated_rmsnorm_as", "kda_chain_with", "kda_replay_with", "kda_exact_replay",
    "kda_conv_shift", "kda_transpose_state", "kda_literal_l2norm", "kda_literal_step",
    "kda_literal_gated_rmsnorm_as", "kda_literal_chain", "kda_chunked_head", "kda_chunked_layer",
    "kda_recurrent_layer", "kda_prefill_head", "kda_prefill",
]


def _f32(x) -> np.ndarray:
    return np.ascontiguousarray(x, dtype=np.float32)


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def channels(heads: int) -> int:
    return 3 * heads * DK


def state_len(heads: int) -> int:
    return heads * DV * DK


# ----------------------------------------------------------------------------- bf16

def bf16_from_f32(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even bfloat16 bits (uint16) of a float32 array."""
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().kda_bf16_encode(_p(x), _p(out), x.size)
    return out


def bf16_to_f32(b: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(b.shape, dtype=np.float32)
    lib().kda_bf16_decode(_p(b), _p(out), b.size)
    return out


def bf16_round(x) -> np.ndarray:
    return bf16_to_f32(bf16_from_f32(x))


def ulp_distance(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """bfloat16 ulp distance between two uint16 arrays of bits (src/bf16.rs:36-46)."""
    def ordered(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x)
    return np.abs(ordered(a) - ordered(b)).astype(np.uint32)


# ----------------------------------------------------------------------------- rng / synth

class Rng:
    """SplitMix64 with the reference's seed mixing (src/synth.rs:10-45)."""

    def __init__(self, seed: int):
        self._r = _Rng()
        lib().kda_rng_new(C.byref(self._r), C.c_uint64(seed & (2**64 - 1)))

    def next_u64(self) -> int:
        return lib().kda_rng_next_u64(C.byref(self._r))

    def uniform(self, lo: float, hi: float) -> float:
        return lib().kda_rng_uniform(C.byref(self._r), lo, hi)

    def fill(self, n: int, lo: float, hi: float) -> np.ndarray:
        out = np.empty(n, dtype=np.float32)
        lib().kda_rng_fill(C.byref(self._r), _p(out), n, lo, hi)
        return out

    def fill_bf16(self, n: int, lo: float, hi: float) -> np.ndarray:
        out = np.empty(n, dtype=np.float32)
        lib().kda_rng_fill_bf16(C.byref(self._r), _p(out), n, lo, hi)
        return out

    def normal(self, n: int) -> np.ndarray:
        out = np.empty(n, dtype=np.float32)
        lib().kda_rng_fill_normal(C.byref(self._r), _p(out), n)
        return out


@dataclass
class LayerParams:
    heads: int
    conv_w: np.ndarray  # [C][TAPS]
    a_log: np.ndarray   # [H]
    dt_bias: np.ndarray # [H*DK]
    norm_w: np.ndarray  # [DV]
    eps: float = RMS_EPS
    lower: float = LOWER_BOUND

    def channels(self) -> int:
        return channels(self.heads)

    def _c(self):
        self.conv_w, self.a_log = _f32(self.conv_w), _f32(self.a_log)
        self.dt_bias, self.norm_w = _f32(self.dt_bias), _f32(self.norm_w)
        assert self.conv_w.size == self.channels() * TAPS and self.a_log.size == self.heads
        assert self.dt_bias.size == self.heads * DK and self.norm_w.size == DV
        return _Layer(self.heads, self.conv_w.ctypes.data, self.a_log.ctypes.data, self.dt_bias.ctypes.data,
                      self.norm_w.ctypes.data, self.eps, self.lower)


@dataclass
class Rows:
    heads: int
    rows: int
    qkv: np.ndarray   # [rows][C]
    a: np.ndarray     # [rows][H*DK]
    b: np.ndarray     # [rows][H]
    gate: np.ndarray  # [rows][H*DV]

    def slice(self, start: int, n: int) -> "Rows":
        assert start + n <= self.rows
        h, c = self.heads, channels(self.heads)
        return Rows(h, n, self.qkv.reshape(-1)[start * c:(start + n) * c].copy(),
                    self.a.reshape(-1)[start * h * DK:(start + n) * h * DK].copy(),
                    self.b.reshape(-1)[start * h:(start + n) * h].copy(),
                    self.gate.reshape(-1)[start * h * DV:(start + n) * h * DV].copy())

    def _c(self):
        self.qkv, self.a, self.b, self.gate = _f32(self.qkv), _f32(self.a), _f32(self.b), _f32(self.gate)
        h, r = self.heads, self.rows
        assert self.qkv.size == r * channels(h) and self.a.size == r * h * DK
        assert self.b.size == r * h and self.gate.size == r * h * DV
        return _Rows(h, r, self.qkv.ctypes.data, self.a.ctypes.data, self.b.ctypes.data, self.gate.ctypes.data)


@dataclass
class Saves:
    heads: int
    rows: int
    k: np.ndarray     # [rows][H][DK]
    v: np.ndarray     # [rows][H][DV]
    g: np.ndarray     # [rows][H][DK]
    beta: np.ndarray  # [rows][H]

    @staticmethod
    def zeros(heads: int, rows: int) -> "Saves":
        z = lambda n: np.zeros(n, dtype=np.float32)
        return Saves(heads, rows, z(rows * heads * DK), z(rows * heads * DV), z(rows * heads * DK), z(rows * heads))


@dataclass
class ChainOut:
    out: np.ndarray    # [rows][H*DV]
    y: np.ndarray      # [rows][H*DV]
    state: np.ndarray  # [H][DV][DK]
    saves: Saves = field(default=None)


def synth_layer(heads: int, seed: int) -> LayerParams:
    cw = np.empty(channels(heads) * TAPS, np.float32)
    al = np.empty(heads, np.float32)
    dt = np.empty(heads * DK, np.float32)
    nw = np.empty(DV, np.float32)
    lib().kda_synth_layer(heads, C.c_uint64(seed), _p(cw), _p(al), _p(dt), _p(nw))
    return LayerParams(heads, cw, al, dt, nw)


def synth_rows(heads: int, rows: int, seed: int) -> Rows:
    qkv = np.empty(rows * channels(heads), np.float32)
    a = np.empty(rows * heads * DK, np.float32)
    b = np.empty(rows * heads, np.float32)
    gate = np.empty(rows * heads * DV, np.float32)
    lib().kda_synth_rows(heads, rows, C.c_uint64(seed), _p(qkv), _p(a), _p(b), _p(gate))
    return Rows(heads, rows, qkv, a, b, gate)


def synth_conv_window(heads: int, seed: int) -> np.ndarray:
    out = np.empty(WINDOW * channels(heads), np.float32)
    lib().kda_synth_conv_window(heads, C.c_uint64(seed), _p(out))
    return out


def synth_state(heads: int, seed: int, scale: float) -> np.ndarray:
    out = np.empty(state_len(heads), np.float32)
    lib().kda_synth_state(heads, C.c_uint64(seed), scale, _p(out))
    return out


# ----------------------------------------------------------------------------- scalar pieces

def sigmoid(x: float) -> float:
    return lib().kda_sigmoid(x)


def silu(x: float) -> float:
    return lib().kda_silu(x)


def warp_sum(lanes) -> float:
    a = _f32(lanes)
    assert a.size == 32
    return lib().kda_warp_sum(_p(a))


def dot128(a, b) -> float:
    a, b = _f32(a), _f32(b)
    return lib().kda_dot128(_p(a), _p(b))


def log_decay(a, dt_bias, a_log, lower) -> float:
    return lib().kda_log_decay(a, dt_bias, a_log, lower)


def decay(a, dt_bias, decay_rate, lower) -> float:
    return lib().kda_decay(a, dt_bias, decay_rate, lower)


def beta(b: float) -> float:
    return lib().kda_beta(b)


def q_scale() -> float:
    return lib().kda_q_scale()


def conv_qkv(p: LayerParams, conv, rows: Rows, r: int, h: int, mode: int = FUSED):
    conv = _f32(conv)
    q, k, v = (np.empty(DK, np.float32) for _ in range(3))
    pc, rc = p._c(), rows._c()
    lib().kda_conv_qkv(C.byref(pc), _p(conv), C.byref(rc), r, h, mode, _p(q), _p(k), _p(v))
    return q, k, v


def l2norm(x, scale: float | None = None) -> np.ndarray:
    x = _f32(x)
    y = np.empty(DK, np.float32)
    lib().kda_l2norm(_p(x), 0.0 if scale is None else scale, _p(y))
    return y


def update(s: np.ndarray, k, g, v, beta_: float) -> None:
    """In place on s ([DV][DK], float32, contiguous)."""
    assert s.dtype == np.float32 and s.flags.c_contiguous and s.size == DV * DK
    k, g, v = _f32(k), _f32(g), _f32(v)
    lib().kda_update(_p(s), _p(k), _p(g), _p(v), beta_)


def read_out(s, q) -> np.ndarray:
    s, q = _f32(s), _f32(q)
    y = np.empty(DV, np.float32)
    lib().kda_read_out(_p(s), _p(q), _p(y))
    return y


def gated_rmsnorm(y, norm_w, gate, eps: float, mode: int = FUSED) -> np.ndarray:
    y, norm_w, gate = _f32(y), _f32(norm_w), _f32(gate)
    o = np.empty(DV, np.float32)
    lib().kda_gated_rmsnorm_as(_p(y), _p(norm_w), _p(gate), eps, mode, _p(o))
    return o


# ----------------------------------------------------------------------------- chain / replay

def _chain(fn_name: str, p: LayerParams, conv, state, rows: Rows, mode: int, bf16_state: bool | None,
           threads: int) -> ChainOut:
    conv, state = _f32(conv), _f32(state)
    assert conv.size == WINDOW * p.channels() and state.size == state_len(p.heads) and rows.heads == p.heads
    h, r = p.heads, rows.rows
    out = np.zeros(r * h * DV, np.float32)
    y = np.zeros(r * h * DV, np.float32)
    st = np.empty(state_len(h), np.float32)
    sv = Saves.zeros(h, r)
    pc, rc = p._c(), rows._c()
    args = [C.byref(pc), _p(conv), _p(state), C.byref(rc), mode]
    if bf16_state is not None:
        args.append(int(bf16_state))
    args += [_p(out), _p(y), _p(st), _p(sv.k), _p(sv.v), _p(sv.g), _p(sv.beta), threads]
    getattr(lib(), fn_name)(*args)
    return ChainOut(out, y, st, sv)


def chain(p, conv, state, rows, mode=FUSED, threads=1) -> ChainOut:
    """cpu::chain (cpu.rs:380-388): the kernels' order of operations, f32 state."""
    return _chain("kda_chain_with", p, conv, state, rows, mode, False, threads)


def chain_bf16_state(p, conv, state, rows, mode=FUSED, threads=1) -> ChainOut:
    """cpu::chain_bf16_state (cpu.rs:394-402): the state rounded to bfloat16 after each row's read-out."""
    return _chain("kda_chain_with", p, conv, state, rows, mode, True, threads)


def literal_chain(p, conv, state, rows, mode=FUSED, threads=1) -> ChainOut:
    """cpu::literal::chain (cpu.rs:639-685): the reference's own formulation."""
    return _chain("kda_literal_chain", p, conv, state, rows, mode, None, threads)


def replay(state, saves: Saves, keep: int, bf16_state: bool = False) -> np.ndarray:
    """cpu::replay / replay_bf16_state (cpu.rs:475-508)."""
    assert keep <= saves.rows
    state = _f32(state)
    out = np.empty_like(state)
    k, v, g, b = _f32(saves.k), _f32(saves.v), _f32(saves.g), _f32(saves.beta)
    lib().kda_replay_with(saves.heads, _p(state), _p(k), _p(v), _p(g), _p(b), keep, int(bf16_state), _p(out))
    return out


def exact_replay(state, saves: Saves, rows: int | None = None, threads: int = 1) -> np.ndarray:
    """The delta rule over the saved rows in f64 (tests/gpu_prefill.rs:502-519): float64 state [H][DV][DK]."""
    rows = saves.rows if rows is None else rows
    assert rows <= saves.rows
    state = _f32(state)
    out = np.empty(state.size, dtype=np.float64)
    k, v, g, b = _f32(saves.k), _f32(saves.v), _f32(saves.g), _f32(saves.beta)
    lib().kda_exact_replay(saves.heads, _p(state), _p(k), _p(v), _p(g), _p(b), rows, out.ctypes.data_as(C.c_void_p),
                           threads)
    return out


def conv_shift(conv, rows: Rows, keep: int) -> np.ndarray:
    """cpu::conv_shift (cpu.rs:512-527)."""
    assert keep <= rows.rows
    conv, qkv = _f32(conv), _f32(rows.qkv)
    out = np.empty(WINDOW * channels(rows.heads), np.float32)
    lib().kda_conv_shift(rows.heads, _p(conv), _p(qkv), rows.rows, keep, _p(out))
    return out


def transpose_state(s) -> np.ndarray:
    s = _f32(s)
    assert s.size % (DK * DV) == 0
    t = np.empty_like(s)
    lib().kda_transpose_state(_p(s), _p(t), s.size)
    return t


def literal_l2norm(x) -> np.ndarray:
    x = _f32(x)
    y = np.empty(DK, np.float32)
    lib().kda_literal_l2norm(_p(x), _p(y))
    return y


def literal_step(s: np.ndarray, q, k, v, g, beta_: float) -> np.ndarray:
    """cpu::literal::step (cpu.rs:573-610): in place on s ([DK][DV]); returns the read-out, not rounded."""
    assert s.dtype == np.float32 and s.flags.c_contiguous and s.size == DK * DV
    q, k, v, g = _f32(q), _f32(k), _f32(v), _f32(g)
    y = np.empty(DV, np.float32)
    lib().kda_literal_step(_p(s), _p(q), _p(k), _p(v), _p(g), beta_, _p(y))
    return y


# ----------------------------------------------------------------------------- chunked

def chunked_head(q, k, v, g, beta_, state: np.ndarray, chunk: int) -> np.ndarray:
    """chunked::head (chunked.rs:67-198): state [DK][DV] updated in place."""
    q, k, v, g, beta_ = _f32(q), _f32(k), _f32(v), _f32(g), _f32(beta_)
    t = beta_.size
    assert state.dtype == np.float32 and state.flags.c_contiguous and state.size == DK * DV
    out = np.empty(t * DV, np.float32)
    lib().kda_chunked_head(_p(q), _p(k), _p(v), _p(g), _p(beta_), t, _p(state), chunk, _p(out))
    return out


def chunked_layer(heads, q, k, v, g, beta_, state: np.ndarray, chunk: int, threads: int = 1) -> np.ndarray:
    """chunked::layer (chunked.rs:205-254): state [H][DK][DV] updated in place."""
    q, k, v, g, beta_ = _f32(q), _f32(k), _f32(v), _f32(g), _f32(beta_)
    t = beta_.size // heads
    assert state.dtype == np.float32 and state.flags.c_contiguous and state.size == heads * DK * DV
    out = np.empty(t * heads * DV, np.float32)
    lib().kda_chunked_layer(heads, _p(q), _p(k), _p(v), _p(g), _p(beta_), t, _p(state), chunk, _p(out), threads)
    return out


def recurrent_layer(heads, q, k, v, g, beta_, state: np.ndarray, threads: int = 1) -> np.ndarray:
    """literal::step row by row on core-level inputs; state [H][DK][DV] updated in place."""
    q, k, v, g, beta_ = _f32(q), _f32(k), _f32(v), _f32(g), _f32(beta_)
    t = beta_.size // heads
    assert state.dtype == np.float32 and state.flags.c_contiguous and state.size == heads * DK * DV
    out = np.empty(t * heads * DV, np.float32)
    lib().kda_recurrent_layer(heads, _p(q), _p(k), _p(v), _p(g), _p(beta_), t, _p(state), _p(out), threads)
    return out


def prefill(p: LayerParams, conv, state, rows: Rows, mode: int = FUSED, threads: int = 1) -> ChainOut:
    """chunked::prefill (chunked.rs:405-467): the reference prefill kernel's 16-row host model."""
    conv, state = _f32(conv), _f32(state)
    h, r = p.heads, rows.rows
    out = np.zeros(r * h * DV, np.float32)
    y = np.zeros(r * h * DV, np.float32)
    st = np.empty(state_len(h), np.float32)
    pc, rc = p._c(), rows._c()
    lib().kda_prefill(C.byref(pc), _p(conv), _p(state), C.byref(rc), mode, _p(out), _p(y), _p(st), threads)
    return ChainOut(out, y, st, Saves.zeros(h, 0))
