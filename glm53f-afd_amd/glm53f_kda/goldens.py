"""Golden fixtures of the reference oracle and what the KDA path needs from them: the host-side mirror of the
reference's crates/glm53f-kda/src/goldens.rs (format :3-38, Set :182-400, roles :413-545, comparisons :640-760,
replay inputs :1015-1052, layer case :1054-1180, writer :1276-1310).

A set is a directory holding `manifest.json` next to raw little-endian `.bin` files. The manifest's `tensors`
object maps names to `{"file", "dtype", "shape", "sha256"}` (a manifest that is that map itself is accepted too);
its `notes` object carries facts about the set, such as `state_heads`. Every file is checked against its size and
digest before use. The oracle names its sets `layerNN-prefill` / `layerNN-decode` and their tensors
`prefill.kda.q`, `decode.kda.core_out` and so on; a tensor belongs to a KDA layer when it names that layer, as a
component of its own name (`layers.4.`, `L04.`, `layer4.`) or through its set's name.

This module only reads, names and lays out: it converts the reference's layouts (state `[H][DK][DV]`, conv cache
`[C][W]`) to the kernels' (`[H][DV][DK]`, window `[3][C]`) and builds kernel-format inputs. Running them is the
caller's business (the tests run the HIP kernels on them).
"""
from __future__ import annotations

import hashlib
import json
import os
from dataclasses import dataclass, field

import numpy as np

from . import DK, DV, WINDOW, channels, state_len

TAPS = 4
DECODER_LAYERS = 45

TOL_F32 = 1e-4        # f32 goldens: the same f32 recurrence or its chunked form (goldens.rs:753-756)
TOL_RECURRENT = 1e-2  # bf16 goldens on the per-token path: a bf16 rounding flip (:757-758)
TOL_CHUNKED = 5e-2    # bf16 goldens on the chunked path (:759-761)


class GoldenError(Exception):
    """Io, Json, Manifest, Digest, Size, Missing or Shape (goldens.rs:46-66); `kind` says which."""

    def __init__(self, kind: str, message: str):
        super().__init__(f"{kind}: {message}")
        self.kind = kind


def is_kda_layer(i: int) -> bool:
    """Every decoder layer except 3, 7, 11, ..., 43 (src/lib.rs:66-70)."""
    return 0 <= i < DECODER_LAYERS and i % 4 != 3


# dtype name -> (canonical name, numpy dtype or None for bf16, bytes)   (goldens.rs:100-145)
_DTYPES = {
    "f64": ("f64", np.dtype("<f8"), 8), "float64": "f64", "double": "f64",
    "f32": ("f32", np.dtype("<f4"), 4), "float32": "f32", "float": "f32",
    "f16": ("f16", np.dtype("<f2"), 2), "float16": "f16", "half": "f16",
    "bf16": ("bf16", None, 2), "bfloat16": "bf16",
    "i64": ("i64", np.dtype("<i8"), 8), "int64": "i64", "long": "i64",
    "i32": ("i32", np.dtype("<i4"), 4), "int32": "i32", "int": "i32",
    "u8": ("u8", np.dtype("u1"), 1), "uint8": "u8", "bool": "u8",
}


def parse_dtype(s: str):
    """(canonical name, numpy dtype or None, element bytes), or None for an unknown name."""
    key = s.lower()
    if key.startswith("torch."):
        key = key[len("torch."):]
    v = _DTYPES.get(key)
    if isinstance(v, str):
        v = _DTYPES[v]
    return v


@dataclass
class Entry:
    name: str
    file: str
    dtype: str
    shape: list
    sha256: str

    def elements(self) -> int:
        return int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1


@dataclass
class Tensor:
    """A tensor read from a set, widened to f32 (integers converted as values)."""
    name: str
    dtype: str
    shape: list
    data: np.ndarray


class Set:
    """A golden set: a directory and its manifest (goldens.rs:182-400)."""

    def __init__(self, directory: str, entries: list, notes):
        self.dir, self.entries, self.notes = directory, entries, notes

    @staticmethod
    def load(directory: str) -> "Set":
        path = os.path.join(directory, "manifest.json")
        try:
            with open(path, "r", encoding="utf-8") as f:
                text = f.read()
        except OSError as e:
            raise GoldenError("Io", f"{path}: {e}") from e
        try:
            doc = json.loads(text)
        except json.JSONDecodeError as e:
            raise GoldenError("Json", f"{path}: {e}") from e
        if not isinstance(doc, dict):
            raise GoldenError("Manifest", "not a JSON object")
        members = doc.get("tensors", doc)
        if not isinstance(members, dict):
            raise GoldenError("Manifest", "not a JSON object")
        entries = []
        for name, v in members.items():
            # Other members (metadata) are skipped; tensor entries have a "file".
            if not isinstance(v, dict) or not isinstance(v.get("file"), str):
                continue
            file = v["file"]
            dt = parse_dtype(v["dtype"]) if isinstance(v.get("dtype"), str) else None
            if not isinstance(v.get("dtype"), str):
                raise GoldenError("Manifest", f"{name}: no dtype")
            if dt is None:
                raise GoldenError("Manifest", f"{name}: unknown dtype")
            shape = v.get("shape")
            if not isinstance(shape, list):
                raise GoldenError("Manifest", f"{name}: no shape")
            if not all(isinstance(x, int) and not isinstance(x, bool) and x >= 0 for x in shape):
                raise GoldenError("Manifest", f"{name}: bad shape")
            if not isinstance(v.get("sha256"), str):
                raise GoldenError("Manifest", f"{name}: no sha256")
            if ".." in file or file.startswith("/"):
                raise GoldenError("Manifest", f"{name}: file must stay inside the set")
            entries.append(Entry(name, file, dt[0], list(shape), v["sha256"].lower()))
        notes = doc.get("notes")
        return Set(directory, entries, notes if isinstance(notes, dict) else None)

    def name(self) -> str:
        return os.path.basename(os.path.normpath(self.dir))

    def layer_phase(self):
        """(layer, "prefill" | "decode") from a name `layerNN-prefill` / `layerNN-decode`, else None."""
        n = self.name()
        if not n.startswith("layer") or "-" not in n:
            return None
        layer, phase = n[len("layer"):].split("-", 1)
        if phase not in ("prefill", "decode") or not layer.isdigit():
            return None
        return int(layer), phase

    def state_heads(self):
        if not self.notes or not isinstance(self.notes.get("state_heads"), list):
            return None
        hs = self.notes["state_heads"]
        return list(hs) if all(isinstance(h, int) and h >= 0 for h in hs) else None

    def entry(self, name: str):
        return next((e for e in self.entries if e.name == name), None)

    def bytes(self, name: str) -> bytes:
        """The raw bytes of `name`, checked against the manifest's size and digest."""
        e = self.entry(name)
        if e is None:
            raise GoldenError("Missing", name)
        path = os.path.join(self.dir, e.file)
        try:
            with open(path, "rb") as f:
                raw = f.read()
        except OSError as err:
            raise GoldenError("Io", f"{path}: {err}") from err
        want = e.elements() * parse_dtype(e.dtype)[2]
        if len(raw) != want:
            raise GoldenError("Size", f"{name}: {len(raw)} bytes, expected {want}")
        got = hashlib.sha256(raw).hexdigest()
        if got != e.sha256:
            raise GoldenError("Digest", f"{name}: sha256 {got} does not match the manifest's {e.sha256}")
        return raw

    def read(self, name: str) -> Tensor:
        e = self.entry(name)
        raw = self.bytes(name)
        _, npdt, _ = parse_dtype(e.dtype)
        if npdt is None:   # bf16: the upper half of an f32
            data = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32)
        else:
            data = np.frombuffer(raw, dtype=npdt).astype(np.float32)
        return Tensor(name, e.dtype, list(e.shape), np.ascontiguousarray(data))


def discover(root: str) -> list:
    """The set directories under `root`, sorted (goldens.rs:390-409)."""
    try:
        names = sorted(os.listdir(root))
    except OSError:
        return []
    return [os.path.join(root, n) for n in names if os.path.isfile(os.path.join(root, n, "manifest.json"))]


# role -> the names it is recognized by (lowercase, after the phase, layer and module names)  (goldens.rs:469-505)
ROLES = {
    "Q": ("q", "query"), "K": ("k", "key"), "V": ("v", "value"), "LogDecay": ("g", "log_decay"), "Beta": ("beta",),
    "StateIn": ("initial_state", "state_in"),
    "StateOut": ("state", "state_final", "final_state", "state_out", "last_recurrent_state"),
    "StateSteps": ("state_heads",), "CoreOut": ("core_out", "core_attn_out"), "Path": ("path",),
    "MixedQkv": ("qkv_preconv", "mixed_qkv"), "ConvStateIn": ("conv_state_in",),
    "ConvStateOut": ("conv_state", "conv_state_final", "conv_state_out"),
    "ForgetProj": ("f_proj", "forget_proj", "f_b_proj"), "BetaLogits": ("b_logits", "b_proj", "beta_logits"),
    "GateProj": ("gate", "g_proj", "g_b_proj"), "NormOut": ("norm_out", "o_norm_out"),
    "ConvW": ("conv1d.weight", "conv_w"), "ConvWQ": ("q_conv1d.weight",), "ConvWK": ("k_conv1d.weight",),
    "ConvWV": ("v_conv1d.weight",), "ALog": ("a_log",), "DtBias": ("dt_bias",), "NormW": ("o_norm.weight", "norm_w"),
}
MODULES = ("weights", "kda", "self_attn", "linear_attn", "forget_gate")


def classify(name: str, set_layer=None):
    """(layer, role) of a tensor name, or None. `set_layer` is the layer the set's name gives, used when the
    tensor name holds none. Only KDA layers qualify (goldens.rs:509-545)."""
    parts = name.lower().replace("/", ".").split(".")
    if parts and parts[0] in ("prefill", "decode"):
        parts = parts[1:]
        # Per-step tensors (`decode.sN.<name>`) are not used.
        if parts and len(parts[0]) > 1 and parts[0][0] == "s" and parts[0][1:].isdigit():
            return None
    found = None
    for i, p in enumerate(parts):
        digits = p[len("layer"):] if p.startswith("layer") else (p[1:] if p.startswith("l") else p)
        if digits and digits.isascii() and digits.isdigit():
            found = (i, int(digits))
            break
    if found is not None:
        rest, layer = parts[found[0] + 1:], found[1]
    elif set_layer is not None:
        rest, layer = parts, set_layer
    else:
        return None
    if not is_kda_layer(layer):
        return None
    key = ".".join(p for p in rest if p not in MODULES)
    for role, names in ROLES.items():
        if key in names:
            return layer, role
    return None


@dataclass
class LayerFixtures:
    """One KDA layer's tensors in a set: role -> tensor name."""
    layer: int
    names: dict = field(default_factory=dict)

    def name(self, role: str):
        return self.names.get(role)

    def has(self, roles) -> bool:
        return all(r in self.names for r in roles)


def kda_layers(s: Set) -> list:
    lp = s.layer_phase()
    set_layer = lp[0] if lp else None
    layers: dict = {}
    for e in s.entries:
        c = classify(e.name, set_layer)
        if c is None:
            continue
        layers.setdefault(c[0], LayerFixtures(c[0])).names.setdefault(c[1], e.name)
    return [layers[k] for k in sorted(layers)]


@dataclass
class Init:
    """What precedes a set's rows: state (reference layout [H][DK][DV]) and conv cache ([C][W]), when known."""
    state: np.ndarray | None = None
    conv: np.ndarray | None = None

    @staticmethod
    def from_prefill(s: Set, layer: int) -> "Init":
        """For a decode set: the state and conv cache after the prompt, from the matching `layerNN-prefill` set
        next to it. Empty for any other set, or when there is none (goldens.rs:606-637)."""
        if s.layer_phase() != (layer, "decode"):
            return Init()
        d = os.path.join(os.path.dirname(os.path.normpath(s.dir)), f"layer{layer:02d}-prefill")
        if not os.path.isfile(os.path.join(d, "manifest.json")):
            return Init()
        pre = Set.load(d)
        lf = next((x for x in kda_layers(pre) if x.layer == layer), None)
        if lf is None:
            return Init()
        rd = lambda role: pre.read(lf.name(role)).data if lf.name(role) else None
        return Init(rd("StateOut"), rd("ConvStateOut"))


def transpose_state(s: np.ndarray) -> np.ndarray:
    """[n][A][B] -> [n][B][A] with A = B = 128: between the reference's [H][DK][DV] and the kernels' [H][DV][DK]."""
    s = np.asarray(s, np.float32)
    return np.ascontiguousarray(s.reshape(-1, DK, DV).transpose(0, 2, 1)).reshape(-1)


def conv_window(cache: np.ndarray, c: int) -> np.ndarray:
    """The kernels' window [3][C] (oldest first) from the reference's conv cache [C][W], W >= 3: its last three
    columns (goldens.rs:1116-1138)."""
    cache = np.asarray(cache, np.float32)
    if cache.size % c != 0 or cache.size // c < WINDOW:
        raise GoldenError("Shape", f"conv cache: expected [{c}][W >= {WINDOW}]")
    w = cache.size // c
    return np.ascontiguousarray(cache.reshape(c, w)[:, w - WINDOW:].T).reshape(-1)


def _tensor(s: Set, lf: LayerFixtures, role: str) -> Tensor:
    n = lf.name(role)
    if n is None:
        raise GoldenError("Missing", f"layer {lf.layer} {role}")
    return s.read(n)


def _optional(s: Set, lf: LayerFixtures, role: str):
    return s.read(lf.name(role)) if lf.name(role) else None


def _expect(t: Tensor, n: int):
    if t.data.size != n:
        raise GoldenError("Shape", f"{t.name}: {t.data.size} elements, expected {n}")


@dataclass
class CoreInputs:
    """The inputs of the recurrent core as the reference passes them to its delta-rule function."""
    heads: int
    rows: int
    q: Tensor
    k: Tensor
    v: Tensor
    g: Tensor
    beta: Tensor
    state: np.ndarray   # reference layout [H][DK][DV]


def core_inputs(s: Set, lf: LayerFixtures, init: Init) -> CoreInputs:
    """goldens.rs:822-895."""
    q, k, v = _tensor(s, lf, "Q"), _tensor(s, lf, "K"), _tensor(s, lf, "V")
    g, beta = _tensor(s, lf, "LogDecay"), _tensor(s, lf, "Beta")
    if beta.data.size == 0 or q.data.size != beta.data.size * DK:
        raise GoldenError("Shape", f"{q.name} and {beta.name} disagree on T * H")
    th = beta.data.size
    if len(beta.shape) >= 2:
        heads = beta.shape[-1]
    elif len(q.shape) >= 2 and q.shape[-1] == DK:
        heads = q.shape[-2]
    else:
        raise GoldenError("Shape", f"{q.name}: cannot tell the number of heads")
    if heads == 0 or th % heads != 0:
        raise GoldenError("Shape", f"{q.name}: {heads} heads do not divide T * H = {th}")
    for x in (k, g):
        _expect(x, th * DK)
    _expect(v, th * DV)
    si = _optional(s, lf, "StateIn")
    if si is not None:
        _expect(si, state_len(heads))
        state = si.data
    elif init.state is not None:
        if init.state.size != state_len(heads):
            raise GoldenError("Shape", f"initial state: {init.state.size} elements, expected {state_len(heads)}")
        state = np.asarray(init.state, np.float32)
    else:
        state = np.zeros(state_len(heads), np.float32)
    return CoreInputs(heads, th // heads, q, k, v, g, beta, state)


def is_recurrent(s: Set, lf: LayerFixtures, rows: int) -> bool:
    """Whether a set's rows came from the recurrent path: its `path` tensor says so, else one row."""
    p = _optional(s, lf, "Path")
    return bool(np.all(p.data == 1.0)) if p is not None else rows == 1


def tolerance(dtype: str, recurrent: bool) -> float:
    if dtype in ("f32", "f64"):
        return TOL_F32
    return TOL_RECURRENT if recurrent else TOL_CHUNKED


def _bf16_round(x: np.ndarray) -> np.ndarray:
    """Round to nearest even to bfloat16, as f32 values (finite inputs)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32)


@dataclass
class ReplayCase:
    """Kernel-format replay inputs for a golden's rows (goldens.rs:1015-1052): normalized k, v rounded to bfloat16
    (the kernels keep v in bfloat16), exp(g), beta; the state before the rows and the golden state after them in the
    kernel layout [H][DV][DK]."""
    heads: int
    rows: int
    k: np.ndarray
    v: np.ndarray
    g: np.ndarray
    beta: np.ndarray
    state: np.ndarray
    after: np.ndarray | None


def l2norm_rows(x: np.ndarray) -> np.ndarray:
    """x / sqrt(sum x^2 + 1e-6) per row of 128, f32 with the kernels' summation order (32 partials of four products,
    then an xor butterfly over the partials with offsets 16, 8, 4, 2, 1)."""
    x = np.ascontiguousarray(x, np.float32).reshape(-1, DK)
    sq = x * x
    part = ((sq[:, 0::4] + sq[:, 1::4]) + sq[:, 2::4]) + sq[:, 3::4]          # [n][32], left to right
    for off in (16, 8, 4, 2, 1):
        part = part + part[:, np.arange(32) ^ off]
    ss = part[:, 0]
    inv = np.float32(1.0) / np.sqrt(ss + np.float32(1e-6), dtype=np.float32)
    return (x * inv[:, None]).astype(np.float32).reshape(-1)


def replay_inputs(s: Set, lf: LayerFixtures, init: Init) -> ReplayCase:
    c = core_inputs(s, lf, init)
    so = _optional(s, lf, "StateOut")
    after = transpose_state(so.data) if so is not None and so.data.size == state_len(c.heads) else None
    return ReplayCase(c.heads, c.rows, l2norm_rows(c.k.data), _bf16_round(c.v.data),
                      np.exp(c.g.data.astype(np.float32)).astype(np.float32), c.beta.data.copy(),
                      transpose_state(c.state), after)


@dataclass
class LayerCase:
    """The inputs of a full-layer golden in the kernels' layouts (goldens.rs:1054-1180)."""
    heads: int
    conv_w: np.ndarray
    a_log: np.ndarray
    dt_bias: np.ndarray
    norm_w: np.ndarray
    conv: np.ndarray        # [3][C]
    state: np.ndarray       # [H][DV][DK]
    rows: int
    qkv: np.ndarray
    a: np.ndarray
    b: np.ndarray
    gate: np.ndarray
    norm_out: np.ndarray    # golden gated-norm output [T][H * DV]
    state_out: np.ndarray | None


def layer_case(s: Set, lf: LayerFixtures, init: Init) -> LayerCase:
    a_log = _tensor(s, lf, "ALog").data
    heads = a_log.size
    c = channels(heads)
    if lf.name("ConvW"):
        conv_w = _tensor(s, lf, "ConvW").data
    else:
        conv_w = np.concatenate([_tensor(s, lf, r).data for r in ("ConvWQ", "ConvWK", "ConvWV")])
    if conv_w.size != c * TAPS:
        raise GoldenError("Shape", f"layer {lf.layer} conv weight: {conv_w.size} elements, expected {c * TAPS}")
    dt_bias, norm_w = _tensor(s, lf, "DtBias").data, _tensor(s, lf, "NormW").data
    qkv = _tensor(s, lf, "MixedQkv")
    if qkv.data.size % c != 0:
        raise GoldenError("Shape", f"{qkv.name}: not a multiple of {c}")
    t = qkv.data.size // c
    a, b = _tensor(s, lf, "ForgetProj"), _tensor(s, lf, "BetaLogits")
    gate, norm_out = _tensor(s, lf, "GateProj"), _tensor(s, lf, "NormOut")
    _expect(a, t * heads * DK)
    _expect(b, t * heads)
    _expect(gate, t * heads * DV)
    _expect(norm_out, t * heads * DV)
    ci = _optional(s, lf, "ConvStateIn")
    cache = ci.data if ci is not None else init.conv
    conv = conv_window(cache, c) if cache is not None else np.zeros(WINDOW * c, np.float32)
    si = _optional(s, lf, "StateIn")
    if si is not None:
        _expect(si, state_len(heads))
        state = transpose_state(si.data)
    elif init.state is not None and init.state.size == state_len(heads):
        state = transpose_state(init.state)
    else:
        state = np.zeros(state_len(heads), np.float32)
    so = _optional(s, lf, "StateOut")
    if so is not None:
        _expect(so, state_len(heads))
    return LayerCase(heads, conv_w, a_log, dt_bias, norm_w, conv, state, t, qkv.data, a.data, b.data, gate.data,
                     norm_out.data, transpose_state(so.data) if so is not None else None)


def conv_cache_after(before: np.ndarray, rows: np.ndarray, c: int) -> np.ndarray:
    """The reference conv cache [C][W] after `rows` ([t][C]) follow `before` ([C][W]): pure data movement."""
    before = np.asarray(before, np.float32).reshape(c, -1)
    w = before.shape[1]
    rows = np.asarray(rows, np.float32).reshape(-1, c)
    joined = np.concatenate([before.T, rows], axis=0)      # [W + t][C], oldest first
    return np.ascontiguousarray(joined[-w:].T).reshape(-1)


@dataclass
class Comparison:
    """A computed tensor against its golden (goldens.rs:640-735): passes when max |diff| <= tol * max(max |ref|, 1e-3)."""
    what: str
    elements: int
    max_abs: float
    max_ref: float
    differing: int
    tol: float

    @staticmethod
    def compare(what: str, got, want, tol: float) -> "Comparison":
        got, want = np.asarray(got, np.float32).reshape(-1), np.asarray(want, np.float32).reshape(-1)
        assert got.size == want.size, f"{what}: length"
        d = np.abs(got.astype(np.float64) - want.astype(np.float64))
        max_abs = float("inf") if np.isnan(d).any() else float(d.max(initial=0.0))
        return Comparison(what, got.size, max_abs, float(np.abs(want).max(initial=0.0)),
                          int(np.count_nonzero(got.view(np.uint32) != want.view(np.uint32))), tol)

    def passes(self) -> bool:
        return self.max_abs <= self.tol * max(self.max_ref, 1e-3)

    def __str__(self) -> str:
        return (f"{self.what}: {self.elements} elements, max |diff| {self.max_abs:.3e} (max |ref| {self.max_ref:.3e}, "
                f"tolerance {self.tol:.1e} relative), {self.differing} differ")


def write_set(directory: str, tensors: list, notes: dict | None = None, flat: bool = False) -> None:
    """Write a set: `tensors` is a list of (name, dtype in {"f32", "bf16", "i32"}, shape, values)
    (goldens.rs:1276-1310). `flat` writes the manifest as the bare tensor map."""
    os.makedirs(directory, exist_ok=True)
    entries = {}
    for name, dtype, shape, values in tensors:
        values = np.asarray(values)
        assert values.size == int(np.prod(shape, dtype=np.int64)), f"{name}: shape"
        if dtype == "f32":
            raw = values.astype("<f4").tobytes()
        elif dtype == "bf16":
            raw = (_bf16_round(values.astype(np.float32)).view(np.uint32) >> 16).astype("<u2").tobytes()
        elif dtype == "i32":
            raw = values.astype("<i4").tobytes()
        else:
            raise ValueError("write_set writes f32, bf16 and i32")
        file = f"{name}.bin"
        with open(os.path.join(directory, file), "wb") as f:
            f.write(raw)
        entries[name] = {"file": file, "dtype": dtype, "shape": list(shape), "sha256": hashlib.sha256(raw).hexdigest()}
    doc = entries if flat else {"tensors": entries, "notes": notes or {}}
    with open(os.path.join(directory, "manifest.json"), "w", encoding="utf-8") as f:
        json.dump(doc, f, indent=1)
