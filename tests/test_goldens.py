"""The golden-set loader (glm53f_kda.goldens) and the kernels on oracle-layout sets.

Follows the reference's crates/glm53f-kda/tests/goldens.rs (synthetic oracle-layout sets pass every check, a
corrupted fixture is rejected, a flat manifest is accepted), the unit tests of src/goldens.rs:1316-1372 (name
classification, f16 widening), tests/gpu.rs:799-852 (the device recurrence on golden activations) and
tests/gpu_prefill.rs:653-760 (the kernels on oracle layers). The reference repository holds manifests without
payloads, so the payload-bearing sets here are synthetic ones in the oracle's layout (written the way
tests/common/mod.rs:107-173 writes them); the loader's naming rules are also held to the tensor names of the
oracle's real manifests (tests/golden/oracle_manifest_names.json). Real sets under $GLM53F_GOLDENS are checked too
when present.
"""
import json
import os

import numpy as np
import pytest

from glm53f_kda import DK, DV, WINDOW, channels, goldens as gd, state_len
from oracle import kda_oracle as o

HERE = os.path.dirname(os.path.abspath(__file__))


# ------------------------------------------------------------------------------------------------ names and formats

def test_classifies_names():
    """The known answers of src/goldens.rs:1316-1361."""
    c = gd.classify
    assert c("layers.4.kda.q") == (4, "Q")
    assert c("model.language_model.layers.4.self_attn.A_log") == (4, "ALog")
    assert c("model.language_model.layers.0.self_attn.forget_gate.dt_bias") == (0, "DtBias")
    assert c("model.language_model.layers.0.self_attn.q_conv1d.weight") == (0, "ConvWQ")
    assert c("L06.kda.core_out") == (6, "CoreOut")
    assert c("prefill.kda.q", 4) == (4, "Q")
    assert c("decode.kda.state_final", 0) == (0, "StateOut")
    assert c("decode.kda.state_heads", 0) == (0, "StateSteps")
    assert c("prefill.kda.conv_state", 4) == (4, "ConvStateOut")
    assert c("prefill.kda.qkv_preconv", 4) == (4, "MixedQkv")
    assert c("decode.s3.kda.q", 4) is None
    assert c("prefill.kda.q") is None
    assert c("prefill.mla.q", 3) is None
    assert c("layers.3.self_attn.q") is None
    assert c("prefill.moe.gate", 4) is None
    assert c("logits") is None
    assert c("L04.prefill.kda.state_heads") is None


def test_kda_layers_are_all_but_every_fourth():
    """src/lib.rs:66-70, :93."""
    got = [i for i in range(60) if gd.is_kda_layer(i)]
    assert len(got) == 34 and 3 not in got and 43 not in got and 44 in got and 45 not in got


def test_dtypes_and_widening(tmp_path):
    """src/goldens.rs:100-145 and the f16 known answers of :1363-1371."""
    assert gd.parse_dtype("torch.bfloat16")[0] == "bf16" and gd.parse_dtype("Float")[0] == "f32"
    assert gd.parse_dtype("long")[2] == 8 and gd.parse_dtype("bool")[0] == "u8" and gd.parse_dtype("complex64") is None
    # f16 bit patterns written raw, read back widened
    raw = np.array([0x3C00, 0xC000, 0x0001, 0x7C00, 0x7BFF], dtype="<u2").tobytes()
    import hashlib
    d = tmp_path / "set"
    d.mkdir()
    (d / "h.bin").write_bytes(raw)
    (d / "manifest.json").write_text(json.dumps({"h": {"file": "h.bin", "dtype": "float16", "shape": [5],
                                                       "sha256": hashlib.sha256(raw).hexdigest().upper()}}))
    t = gd.Set.load(str(d)).read("h")
    assert t.data.tolist() == [1.0, -2.0, 2.0 ** -24, float("inf"), 65504.0]


def test_real_oracle_manifest_names_get_their_roles():
    """Every KDA tensor the oracle's own manifests list is recognized, with the shapes the checks expect."""
    with open(os.path.join(HERE, "golden", "oracle_manifest_names.json")) as f:
        real = json.load(f)
    want = {
        "kda.q": "Q", "kda.k": "K", "kda.v": "V", "kda.g": "LogDecay", "kda.beta": "Beta", "kda.core_out": "CoreOut",
        "kda.path": "Path", "kda.qkv_preconv": "MixedQkv", "kda.f_proj": "ForgetProj", "kda.b_logits": "BetaLogits",
        "kda.gate": "GateProj", "kda.norm_out": "NormOut",
    }
    for set_name, body in real.items():
        layer, phase = int(set_name[5:7]), set_name.split("-")[1]
        names = body["tensors"]
        roles = {}
        for n in names:
            c = gd.classify(n, layer)
            if c is not None:
                assert c[0] == layer
                roles[c[1]] = n
        for suffix, role in want.items():
            assert roles.get(role) == f"{phase}.{suffix}", (set_name, role)
        assert roles["StateOut"] == (f"{phase}.kda.state" if phase == "prefill" else f"{phase}.kda.state_final")
        assert roles["ConvStateOut"].startswith(f"{phase}.kda.conv_state")
        assert roles["ALog"] == "weights.self_attn.A_log" and roles["DtBias"] == "weights.self_attn.dt_bias"
        assert roles["NormW"] == "weights.self_attn.o_norm.weight"
        assert {"ConvWQ", "ConvWK", "ConvWV"} <= set(roles)
        if phase == "decode":
            assert roles["StateSteps"] == "decode.kda.state_heads" and body["state_heads"] == [0, 21, 42, 63]
        # nothing outside the KDA module is taken for a KDA tensor
        assert all(".kda." in n or n.startswith("weights.self_attn.") for n in roles.values())
        # shapes: [T, H, 128] activations, [H, DK, DV] state, [C, 4] conv cache
        t = names[roles["Beta"]]["shape"][0]
        assert names[roles["Q"]]["shape"] == [t, 64, DK] and names[roles["StateOut"]]["shape"] == [64, DK, DV]
        assert names[roles["ConvStateOut"]]["shape"] == [channels(64), 4]
        assert names[roles["MixedQkv"]]["shape"] == [t, channels(64)]


def test_host_helpers_agree_with_the_oracle():
    rng = o.Rng(11)
    x = rng.fill(7 * DK, -3.0, 3.0)
    want = np.concatenate([o.l2norm(x[i * DK:(i + 1) * DK]) for i in range(7)])
    assert np.array_equal(gd.l2norm_rows(x).view(np.uint32), want.view(np.uint32))
    s = rng.fill(2 * DK * DV, -1.0, 1.0)
    assert np.array_equal(gd.transpose_state(s), o.transpose_state(s))
    assert np.array_equal(gd.transpose_state(gd.transpose_state(s)), s)
    y = np.concatenate([rng.fill(1000, -70000.0, 70000.0), rng.fill(1000, -1e-3, 1e-3)])
    assert np.array_equal(gd._bf16_round(y).view(np.uint32), o.bf16_round(y).view(np.uint32))
    # conv cache [C][W] -> window [3][C]: the last three columns, oldest first
    cache = np.arange(5 * 4, dtype=np.float32).reshape(5, 4)
    assert gd.conv_window(cache, 5).reshape(3, 5)[:, 2].tolist() == [9.0, 10.0, 11.0]
    after = gd.conv_cache_after(cache, np.full((2, 5), 99.0, np.float32), 5).reshape(5, 4)
    assert after[2].tolist() == [10.0, 11.0, 99.0, 99.0]


# ------------------------------------------------------------------------------------------------ synthetic sets

def core(heads, rows, seed):
    """q, k (the conv outputs, before their L2 norms, as the oracle records them), v, log decay and beta, seeded."""
    rng = o.Rng(seed)
    q = rng.fill(rows * heads * DK, -1.0, 1.0)
    k = rng.fill(rows * heads * DK, -1.0, 1.0)
    v = rng.fill(rows * heads * DV, -2.0, 2.0)
    g = -np.abs(rng.fill(rows * heads * DK, 0.0, 3.0))
    beta = rng.fill(rows * heads, 0.05, 0.95)
    return q, k, v, g.astype(np.float32), beta


def normalized(x, scale=None):
    return np.concatenate([o.l2norm(x[i * DK:(i + 1) * DK], scale) for i in range(x.size // DK)])


def write_oracle_pair(root, heads=8, prompt=70, steps=8):
    """A prefill set and its decode set for layer 4 in the oracle's layout, f32 like its primary contract: the
    prefill by the chunked form, then the decode steps by the recurrence, which also records the per-row states of
    heads 0, 1 and heads - 1 (tests/common/mod.rs:107-173)."""
    c = channels(heads)
    rng = o.Rng(42)
    q, k, v, g, beta = core(heads, prompt, 41)
    qn, kn = normalized(q, o.q_scale()), normalized(k)
    qkv_p = rng.fill(prompt * c, -2.0, 2.0)
    state = np.zeros(state_len(heads), np.float32)                 # reference layout [H][DK][DV]
    y_p = o.chunked_layer(heads, qn, kn, v, g, beta, state, 64)
    conv_p = gd.conv_cache_after(np.zeros(c * 4, np.float32), qkv_p, c)
    thd = lambda t: [t, heads, DK]
    gd.write_set(os.path.join(root, "layer04-prefill"), [
        ("prefill.kda.qkv_preconv", "f32", [prompt, c], qkv_p), ("prefill.kda.q", "f32", thd(prompt), q),
        ("prefill.kda.k", "f32", thd(prompt), k), ("prefill.kda.v", "f32", thd(prompt), v),
        ("prefill.kda.g", "f32", thd(prompt), g), ("prefill.kda.beta", "f32", [prompt, heads], beta),
        ("prefill.kda.core_out", "f32", thd(prompt), y_p), ("prefill.kda.state", "f32", [heads, DK, DV], state),
        ("prefill.kda.conv_state", "f32", [c, 4], conv_p), ("prefill.kda.path", "i32", [1], [0]),
        ("prefill.attn_norm", "f32", [prompt, 8], np.full(prompt * 8, 0.5, np.float32)),      # not a KDA tensor
    ], {"layer": 4, "attention": "kda", "phase": "prefill"})
    kept = [0, 1, heads - 1]
    q, k, v, g, beta = core(heads, steps, 43)
    qkv_d = rng.fill(steps * c, -2.0, 2.0)
    y_d, per_step = [], []
    st = state.reshape(heads, DK, DV)
    for r in range(steps):
        for h in range(heads):
            i = r * heads + h      # the literal step takes q and k as recorded and normalizes them itself
            y_d.append(o.literal_step(st[h], q[i * DK:(i + 1) * DK], k[i * DK:(i + 1) * DK], v[i * DV:(i + 1) * DV],
                                      g[i * DK:(i + 1) * DK], float(beta[i])))
        per_step.append(st[kept].copy())
    gd.write_set(os.path.join(root, "layer04-decode"), [
        ("decode.kda.qkv_preconv", "f32", [steps, c], qkv_d), ("decode.kda.q", "f32", thd(steps), q),
        ("decode.kda.k", "f32", thd(steps), k), ("decode.kda.v", "f32", thd(steps), v),
        ("decode.kda.g", "f32", thd(steps), g), ("decode.kda.beta", "f32", [steps, heads], beta),
        ("decode.kda.core_out", "f32", thd(steps), np.concatenate(y_d)),
        ("decode.kda.state_heads", "f32", [steps, len(kept), DK, DV], np.concatenate([p.reshape(-1) for p in per_step])),
        ("decode.kda.state_final", "f32", [heads, DK, DV], st.reshape(-1)),
        ("decode.kda.conv_state_final", "f32", [c, 4], gd.conv_cache_after(conv_p, qkv_d, c)),
        ("decode.kda.path", "i32", [steps, 1], np.ones(steps)),
        ("decode.s0.idx.scores", "f32", [2], [1.0, 2.0]),                                      # per step: skipped
    ], {"layer": 4, "attention": "kda", "phase": "decode", "state_heads": kept})


def check_core(s, lf, init):
    """The recurrent core against a golden: q, k, v, g, beta through the literal step row by row, compared with the
    core output, the state after the rows and the per-row states of notes.state_heads (goldens.rs:897-960)."""
    c = gd.core_inputs(s, lf, init)
    core_out = s.read(lf.name("CoreOut"))
    st = c.state.copy().reshape(c.heads, DK, DV)
    kept = s.state_heads()
    y, per_step = [], []
    for r in range(c.rows):
        for h in range(c.heads):
            i = r * c.heads + h
            y.append(o.literal_step(st[h], c.q.data[i * DK:(i + 1) * DK], c.k.data[i * DK:(i + 1) * DK],
                                    c.v.data[i * DV:(i + 1) * DV], c.g.data[i * DK:(i + 1) * DK], float(c.beta.data[i])))
        if kept and lf.name("StateSteps"):
            per_step.append(st[kept].copy().reshape(-1))
    tol = gd.tolerance(core_out.dtype, gd.is_recurrent(s, lf, c.rows))
    out = [gd.Comparison.compare(f"layer {lf.layer} core output", np.concatenate(y), core_out.data, tol)]
    if lf.name("StateOut"):
        out.append(gd.Comparison.compare(f"layer {lf.layer} state after the rows", st.reshape(-1),
                                         s.read(lf.name("StateOut")).data, tol))
    if per_step:
        out.append(gd.Comparison.compare(f"layer {lf.layer} per-row states of heads {kept}", np.concatenate(per_step),
                                         s.read(lf.name("StateSteps")).data, tol))
    return out


def check_conv_cache(s, lf, init):
    """The conv cache after the rows against the cache before them followed by the rows' q | k | v projections:
    data movement, exact (goldens.rs:962-1013)."""
    qkv = s.read(lf.name("MixedQkv"))
    after = s.read(lf.name("ConvStateOut"))
    c = after.shape[0]
    before = init.conv if init.conv is not None else np.zeros(after.data.size, np.float32)
    return np.array_equal(gd.conv_cache_after(before, qkv.data, c), after.data)


def test_oracle_layout_sets_pass_every_check(tmp_path):
    root = str(tmp_path)
    write_oracle_pair(root)
    dirs = gd.discover(root)
    assert [os.path.basename(d) for d in dirs] == ["layer04-decode", "layer04-prefill"]
    for d in dirs:
        s = gd.Set.load(d)
        layers = gd.kda_layers(s)
        assert [lf.layer for lf in layers] == [4]
        lf = layers[0]
        assert "attn_norm" not in " ".join(lf.names.values()) and "scores" not in " ".join(lf.names.values())
        init = gd.Init.from_prefill(s, 4)
        assert (init.state is not None) == (s.layer_phase()[1] == "decode")
        results = check_core(s, lf, init)
        assert len(results) == (3 if s.layer_phase()[1] == "decode" else 2)
        for r in results:
            print(r)
            assert r.passes(), str(r)
        assert gd.is_recurrent(s, lf, 8) == (s.layer_phase()[1] == "decode")
        assert check_conv_cache(s, lf, init)


def test_corrupted_fixture_is_rejected(tmp_path):
    root = str(tmp_path)
    write_oracle_pair(root, heads=2, prompt=5, steps=2)
    d = os.path.join(root, "layer04-prefill")
    s = gd.Set.load(d)
    path = os.path.join(d, "prefill.kda.k.bin")
    raw = bytearray(open(path, "rb").read())
    raw[17] ^= 0x40
    open(path, "wb").write(bytes(raw))
    with pytest.raises(gd.GoldenError) as e:
        s.read("prefill.kda.k")
    assert e.value.kind == "Digest"
    open(path, "wb").write(bytes(raw[:-4]))
    with pytest.raises(gd.GoldenError) as e:
        s.read("prefill.kda.k")
    assert e.value.kind == "Size"
    os.remove(path)
    with pytest.raises(gd.GoldenError) as e:
        s.read("prefill.kda.k")
    assert e.value.kind == "Io"
    with pytest.raises(gd.GoldenError) as e:
        s.read("prefill.kda.nothing")
    assert e.value.kind == "Missing"
    # a manifest that points outside its set
    (tmp_path / "bad").mkdir()
    (tmp_path / "bad" / "manifest.json").write_text(json.dumps(
        {"tensors": {"x": {"file": "../x.bin", "dtype": "f32", "shape": [1], "sha256": "00"}}}))
    with pytest.raises(gd.GoldenError) as e:
        gd.Set.load(str(tmp_path / "bad"))
    assert e.value.kind == "Manifest"


def test_flat_manifest_is_accepted(tmp_path):
    d = str(tmp_path / "layer08-prefill")
    gd.write_set(d, [("prefill.kda.beta", "f32", [3, 2], np.arange(6, dtype=np.float32)),
                     ("prefill.kda.v", "bf16", [3, 2, DV], np.full(3 * 2 * DV, 1.00390625, np.float32))], flat=True)
    s = gd.Set.load(d)
    assert s.notes is None and len(s.entries) == 2 and s.layer_phase() == (8, "prefill")
    assert s.read("prefill.kda.beta").data.tolist() == [0.0, 1.0, 2.0, 3.0, 4.0, 5.0]
    assert np.all(s.read("prefill.kda.v").data == 1.0)          # 1 + 2^-8 rounds to even in bf16
    assert gd.kda_layers(s)[0].has(["Beta", "V"]) and not gd.kda_layers(s)[0].has(["Q"])


# ------------------------------------------------------------------------------------------------ the kernels on sets

def golden_roots(tmp_root):
    roots = [tmp_root]
    if os.environ.get("GLM53F_GOLDENS"):
        roots.append(os.environ["GLM53F_GOLDENS"])
    return [d for r in roots for d in gd.discover(r)]


def payloads_present(s):
    return all(os.path.isfile(os.path.join(s.dir, e.file)) for e in s.entries)


@pytest.mark.gpu
def test_device_recurrence_on_golden_activations(tmp_path):
    """tests/gpu.rs:799-852: the replay kernel on the golden's k, v, g and beta equals the CPU replay bit for bit and
    the golden state within 1e-2 (the kernels keep v in bfloat16, the f32 goldens do not)."""
    import torch

    from glm53f_kda import ffi

    import harness as hs

    write_oracle_pair(str(tmp_path), heads=8, prompt=70, steps=8)
    checked = 0
    for d in golden_roots(str(tmp_path)):
        s = gd.Set.load(d)
        if not payloads_present(s):
            continue
        for lf in gd.kda_layers(s):
            if not lf.has(["K", "V", "LogDecay", "Beta", "StateOut"]):
                continue
            rc = gd.replay_inputs(s, lf, gd.Init.from_prefill(s, lf.layer))
            sv = hs.Saves(rc.heads, rc.rows)
            saves = o.Saves(rc.heads, rc.rows, rc.k, rc.v, rc.g, rc.beta)
            sv.upload(saves)
            st = hs.to_f32(rc.state)
            hs.check(ffi.glm53f_kda_replay(rc.heads, rc.rows, hs.ptr(st), hs.ptr(st), *sv.args(), None), "replay")
            hs.sync()
            got = hs.back(st)
            assert np.array_equal(hs.bits(got), hs.bits(o.replay(rc.state, saves, rc.rows))), (s.name(), lf.layer)
            c = gd.Comparison.compare(f"{s.name()}: layer {lf.layer} device state after {rc.rows} rows", got, rc.after, 1e-2)
            print(c)
            assert c.passes(), str(c)
            checked += 1
    assert checked >= 2, "the synthetic prefill and decode sets"


def write_layer_set(root, heads=8, rows=100, seed=77):
    """A full-layer set in the oracle's layout and names (weights, projections, caches, outputs), f32 activations:
    what the oracle's real sets carry for a KDA layer. The outputs are the FP32 recurrent reference's."""
    p = o.synth_layer(heads, seed)
    r = o.synth_rows(heads, rows, seed)
    c = channels(heads)
    conv = o.synth_conv_window(heads, seed)                       # [3][C]
    s0 = o.synth_state(heads, seed, 0.3)                          # kernel layout
    lit = o.literal_chain(p, conv, s0, r)
    cache_in = np.ascontiguousarray(np.concatenate([np.zeros((1, c), np.float32), conv.reshape(3, c)]).T).reshape(-1)
    cw = p.conv_w.reshape(3, heads * DK, 4)
    gd.write_set(os.path.join(root, "layer08-prefill"), [
        ("prefill.kda.qkv_preconv", "f32", [rows, c], r.qkv), ("prefill.kda.f_proj", "f32", [rows, heads, DK], r.a),
        ("prefill.kda.b_logits", "f32", [rows, heads], r.b), ("prefill.kda.gate", "f32", [rows, heads, DV], r.gate),
        ("prefill.kda.norm_out", "f32", [rows, heads, DV], lit.out),
        ("prefill.kda.initial_state", "f32", [heads, DK, DV], gd.transpose_state(s0)),
        ("prefill.kda.conv_state_in", "f32", [c, 4], cache_in),
        ("prefill.kda.state", "f32", [heads, DK, DV], gd.transpose_state(lit.state)),
        ("weights.self_attn.q_conv1d.weight", "bf16", [heads * DK, 1, 4], cw[0]),
        ("weights.self_attn.k_conv1d.weight", "bf16", [heads * DK, 1, 4], cw[1]),
        ("weights.self_attn.v_conv1d.weight", "bf16", [heads * DK, 1, 4], cw[2]),
        ("weights.self_attn.A_log", "f32", [heads], p.a_log), ("weights.self_attn.dt_bias", "f32", [heads * DK], p.dt_bias),
        ("weights.self_attn.o_norm.weight", "bf16", [DV], p.norm_w),
    ], {"layer": 8, "attention": "kda", "phase": "prefill"})
    return p


LAYER_ROLES = ["ALog", "DtBias", "NormW", "MixedQkv", "ForgetProj", "BetaLogits", "GateProj", "NormOut"]


@pytest.mark.gpu
def test_kernels_on_oracle_layers(tmp_path):
    """tests/gpu_prefill.rs:653-760: chain and prefill on a layer set's weights, projections and caches, against the
    set's outputs (at bfloat16 scale) and state."""
    import harness as hs

    p_written = write_layer_set(str(tmp_path))
    checked = 0
    for d in golden_roots(str(tmp_path)):
        s = gd.Set.load(d)
        if not payloads_present(s):
            continue
        for lf in gd.kda_layers(s):
            if not lf.has(LAYER_ROLES) or not (lf.name("ConvW") or lf.has(["ConvWQ", "ConvWK", "ConvWV"])):
                continue
            case = gd.layer_case(s, lf, gd.Init.from_prefill(s, lf.layer))
            p = o.LayerParams(case.heads, case.conv_w, case.a_log, case.dt_bias, case.norm_w)
            rows = o.Rows(case.heads, case.rows, o.bf16_round(case.qkv), o.bf16_round(case.a), o.bf16_round(case.b),
                          o.bf16_round(case.gate))
            conv = o.bf16_round(case.conv)
            chain = hs.chain_gpu(p, conv, case.state, rows, want_saves=False)
            out_p, st_p, _ = hs.prefill_gpu(p, conv, case.state, rows)
            cpu = o.chain(p, conv, case.state, rows)
            ps, po = hs.rel_err(st_p, chain.state), hs.rel_err(out_p, chain.out)
            cs, co = hs.rel_err(chain.state, cpu.state), hs.rel_err(chain.out, cpu.out)
            go = hs.rel_err(chain.out, case.norm_out)
            gs = hs.rel_err(chain.state, case.state_out) if case.state_out is not None else 0.0
            print(f"{s.name()} layer {lf.layer} ({case.rows} rows): prefill vs chain: state {ps:.1e}, output {po:.1e}; "
                  f"chain vs CPU: state {cs:.1e}, output {co:.1e}; chain vs golden: state {gs:.1e}, output {go:.1e}")
            assert ps <= 1e-3 and po <= 2.0 ** -7
            assert cs <= 1e-3 and co <= 1.0 / 256.0
            assert gs <= 1e-2 and go <= 2.0 ** -6        # bf16 activations against f32 goldens, at bf16 scale
            checked += 1
    assert checked >= 1
    # the set written above reads back as what was written
    s = gd.Set.load(os.path.join(str(tmp_path), "layer08-prefill"))
    case = gd.layer_case(s, gd.kda_layers(s)[0], gd.Init())
    assert np.array_equal(case.conv_w, p_written.conv_w) and np.array_equal(case.norm_w, p_written.norm_w)
