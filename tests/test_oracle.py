"""Pins the CPU oracle (oracle/kda_ref.c) before anything trusts it.

Known answers and invariants are those of the reference's own CPU tests
(crates/glm53f-kda/tests/cpu_reference.rs and src/bf16.rs); on top of them come checks the mathematics
fixes: an f64 textbook delta-rule recurrence written from the formula, torch's bfloat16 cast, and Vigna's
published SplitMix64 vector. No GPU needed.
"""
import math

import numpy as np
import pytest
import torch

from oracle import kda_oracle as o

DK, DV, WINDOW = o.DK, o.DV, o.WINDOW


def bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)


def rel_err(a, b):
    """max |a - b| / max(max |b|, tiny) (cpu_reference.rs:12-21)."""
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.max(np.abs(a - b)) / max(np.max(np.abs(b)), 1e-30))


def bf16_diff(a, b):
    d = o.ulp_distance(o.bf16_from_f32(a), o.bf16_from_f32(b))
    return int(d.max()), int((d != 0).sum())


# ---------------------------------------------------------------- bf16 (src/bf16.rs:52-77)

def test_bf16_rounds_to_nearest_even():
    L = o.lib()
    assert L.kda_bf16_from_f32(1.0) == 0x3F80
    assert L.kda_bf16_from_f32(1.0 + 1.0 / 256.0) == 0x3F80
    assert L.kda_bf16_from_f32(1.0 + 3.0 / 256.0) == 0x3F82
    assert L.kda_bf16_from_f32(np.uint32(0x3F808001).view(np.float32).item()) == 0x3F81
    assert L.kda_bf16_round(-2.5) == -2.5
    assert L.kda_bf16_to_f32(0xC020) == -2.5


def test_bf16_specials():
    L = o.lib()
    assert L.kda_bf16_from_f32(float("inf")) == 0x7F80
    assert L.kda_bf16_from_f32(float("-inf")) == 0xFF80
    assert L.kda_bf16_from_f32(float(np.finfo(np.float32).max)) == 0x7F80
    assert math.isnan(L.kda_bf16_to_f32(L.kda_bf16_from_f32(float("nan"))))
    assert L.kda_bf16_from_f32(0.0) == 0x0000
    assert L.kda_bf16_from_f32(-0.0) == 0x8000
    assert L.kda_bf16_from_f32(np.uint32(0x00018000).view(np.float32).item()) == 0x0002
    assert L.kda_bf16_ulp_distance(0x3F80, 0x3F81) == 1
    assert L.kda_bf16_ulp_distance(0x0001, 0x8001) == 2


def test_bf16_matches_torch_cast():
    # An independent library routine: torch's float32 -> bfloat16 cast is round-to-nearest-even.
    rng = np.random.default_rng(3)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 20000),
        rng.integers(0, 2**32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32),
    ]).astype(np.float32)
    x = x[np.isfinite(x)]
    got = o.bf16_from_f32(x)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(o.bf16_to_f32(got), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


# ---------------------------------------------------------------- rng (src/synth.rs:10-45)

def test_splitmix64_published_vector():
    # Vigna's splitmix64.c with state 1234567 gives this well-known sequence. The reference xors the seed
    # with 0x6a09e667f3bcc909 first (synth.rs:15-17), so undo that here.
    r = o.Rng(1234567 ^ 0x6A09E667F3BCC909)
    want = [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431,
            16408922859458223821]
    assert [r.next_u64() for _ in range(5)] == want


def test_uniform_is_24_bit_in_f32():
    r1, r2 = o.Rng(5), o.Rng(5)
    for _ in range(100):
        u = r1.next_u64()
        want = np.float32(-2.0) + (np.float32(3.0) - np.float32(-2.0)) * (np.float32(u >> 40) / np.float32(1 << 24))
        assert r2.uniform(-2.0, 3.0) == want
    x = o.Rng(6).fill_bf16(1000, -2.0, 2.0)
    assert np.array_equal(x, o.bf16_round(x)) and x.min() >= -2.0 and x.max() <= 2.0


def test_normal_moments():
    x = o.Rng(7).normal(200000).astype(np.float64)
    assert abs(x.mean()) < 0.01 and abs(x.std() - 1.0) < 0.01
    assert abs(((x - x.mean()) ** 4).mean() / x.var() ** 2 - 3.0) < 0.1


# ---------------------------------------------------------------- gates (cpu_reference.rs:36-55)

def test_forget_gate_and_beta_hand_values():
    assert o.log_decay(0.0, 0.0, 0.0, -5.0) == -2.5
    d = o.decay(0.0, 0.0, 1.0, -5.0)
    assert abs(d - math.exp(-2.5)) < 1e-8
    assert abs(o.decay(1e4, 0.0, 1.0, -5.0) - math.exp(-5.0)) < 1e-9
    assert o.decay(-1e4, 0.0, 1.0, -5.0) == 1.0
    assert o.log_decay(1.0, -1.0, 3.0, -5.0) == -2.5
    assert o.decay(2.0, -1.0, 0.5, -5.0) == o.decay(0.5, 0.0, 1.0, -5.0)
    assert o.beta(0.0) == 0.5
    assert o.beta(20.0) == 1.0
    assert o.beta(-200.0) == 0.0
    assert o.beta(1.0) == o.bf16_round(np.float32(0.7310586)).item()


def test_gates_against_f64_closed_form():
    rng = np.random.default_rng(11)
    for _ in range(500):
        a, dt, al = rng.uniform(-4, 4), rng.uniform(-1, 1), rng.uniform(-1.5, 1.5)
        a32, dt32, al32 = np.float32(a), np.float32(dt), np.float32(al)
        want = -5.0 / (1.0 + math.exp(-math.exp(float(al32)) * (float(a32) + float(dt32))))
        assert abs(o.log_decay(a32, dt32, al32, -5.0) - want) < 4e-6 * max(1.0, abs(want))
        got = o.decay(a32, dt32, np.float32(math.exp(float(al32))), -5.0)
        assert abs(got - math.exp(want)) < 4e-6 * math.exp(want) + 1e-9


# ---------------------------------------------------------------- conv (cpu_reference.rs:57-100)

def one_head(w):
    p = o.synth_layer(1, 1)
    p.conv_w = np.tile(np.asarray(w, np.float32), p.channels())
    return p


def test_conv_hand_values():
    p = one_head([1.0, 2.0, 3.0, 4.0])
    c = p.channels()
    conv = np.repeat(np.arange(1, WINDOW + 1, dtype=np.float32), c)
    rows = o.synth_rows(1, 2, 2)
    rows.qkv[:c] = 4.0
    rows.qkv[c:] = 5.0
    for r, want in [(0, 30.0), (1, 40.0)]:
        q, k, v = o.conv_qkv(p, conv, rows, r, 0, o.FUSED)
        assert np.all(np.concatenate([q, k, v]) == want), r
    rows.qkv[:c] = -11.0
    q, _, _ = o.conv_qkv(p, conv, rows, 0, 0, o.FUSED)
    want = o.bf16_round(np.float32(-30.0) / (np.float32(1.0) + np.exp(np.float32(30.0)))).item()
    assert q[0] == want and -1e-11 < q[0] < 0.0
    rows2 = o.synth_rows(1, 2, 3)
    w1 = o.conv_shift(conv, rows2, 1)
    assert np.array_equal(w1[:c], conv[c:2 * c]) and np.array_equal(w1[c:2 * c], conv[2 * c:])
    assert np.array_equal(w1[2 * c:], rows2.qkv[:c])
    w2 = o.conv_shift(conv, rows2, 2)
    assert np.array_equal(w2[:c], conv[2 * c:]) and np.array_equal(w2[c:], rows2.qkv)
    assert np.array_equal(o.conv_shift(conv, rows2, 0), conv)


def test_conv_tap_order_and_channel_blocks():
    # Distinct taps and distinct q | k | v blocks: a transposed weight or a swapped block fails.
    heads = 2
    p = o.synth_layer(heads, 21)
    conv = o.synth_conv_window(heads, 21)
    rows = o.synth_rows(heads, 5, 21)
    c = p.channels()
    seq = np.concatenate([conv.reshape(WINDOW, c), rows.qkv.reshape(5, c)]).astype(np.float64)
    w = p.conv_w.reshape(c, 4).astype(np.float64)
    for r in (0, 2, 4):
        acc = sum(w[:, tap] * seq[r + tap] for tap in range(4))
        want = acc / (1.0 + np.exp(-acc))
        for h in range(heads):
            q, k, v = o.conv_qkv(p, conv, rows, r, h, o.F32)
            blocks = [want[h * DK:(h + 1) * DK], want[heads * DK + h * DK:heads * DK + (h + 1) * DK],
                      want[2 * heads * DK + h * DK:2 * heads * DK + (h + 1) * DK]]
            for got, wnt in zip((q, k, v), blocks):
                assert np.max(np.abs(got - wnt)) < 2e-6


# ---------------------------------------------------------------- butterfly (cpu_reference.rs:102-121)

def test_warp_sum_is_the_butterfly():
    lanes = np.zeros(32, np.float32)
    lanes[0], lanes[16], lanes[1] = 1e8, -1e8, 1.0
    seq = np.float32(0.0)
    for x in lanes:
        seq = np.float32(seq + x)
    assert seq == 0.0
    assert o.warp_sum(lanes) == 1.0
    lanes = np.zeros(32, np.float32)
    lanes[0], lanes[1], lanes[17] = 1.0, 1e8, -1e8
    assert o.warp_sum(lanes) == 1.0
    assert o.warp_sum(np.arange(32, dtype=np.float32)) == 496.0


# ---------------------------------------------------------------- norms (cpu_reference.rs:123-145)

def test_l2norm_and_gated_norm_hand_values():
    x = np.zeros(DK, np.float32)
    x[5], x[9] = 3.0, 4.0
    y = o.l2norm(x)
    n = np.sqrt(np.float32(25.0) + np.float32(1e-6))
    assert y[5] == np.float32(3.0) * (np.float32(1.0) / n)
    assert y[9] == np.float32(4.0) * (np.float32(1.0) / n)
    yq = o.l2norm(x, o.q_scale())
    assert yq[5] == y[5] * (np.float32(1.0) / np.sqrt(np.float32(128.0)))
    yl = o.literal_l2norm(x)
    assert abs(yl[9] - y[9]) <= np.finfo(np.float32).eps * y[9]
    yc = np.full(DV, 0.5, np.float32)
    w = np.full(DV, 2.0, np.float32)
    gate = np.zeros(DV, np.float32)
    got = o.gated_rmsnorm(yc, w, gate, 1e-5)
    want = o.bf16_round(np.float32(2.0) * (np.float32(0.5) * (np.float32(1.0) / np.sqrt(np.float32(0.25) + np.float32(1e-5))))
                        * np.float32(0.5)).item()
    assert np.all(got == want) and abs(want - 1.0) < 1e-2


# ---------------------------------------------------------------- delta rule (cpu_reference.rs:147-207)

def test_delta_rule_writes_the_value_under_its_key():
    rng = o.Rng(9)
    s0 = rng.fill(DV * DK, -0.5, 0.5)
    s = s0.copy()
    k = np.zeros(DK, np.float32)
    k[3] = 1.0
    g = np.ones(DK, np.float32)
    v = rng.fill(DV, -2.0, 2.0)
    o.update(s, k, g, v, 1.0)
    read = o.read_out(s, k)
    assert np.all(np.abs(read - v) <= 4.0 * np.finfo(np.float32).eps * 2.5)
    keep = np.ones(DK, bool)
    keep[3] = False
    assert np.array_equal(s.reshape(DV, DK)[:, keep], s0.reshape(DV, DK)[:, keep])


def test_gates_saturated():
    heads = 2
    p = o.synth_layer(heads, 4)
    p.a_log[:] = 0.0
    p.dt_bias[:] = 0.0
    conv = o.synth_conv_window(heads, 4)
    s0 = o.synth_state(heads, 4, 0.5)
    rows = o.synth_rows(heads, 20, 4)
    rows.a[:] = 1e4
    rows.b[:] = -200.0
    r = o.chain(p, conv, s0, rows)
    assert np.all(r.saves.beta == 0.0)
    e5 = np.float32(o.decay(1e4, 0.0, 1.0, -5.0))
    assert np.all(r.saves.g == e5)
    expect = s0.copy()
    for _ in range(20):
        expect = expect * e5
    assert np.array_equal(r.state, expect)
    assert np.max(np.abs(r.state)) < 1e-40
    rows.a[:] = -1e4
    r = o.chain(p, conv, s0, rows)
    assert np.all(r.saves.g == 1.0)
    assert np.array_equal(r.state, s0)


def textbook_f64(q, k, v, g, beta, s0):
    """S_t = diag(e^g) S + beta k (v - k^T diag(e^g) S)^T, y_t = S_t^T q, S is [DK][DV], in f64."""
    s = s0.astype(np.float64).copy()
    ys = []
    for t in range(len(beta)):
        s = np.exp(g[t].astype(np.float64))[:, None] * s
        kt = k[t].astype(np.float64)
        s = s + beta[t] * np.outer(kt, v[t].astype(np.float64) - kt @ s)
        ys.append(q[t].astype(np.float64) @ s)
    return np.array(ys), s


def core_case(t, seed, slow=False):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((t, DK)).astype(np.float32)
    k = rng.standard_normal((t, DK)).astype(np.float32)
    v = rng.standard_normal((t, DV)).astype(np.float32)
    z = rng.standard_normal((t, DK))
    g = (-np.log1p(np.exp(z)) * (0.02 if slow else 1.0)).astype(np.float32)
    beta = (1.0 / (1.0 + np.exp(-rng.standard_normal(t)))).astype(np.float32)
    s0 = (rng.standard_normal((DK, DV)) * 0.3).astype(np.float32)
    return q, k, v, g, beta, s0


@pytest.mark.parametrize("slow", [False, True])
def test_literal_step_against_f64_textbook(slow):
    t = 12
    q, k, v, g, beta, s0 = core_case(t, 31, slow)
    qn = q / np.sqrt((q.astype(np.float64) ** 2).sum(1, keepdims=True) + 1e-6) / math.sqrt(128.0)
    kn = k / np.sqrt((k.astype(np.float64) ** 2).sum(1, keepdims=True) + 1e-6)
    y64, s64 = textbook_f64(qn, kn, v, g, beta, s0)
    s = s0.copy()
    ys = np.array([o.literal_step(s, q[i], k[i], v[i], g[i], float(beta[i])) for i in range(t)])
    assert rel_err(ys, y64) < 5e-6 and rel_err(s, s64) < 5e-6
    # The kernel-order update on the transposed state agrees with the same textbook recurrence.
    st = np.ascontiguousarray(s0.T)
    yk = []
    for i in range(t):
        o.update(st, kn[i].astype(np.float32), np.exp(g[i]).astype(np.float32), v[i], float(beta[i]))
        yk.append(o.read_out(st, qn[i].astype(np.float32)))
    assert rel_err(np.array(yk), y64) < 5e-6 and rel_err(st.T, s64) < 5e-6


# ---------------------------------------------------------------- bitwise self-consistency (cpu_reference.rs:209-257)

def test_replay_of_a_prefix_equals_the_shorter_chain_bitwise():
    heads = 4
    p = o.synth_layer(heads, 11)
    conv = o.synth_conv_window(heads, 11)
    s0 = o.synth_state(heads, 11, 0.5)
    rows = o.synth_rows(heads, 8, 11)
    full = o.chain(p, conv, s0, rows)
    assert np.array_equal(bits(o.replay(s0, full.saves, 8)), bits(full.state))
    for keep in range(9):
        short = o.chain(p, conv, s0, rows.slice(0, keep))
        assert np.array_equal(bits(o.replay(s0, full.saves, keep)), bits(short.state)), keep
        n = keep * heads * DV
        assert np.array_equal(bits(full.out[:n]), bits(short.out)), keep


@pytest.mark.parametrize("bf16_state", [False, True])
def test_serial_steps_equal_one_window_bitwise(bf16_state):
    heads = 3
    p = o.synth_layer(heads, 12)
    conv0 = o.synth_conv_window(heads, 12)
    s0 = o.synth_state(heads, 12, 0.5)
    if bf16_state:
        s0 = o.bf16_round(s0)
    rows = o.synth_rows(heads, 8, 12)
    run = o.chain_bf16_state if bf16_state else o.chain
    window = run(p, conv0, s0, rows)
    conv, s = conv0.copy(), s0.copy()
    n = heads * DV
    for r in range(8):
        row = rows.slice(r, 1)
        step = run(p, conv, s, row)
        assert np.array_equal(bits(step.out), bits(window.out[r * n:(r + 1) * n])), r
        conv = o.conv_shift(conv, row, 1)
        s = step.state
    assert np.array_equal(bits(s), bits(window.state))
    assert np.array_equal(conv, o.conv_shift(conv0, rows, 8))
    if bf16_state:
        assert np.array_equal(window.state, o.bf16_round(window.state))
        assert np.array_equal(bits(o.replay(s0, window.saves, 8, bf16_state=True)), bits(window.state))


# ---------------------------------------------------------------- chain vs literal (cpu_reference.rs:259-285)

def test_kernel_order_agrees_with_the_literal_formulation():
    heads = 4
    p = o.synth_layer(heads, 13)
    conv = o.synth_conv_window(heads, 13)
    s0 = o.synth_state(heads, 13, 0.5)
    rows = o.synth_rows(heads, 8, 13)
    a = o.chain(p, conv, s0, rows)
    b = o.literal_chain(p, conv, s0, rows)
    assert np.array_equal(bits(a.saves.v), bits(b.saves.v))
    assert np.array_equal(bits(a.saves.beta), bits(b.saves.beta))
    assert rel_err(a.state, b.state) < 1e-5
    assert rel_err(a.saves.k, b.saves.k) < 1e-6 and rel_err(a.saves.g, b.saves.g) < 1e-6
    ulp_y, n_y = bf16_diff(a.y, b.y)
    ulp_o, n_o = bf16_diff(a.out, b.out)
    assert ulp_y <= 1 and ulp_o <= 1
    assert n_y * 100 <= a.y.size and n_o * 100 <= a.out.size


def test_conv_roundings_differ_slightly():
    heads = 2
    p = o.synth_layer(heads, 14)
    conv = o.synth_conv_window(heads, 14)
    rows = o.synth_rows(heads, 4, 14)
    differ = total = 0
    for r in range(4):
        for h in range(heads):
            a = np.concatenate(o.conv_qkv(p, conv, rows, r, h, o.FUSED))
            b = np.concatenate(o.conv_qkv(p, conv, rows, r, h, o.UNFUSED))
            assert np.all(np.abs(a - b) <= np.maximum(np.maximum(np.abs(a), np.abs(b)), 1.0) / 64.0)
            differ += bf16_diff(a, b)[1]
            total += 3 * DK
    assert 0 < differ and differ * 2 < total


def test_state_layout_transpose():
    s = o.synth_state(2, 15, 1.0)
    t = o.transpose_state(s)
    assert t[DV + 3] == s[3 * DK + 1]
    assert t[DK * DV + 7 * DV + 2] == s[DK * DV + 2 * DK + 7]
    assert np.array_equal(o.transpose_state(t), s)


# ---------------------------------------------------------------- chunked (cpu_reference.rs:330-384)

def core_inputs(heads, t, seed):
    rng = o.Rng(seed)
    q = rng.fill_bf16(t * heads * DK, -1.0, 1.0)
    k = rng.fill_bf16(t * heads * DK, -1.0, 1.0)
    v = rng.fill_bf16(t * heads * DV, -1.0, 1.0)
    g = np.array([o.log_decay(rng.uniform(-4.0, 4.0), 0.0, 0.0, -5.0) for _ in range(t * heads * DK)], np.float32)
    beta = np.array([o.beta(rng.uniform(-4.0, 4.0)) for _ in range(t * heads)], np.float32)
    return q, k, v, g, beta


@pytest.mark.parametrize("t,chunk", [(1, 64), (7, 64), (64, 64), (65, 64), (150, 64), (40, 16)])
def test_chunked_form_matches_the_recurrence(t, chunk):
    heads = 2
    q, k, v, g, beta = core_inputs(heads, t, 16 + t)
    s0 = o.synth_state(heads, t, 0.5)
    s_rec = s0.copy()
    y_rec = o.recurrent_layer(heads, q, k, v, g, beta, s_rec)
    s_chunk = s0.copy()
    y_chunk = o.chunked_layer(heads, q, k, v, g, beta, s_chunk, chunk)
    assert rel_err(y_chunk, y_rec) < 2e-5 and rel_err(s_chunk, s_rec) < 2e-5


def test_chunked_head_against_f64_textbook():
    # The chunked form against the recurrence in f64: pins chunked_head independently of literal_step.
    t = 150
    q, k, v, g, beta, s0 = core_case(t, 41)
    qn = (q / np.sqrt((q.astype(np.float64) ** 2).sum(1, keepdims=True) + 1e-6) / math.sqrt(128.0)).astype(np.float32)
    kn = (k / np.sqrt((k.astype(np.float64) ** 2).sum(1, keepdims=True) + 1e-6)).astype(np.float32)
    y64, s64 = textbook_f64(qn, kn, v, g, beta, s0)
    for chunk in (64, 16, 1):
        s = s0.copy()
        y = o.chunked_head(qn, kn, v, g, beta, s, chunk).reshape(t, DV)
        assert rel_err(y, y64) < 2e-5 and rel_err(s, s64) < 2e-5, chunk


def test_baseline_config0_chunked_vs_recurrent():
    """benchmark configuration 0: one sequence, T=256, 64 heads, chunk 64, fp32, zero initial state."""
    heads, t = 64, 256
    rng = o.Rng(2026)
    q = rng.normal(t * heads * DK)
    k = rng.normal(t * heads * DK)
    v = rng.normal(t * heads * DV)
    beta = (1.0 / (1.0 + np.exp(-rng.normal(t * heads).astype(np.float64)))).astype(np.float32)
    g = (-np.log1p(np.exp(rng.normal(t * heads * DK).astype(np.float64)))).astype(np.float32)
    s_rec = np.zeros(heads * DK * DV, np.float32)
    s_chunk = np.zeros(heads * DK * DV, np.float32)
    y_rec = o.recurrent_layer(heads, q, k, v, g, beta, s_rec, threads=8)
    y_chunk = o.chunked_layer(heads, q, k, v, g, beta, s_chunk, 64, threads=8)
    assert rel_err(y_chunk, y_rec) < 2e-5 and rel_err(s_chunk, s_rec) < 2e-5


# ---------------------------------------------------------------- prefill host model (cpu_reference.rs:395-450)

@pytest.mark.parametrize("t,gates", [(1, "random"), (5, "random"), (16, "random"), (17, "random"), (40, "random"),
                                     (100, "random"), (48, "strongest"), (48, "mixed")])
def test_prefill_form_matches_the_chain(t, gates):
    heads = 2
    p = o.synth_layer(heads, 60 + t)
    conv = o.synth_conv_window(heads, 60 + t)
    s0 = o.synth_state(heads, 60 + t, 0.5)
    rows = o.synth_rows(heads, t, 60 + t)
    if gates == "strongest":
        rows.a[:] = 1e4
    elif gates == "mixed":
        idx = np.arange(rows.a.size) // (heads * DK)
        rows.a[:] = np.where(idx % 3 == 0, -1e4, 1e4).astype(np.float32)
    c = o.chain(p, conv, s0, rows)
    f = o.prefill(p, conv, s0, rows)
    assert rel_err(f.state, c.state) < 1e-5
    assert rel_err(f.y, c.y) < 1.0 / 256.0 and rel_err(f.out, c.out) < 1.0 / 256.0
    assert bf16_diff(f.out, c.out)[1] * 1000 <= c.out.size
    assert np.all(np.isfinite(f.state))


def test_threads_do_not_change_bits():
    heads = 8
    p = o.synth_layer(heads, 70)
    conv = o.synth_conv_window(heads, 70)
    s0 = o.synth_state(heads, 70, 0.5)
    rows = o.synth_rows(heads, 6, 70)
    a, b = o.chain(p, conv, s0, rows, threads=1), o.chain(p, conv, s0, rows, threads=4)
    assert np.array_equal(bits(a.out), bits(b.out)) and np.array_equal(bits(a.state), bits(b.state))


def test_oracle_exports_every_declared_symbol():
    import re, os
    hdr = open(os.path.join(os.path.dirname(o.__file__), "kda_ref.h")).read()
    declared = set(re.findall(r"\b(kda_[a-z0-9_]+)\s*\(", hdr))
    assert declared == set(o.EXPORTS)
    for name in declared:
        assert hasattr(o.lib(), name)


def test_exact_replay_is_the_f64_recurrence():
    """The f64 yardstick of the accuracy tests against the same recurrence written with numpy."""
    heads, n = 2, 6
    p, conv, s0 = o.synth_layer(heads, 5), o.synth_conv_window(heads, 5), o.synth_state(heads, 5, 0.5)
    c = o.chain(p, conv, s0, o.synth_rows(heads, n, 5))
    got = o.exact_replay(s0, c.saves).reshape(heads, 128, 128)
    s = s0.astype(np.float64).reshape(heads, 128, 128).copy()
    k = c.saves.k.reshape(n, heads, 128).astype(np.float64)
    v = c.saves.v.reshape(n, heads, 128).astype(np.float64)
    g = c.saves.g.reshape(n, heads, 128).astype(np.float64)
    b = c.saves.beta.reshape(n, heads).astype(np.float64)
    for r in range(n):
        for h in range(heads):
            s[h] *= g[r, h][None, :]
            s[h] += np.outer((v[r, h] - s[h] @ k[r, h]) * b[r, h], k[r, h])
    assert np.max(np.abs(got - s)) <= 1e-15
    # a prefix, and the f32 chain is within f32 rounding of it
    assert np.array_equal(o.exact_replay(s0, c.saves, rows=0), s0.astype(np.float64))
    assert np.max(np.abs(c.state - got.reshape(-1))) <= 1e-6 * np.max(np.abs(got))
