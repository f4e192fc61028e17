// Tests of the C++ host layer (glm53f-afd_amd/host). `--cpu`: the argument checks, without touching a GPU
// (reference: crates/glm53f-kda/tests/gpu.rs:727-792, tests/gpu_prefill.rs:541-584, :623-650, and the unit tests
// of BatchMeta in src/kernel.rs). `--gpu`: launches through the wrappers, checked against the CPU oracle.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "kernel.hpp"
#include "kda_ref.h"   // the oracle: test infrastructure

using namespace glm53f_kda;

static int failures = 0;
#define EXPECT(cond)                                                          \
    do {                                                                      \
        if (!(cond)) {                                                        \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);       \
            ++failures;                                                       \
        }                                                                     \
    } while (0)
#define EXPECT_INVALID(expr)                                                  \
    do {                                                                      \
        Error e_ = (expr);                                                    \
        if (e_.kind != Error::Invalid) {                                      \
            std::printf("FAIL %s:%d: expected Invalid from %s, got kind %d (%s)\n", __FILE__, __LINE__, #expr, (int)e_.kind, e_.what.c_str()); \
            ++failures;                                                       \
        }                                                                     \
    } while (0)
#define EXPECT_OK(expr)                                                       \
    do {                                                                      \
        Error e_ = (expr);                                                    \
        if (!e_) {                                                            \
            std::printf("FAIL %s:%d: %s -> %s\n", __FILE__, __LINE__, #expr, e_.what.c_str()); \
            ++failures;                                                       \
        }                                                                     \
    } while (0)

// A fake device region: never dereferenced by check().
static Buf fake(uintptr_t addr, size_t bytes) { return Buf(reinterpret_cast<void*>(addr), bytes); }

static void cpu_tests() {
    const size_t h = 4, c = channels(h), n = state_len(h);
    Weights w{h, fake(0x1000, c * TAPS * 2), fake(0x2000, h * 4), fake(0x3000, h * DK * 4), fake(0x4000, DV * 2), RMS_EPS, LOWER_BOUND};
    EXPECT_OK(w.check());
    Weights bad_w = w;
    bad_w.dt_bias.bytes -= 4;
    EXPECT_INVALID(bad_w.check());

    const size_t rows = 5, ps = c + h;
    Buf p = fake(0x10000, rows * ps * 2), a = fake(0x20000, rows * h * DK * 2), g = fake(0x30000, rows * h * DV * 2);
    Buf out = fake(0x40000, rows * h * DV * 2), conv = fake(0x50000, WINDOW * c * 2), state = fake(0x60000, 3 * n * 4);
    Chain ch;
    ch.weights = &w; ch.rows = rows; ch.p = RowView(p, 0, ps); ch.b_off = (int64_t)c;
    ch.a = RowView::dense(a, h * DK); ch.g = RowView::dense(g, h * DV); ch.conv = conv; ch.state = state;
    ch.state_out = StateOut::in_place(); ch.out = RowView::dense(out, h * DV);
    float* so = nullptr;
    EXPECT_OK(ch.check(&so));
    EXPECT(so == state.ptr<float>(0));
    { Chain x = ch; x.rows = 0; EXPECT_INVALID(x.check(&so)); }
    { Chain x = ch; x.rows = rows + 1; EXPECT_INVALID(x.check(&so)); }                     // p, a, g, out too short
    { Chain x = ch; x.b_off = -1; EXPECT_INVALID(x.check(&so)); }                           // beta logits before the buffer
    { Chain x = ch; x.p = RowView(p, h, ps); x.b_off = -(int64_t)h; x.rows = rows - 1; EXPECT_OK(x.check(&so)); }
    { Chain x = ch; x.out = RowView(out, 0, h * DV - 8); EXPECT_INVALID(x.check(&so)); }    // out rows overlap
    { Chain x = ch; x.conv_offset = 1; EXPECT_INVALID(x.check(&so)); }
    { Chain x = ch; x.state_offset = 2 * n + 1; EXPECT_INVALID(x.check(&so)); }
    { Chain x = ch; x.state_out = StateOut::to(state, n); EXPECT_OK(x.check(&so)); EXPECT(so == state.ptr<float>(n)); }
    { Chain x = ch; x.state_out = StateOut::to(state, n / 2); EXPECT_INVALID(x.check(&so)); }   // partial overlap
    { Chain x = ch; x.state_out = StateOut::to(state, 0); EXPECT_OK(x.check(&so)); }            // coincides
    { Chain x = ch; x.state_out = StateOut::skip(); EXPECT_OK(x.check(&so)); EXPECT(so == nullptr); }
    Saves sv{h, rows, fake(0x70000, rows * h * DK * 4), fake(0x80000, rows * h * DV * 2), fake(0x90000, rows * h * DK * 4), fake(0xa0000, rows * h * 4)};
    { Chain x = ch; x.saves = &sv; EXPECT_OK(x.check(&so)); }
    { Saves s2 = sv; s2.rows = rows - 1; Chain x = ch; x.saves = &s2; EXPECT_INVALID(x.check(&so)); }
    { Saves s2 = sv; s2.heads = h + 1; Chain x = ch; x.saves = &s2; EXPECT_INVALID(x.check(&so)); }

    Stream st = Stream::null();
    EXPECT_OK(replay(h, rows, state, 0, state, n, sv, st, true));
    EXPECT_INVALID(replay(h, rows, state, 0, state, n / 2, sv, st, true));
    EXPECT_INVALID(replay(h, rows + 1, state, 0, state, 0, sv, st, true));
    EXPECT_OK(conv_shift(h, 2, conv, 0, RowView(p, 0, ps), st, true));
    EXPECT_INVALID(conv_shift(h, rows + 4, conv, 0, RowView(p, 0, ps), st, true));
    EXPECT_OK(conv_shift(h, 0, conv, 0, RowView(fake(0, 0), 0, ps), st, true));          // keeps nothing: reads no rows

    // BatchMeta (kernel.rs:432-471)
    BatchMeta meta(3);
    EXPECT_INVALID(meta.set({}));
    EXPECT_INVALID(meta.set({{1, 0, 0}, {1, 0, n}, {1, 0, 2 * n}, {1, 0, 3 * n}}));         // over capacity
    EXPECT_INVALID(meta.set({{2, 0, 0}}, {3}));                                             // keep > rows
    EXPECT_INVALID(meta.set({{2, 0, 0}, {1, 0, n}}, {1}));                                  // one keep per request
    EXPECT_INVALID(meta.set({{(size_t)2147483647, 0, 0}, {1, 0, n}}));                      // total rows overflow i32
    EXPECT_OK(meta.set({{2, 0, n}, {0, WINDOW * c, 2 * n}, {3, 0, 0}}, {1, 0, 3}));
    EXPECT(meta.total_rows() == 5 && meta.max_rows() == 3);

    Buf conv2 = fake(0x50000, 2 * WINDOW * c * 2);
    ChainBatch cb;
    cb.weights = &w; cb.p = RowView(p, 0, ps); cb.b_off = (int64_t)c; cb.a = RowView::dense(a, h * DK);
    cb.g = RowView::dense(g, h * DV); cb.conv = conv2; cb.state = state; cb.state_out = StateOut::in_place();
    cb.out = RowView::dense(out, h * DV);
    void* sov = nullptr;
    EXPECT_OK(cb.check(meta, StateType::F32, &sov));                                        // shared conv window is fine for a chain
    { BatchMeta m2(3); EXPECT_OK(m2.set({{2, 0, 0}, {3, 0, n / 2}})); EXPECT_INVALID(cb.check(m2, StateType::F32, &sov)); }  // states overlap
    { ChainBatch x = cb; x.state_out = StateOut::to(state); EXPECT_INVALID(x.check(meta, StateType::F32, &sov)); }         // To(same buffer)
    { ChainBatch x = cb; x.state_out = StateOut::to(fake(0x100000, 3 * n * 4)); EXPECT_OK(x.check(meta, StateType::F32, &sov)); }
    { ChainBatch x = cb; EXPECT_OK(x.check(meta, StateType::Bf16, &sov)); }                 // bf16: half the bytes needed
    { ChainBatch x = cb; x.state = fake(0x60000, 3 * n * 2 - 2); EXPECT_INVALID(x.check(meta, StateType::Bf16, &sov)); }
    { ChainBatch x = cb; x.ckpt = fake(0x200000, 5 * n * 2); EXPECT_INVALID(x.check(meta, StateType::Bf16, &sov)); }        // verify must Skip
    { ChainBatch x = cb; x.ckpt = fake(0x200000, 5 * n * 2); x.state_out = StateOut::skip(); EXPECT_OK(x.check(meta, StateType::Bf16, &sov)); }
    { ChainBatch x = cb; x.ckpt = fake(0x200000, 5 * n * 2 - 2); x.state_out = StateOut::skip(); EXPECT_INVALID(x.check(meta, StateType::Bf16, &sov)); }
    { ChainBatch x = cb; x.ckpt = fake(0x200000, 5 * n * 2); x.state_out = StateOut::skip(); EXPECT_INVALID(x.check(meta, StateType::F32, &sov)); }

    // replay_batch, select and conv_shift_batch across layers (kernel.rs:849-861, :927-937)
    const size_t layers = 3, stride = 3 * n;
    LayerSaves ls{layers, h, 5, fake(0x300000, layers * 5 * h * DK * 4), fake(0x400000, layers * 5 * h * DV * 2),
                  fake(0x500000, layers * 5 * h * DK * 4), fake(0x600000, layers * 5 * h * 4)};
    Buf big = fake(0x700000, layers * stride * 4);
    EXPECT_OK(replay_batch_as(meta, big, big, stride, ls, st, StateType::F32, true));
    EXPECT_INVALID(replay_batch_as(meta, big, big, stride - 1, ls, st, StateType::F32, true));   // layers' regions overlap
    { LayerSaves l2 = ls; l2.rows = 4; EXPECT_INVALID(replay_batch_as(meta, big, big, stride, l2, st, StateType::F32, true)); }
    { LayerSaves l2 = ls; l2.layers = 0; EXPECT_INVALID(replay_batch_as(meta, big, big, stride, l2, st, StateType::F32, true)); }
    EXPECT_OK(replay_layers(5, big, big, stride, ls, st, true));
    EXPECT_INVALID(replay_layers(6, big, big, stride, ls, st, true));
    EXPECT_INVALID(replay_layers(5, big, big, n - 1, ls, st, true));
    Buf ck = fake(0x800000, layers * 5 * n * 2);
    EXPECT_OK(select_batch_bf16_state(h, layers, meta, ck, 5 * n, fake(0x700000, layers * stride * 2), stride, st, true));
    EXPECT_INVALID(select_batch_bf16_state(h, layers, meta, ck, 5 * n - 8, fake(0x700000, layers * stride * 2), stride, st, true));
    EXPECT_INVALID(select_batch_bf16_state(h, 0, meta, ck, 5 * n, fake(0x700000, layers * stride * 2), stride, st, true));
    BatchMeta mconv(3);
    EXPECT_OK(mconv.set({{2, 0, 0}, {3, WINDOW * c, n}}));
    Buf convL = fake(0x900000, layers * 2 * WINDOW * c * 2), pL = fake(0xa00000, layers * rows * ps * 2);
    EXPECT_OK(conv_shift_batch(h, layers, mconv, convL, 2 * WINDOW * c, RowView(pL, 0, ps), rows * ps, st, true));
    EXPECT_INVALID(conv_shift_batch(h, layers, mconv, convL, 2 * WINDOW * c - 1, RowView(pL, 0, ps), rows * ps, st, true));
    EXPECT_INVALID(conv_shift_batch(h, layers, meta, convL, 2 * WINDOW * c, RowView(pL, 0, ps), rows * ps, st, true));  // windows overlap (meta shares one)
    EXPECT_INVALID(conv_shift_batch(h, 0, mconv, convL, 2 * WINDOW * c, RowView(pL, 0, ps), rows * ps, st, true));

    // prefill (kernel.rs:1043-1050, :1094-1096, :1031-1040, :975-986)
    PrefillWorkspace ws;
    ws.heads = h; ws.batch = 2; ws.rows_per_pass = 128;
    ws.buf = fake(0xb00000, PrefillWorkspace::bytes_for(h, 2, 128));
    // two chunks of two requests: linear in chunks, requests and heads
    EXPECT(ws.buf.bytes == 2 * 2 * h * (size_t)glm53f_kda_prefill_workspace_bytes(1, 1, PREFILL_CHUNK));
    EXPECT(glm53f_kda_prefill_workspace_bytes(1, 1, PREFILL_CHUNK) > 0);
    Prefill pf;
    pf.weights = &w; pf.rows = rows; pf.p = RowView(p, 0, ps); pf.b_off = (int64_t)c; pf.a = RowView::dense(a, h * DK);
    pf.g = RowView::dense(g, h * DV); pf.conv = conv; pf.state = state; pf.state_out = StateOut::in_place();
    pf.out = RowView::dense(out, h * DV); pf.workspace = &ws;
    float* wsp = nullptr; int32_t vb = 0; int64_t wsb = 0;
    EXPECT_OK(pf.check(&so, &vb, &wsp, &wsb));
    { Prefill x = pf; x.value_blocks = 3; EXPECT_INVALID(x.check(&so, &vb, &wsp, &wsb)); }
    { Prefill x = pf; x.state_out = StateOut::skip(); EXPECT_INVALID(x.check(&so, &vb, &wsp, &wsb)); }
    { Weights w2 = w; w2.lower = -6.0f; Prefill x = pf; x.weights = &w2; EXPECT_INVALID(x.check(&so, &vb, &wsp, &wsb)); }
    { PrefillWorkspace w2; w2.heads = h + 1; w2.batch = 2; w2.buf = ws.buf; Prefill x = pf; x.workspace = &w2; EXPECT_INVALID(x.check(&so, &vb, &wsp, &wsb)); }
    { Prefill x = pf; x.rows = 0; EXPECT_OK(x.check(&so, &vb, &wsp, &wsb)); }               // zero rows are legal for a prefill
    PrefillBatch pb;
    pb.weights = &w; pb.p = RowView(p, 0, ps); pb.b_off = (int64_t)c; pb.a = RowView::dense(a, h * DK);
    pb.g = RowView::dense(g, h * DV); pb.conv = conv2; pb.state = state; pb.state_out = StateOut::in_place();
    pb.out = RowView::dense(out, h * DV); pb.workspace = &ws;
    EXPECT_OK(pb.check(mconv, StateType::F32, &sov, &vb, &wsp, &wsb));
    EXPECT_INVALID(pb.check(meta, StateType::F32, &sov, &vb, &wsp, &wsb));                  // 3 requests, workspace for 2; windows shared
    { BatchMeta m2(3); EXPECT_OK(m2.set({{2, 0, 0}, {3, 0, n}})); EXPECT_INVALID(pb.check(m2, StateType::F32, &sov, &vb, &wsp, &wsb)); }  // windows overlap
    EXPECT(coincide_or_disjoint(0, 0, 4) && coincide_or_disjoint(0, 4, 4) && !coincide_or_disjoint(0, 3, 4));
}

static std::vector<uint16_t> enc(const std::vector<float>& x) {
    std::vector<uint16_t> o(x.size());
    kda_bf16_encode(x.data(), o.data(), (int64_t)x.size());
    return o;
}
static std::vector<float> dec(const std::vector<uint16_t>& x) {
    std::vector<float> o(x.size());
    kda_bf16_decode(x.data(), o.data(), (int64_t)x.size());
    return o;
}
static float rel_err(const std::vector<float>& a, const std::vector<float>& b) {
    float d = 0, m = 0;
    for (size_t i = 0; i < a.size(); ++i) { d = std::fmax(d, std::fabs(a[i] - b[i])); m = std::fmax(m, std::fabs(b[i])); }
    return d / std::fmax(m, 1e-30f);
}

static void gpu_tests() {
    const size_t h = 4, c = channels(h), n = state_len(h), rows = 6;
    std::vector<float> conv_w(c * TAPS), a_log(h), dt_bias(h * DK), norm_w(DV), qkv(rows * c), av(rows * h * DK), bv(rows * h),
        gate(rows * h * DV), conv(WINDOW * c), s0(n);
    kda_synth_layer((int32_t)h, 21, conv_w.data(), a_log.data(), dt_bias.data(), norm_w.data());
    kda_synth_rows((int32_t)h, (int32_t)rows, 21, qkv.data(), av.data(), bv.data(), gate.data());
    kda_synth_conv_window((int32_t)h, 21, conv.data());
    kda_synth_state((int32_t)h, 21, 0.5f, s0.data());
    // device staging: engine layout (beta logits behind q|k|v)
    const size_t ps = c + h;
    std::vector<float> prow(rows * ps);
    for (size_t r = 0; r < rows; ++r) {
        std::memcpy(&prow[r * ps], &qkv[r * c], c * 4);
        std::memcpy(&prow[r * ps + c], &bv[r * h], h * 4);
    }
    DeviceBuffer d_cw, d_al, d_dt, d_nw, d_p, d_a, d_g, d_out, d_conv, d_state, d_state2;
    EXPECT_OK(DeviceBuffer::from_slice(enc(conv_w), &d_cw));
    EXPECT_OK(DeviceBuffer::from_slice(a_log, &d_al));
    EXPECT_OK(DeviceBuffer::from_slice(dt_bias, &d_dt));
    EXPECT_OK(DeviceBuffer::from_slice(enc(norm_w), &d_nw));
    EXPECT_OK(DeviceBuffer::from_slice(enc(prow), &d_p));
    EXPECT_OK(DeviceBuffer::from_slice(enc(av), &d_a));
    EXPECT_OK(DeviceBuffer::from_slice(enc(gate), &d_g));
    EXPECT_OK(DeviceBuffer::zeroed(rows * h * DV * 2, &d_out));
    EXPECT_OK(DeviceBuffer::from_slice(enc(conv), &d_conv));
    EXPECT_OK(DeviceBuffer::from_slice(s0, &d_state));
    EXPECT_OK(DeviceBuffer::zeroed(n * 4, &d_state2));
    Weights w{h, d_cw, d_al, d_dt, d_nw, RMS_EPS, LOWER_BOUND};
    SavesStorage sv;
    EXPECT_OK(SavesStorage::alloc(h, rows, &sv));
    Stream stream = Stream::null();
    EXPECT_OK(Stream::create(&stream));

    // the oracle
    kda_layer lp{(int32_t)h, conv_w.data(), a_log.data(), dt_bias.data(), norm_w.data(), RMS_EPS, LOWER_BOUND};
    kda_rows rw{(int32_t)h, (int32_t)rows, qkv.data(), av.data(), bv.data(), gate.data()};
    std::vector<float> o_out(rows * h * DV), o_y(rows * h * DV), o_state(n), ok_(rows * h * DK), ov(rows * h * DV), og(rows * h * DK), ob(rows * h);
    kda_chain_with(&lp, conv.data(), s0.data(), &rw, KDA_FUSED, 0, o_out.data(), o_y.data(), o_state.data(), ok_.data(), ov.data(), og.data(), ob.data(), 1);

    // Chain through the wrapper: outputs within a bf16 rounding, the CPU replay of the device's saves bit for bit
    Chain ch;
    ch.weights = &w; ch.rows = rows; ch.p = RowView(d_p, 0, ps); ch.b_off = (int64_t)c; ch.a = RowView::dense(d_a, h * DK);
    ch.g = RowView::dense(d_g, h * DV); ch.conv = d_conv; ch.state = d_state; ch.state_out = StateOut::to(d_state2, 0);
    ch.out = RowView::dense(d_out, h * DV); ch.saves = &sv.view;
    EXPECT_OK(ch.launch(stream));
    EXPECT_OK(stream.synchronize());
    std::vector<uint16_t> out16, v16;
    std::vector<float> st, sk, sg, sb;
    EXPECT_OK(d_out.to_vec(&out16));
    EXPECT_OK(d_state2.to_vec(&st));
    EXPECT_OK(sv.k.to_vec(&sk)); EXPECT_OK(sv.v.to_vec(&v16)); EXPECT_OK(sv.g.to_vec(&sg)); EXPECT_OK(sv.b.to_vec(&sb));
    EXPECT(rel_err(dec(out16), o_out) <= 1.0f / 256.0f);
    EXPECT(rel_err(st, o_state) <= 1e-3f);
    std::vector<float> rep(n), svv = dec(v16);
    kda_replay_with((int32_t)h, s0.data(), sk.data(), svv.data(), sg.data(), sb.data(), (int32_t)rows, 0, rep.data());
    EXPECT(std::memcmp(rep.data(), st.data(), n * 4) == 0);

    // replay of a prefix through the wrapper == CPU replay, bit for bit; conv shift exact
    EXPECT_OK(replay(h, 4, d_state, 0, d_state2, 0, sv.view, stream));
    EXPECT_OK(conv_shift(h, 4, d_conv, 0, RowView(d_p, 0, ps), stream));
    EXPECT_OK(stream.synchronize());
    EXPECT_OK(d_state2.to_vec(&st));
    kda_replay_with((int32_t)h, s0.data(), sk.data(), svv.data(), sg.data(), sb.data(), 4, 0, rep.data());
    EXPECT(std::memcmp(rep.data(), st.data(), n * 4) == 0);
    std::vector<uint16_t> cv16;
    EXPECT_OK(d_conv.to_vec(&cv16));
    std::vector<float> want_conv(WINDOW * c);
    kda_conv_shift((int32_t)h, conv.data(), qkv.data(), (int32_t)rows, 4, want_conv.data());
    EXPECT(dec(cv16) == want_conv);

    // Batch: bf16 pool of 3 slots, two requests (rows 4 and 2), verify with checkpoints, then select
    const size_t slots = 3;
    std::vector<float> pool(slots * n);
    kda_synth_state((int32_t)h, 22, 0.5f, pool.data());   // the first slot's worth; fill the rest by shifting seeds
    for (size_t s = 1; s < slots; ++s) kda_synth_state((int32_t)h, 22 + s, 0.5f, pool.data() + s * n);
    for (float& x : pool) x = kda_bf16_round(x);
    DeviceBuffer d_pool, d_convs, d_ck;
    EXPECT_OK(DeviceBuffer::from_slice(enc(pool), &d_pool));
    std::vector<float> convs(slots * WINDOW * c);
    for (size_t s = 0; s < slots; ++s) kda_synth_conv_window((int32_t)h, 30 + s, convs.data() + s * WINDOW * c);
    EXPECT_OK(DeviceBuffer::from_slice(enc(convs), &d_convs));
    EXPECT_OK(DeviceBuffer::zeroed(rows * n * 2, &d_ck));
    BatchMeta meta(0);
    EXPECT_OK(BatchMeta::create(4, &meta));
    EXPECT_OK(meta.set({{4, 2 * WINDOW * c, 2 * n}, {2, 0, 0}}, {3, 0}));
    ChainBatch cb;
    cb.weights = &w; cb.p = RowView(d_p, 0, ps); cb.b_off = (int64_t)c; cb.a = RowView::dense(d_a, h * DK);
    cb.g = RowView::dense(d_g, h * DV); cb.conv = d_convs; cb.state = d_pool; cb.state_out = StateOut::skip();
    cb.out = RowView::dense(d_out, h * DV); cb.saves = &sv.view; cb.ckpt = d_ck;
    EXPECT_OK(cb.launch_bf16_state(meta, stream));
    EXPECT_OK(select_batch_bf16_state(h, 1, meta, d_ck, 0, d_pool, 0, stream));
    EXPECT_OK(stream.synchronize());
    std::vector<uint16_t> pool16;
    EXPECT_OK(d_pool.to_vec(&pool16));
    EXPECT_OK(sv.k.to_vec(&sk)); EXPECT_OK(sv.v.to_vec(&v16)); EXPECT_OK(sv.g.to_vec(&sg)); EXPECT_OK(sv.b.to_vec(&sb));
    svv = dec(v16);
    // request 0 kept 3 rows in slot 2: the CPU's bf16 replay of the device saves; slots 0 and 1 untouched
    kda_replay_with((int32_t)h, pool.data() + 2 * n, sk.data(), svv.data(), sg.data(), sb.data(), 3, 1, rep.data());
    std::vector<float> got = dec(pool16);
    EXPECT(std::memcmp(rep.data(), got.data() + 2 * n, n * 4) == 0);
    EXPECT(std::memcmp(pool.data(), got.data(), 2 * n * 4) == 0);

    // A decode round in one launch: the chain in place with the windows advanced == the chain, then conv_shift_batch
    {
        DeviceBuffer d_pool_a, d_pool_b, d_conv_a, d_conv_b, d_out_b;
        EXPECT_OK(DeviceBuffer::from_slice(enc(pool), &d_pool_a));
        EXPECT_OK(DeviceBuffer::from_slice(enc(pool), &d_pool_b));
        EXPECT_OK(DeviceBuffer::from_slice(enc(convs), &d_conv_a));
        EXPECT_OK(DeviceBuffer::from_slice(enc(convs), &d_conv_b));
        EXPECT_OK(DeviceBuffer::zeroed(rows * h * DV * 2, &d_out_b));
        BatchMeta m2(0);
        EXPECT_OK(BatchMeta::create(4, &m2));
        EXPECT_OK(m2.set({{4, 2 * WINDOW * c, 2 * n}, {2, 0, 0}}, {4, 2}));
        ChainBatch two = cb;
        two.ckpt = Buf(); two.saves = nullptr; two.conv = d_conv_a; two.state = d_pool_a; two.state_out = StateOut::in_place();
        EXPECT_OK(two.launch_bf16_state(m2, stream));
        EXPECT_OK(conv_shift_batch(h, 1, m2, d_conv_a, 0, RowView(d_p, 0, ps), 0, stream));
        ChainBatch one = two;
        one.conv = d_conv_b; one.state = d_pool_b; one.out = RowView::dense(d_out_b, h * DV); one.advance_conv = true;
        EXPECT_OK(one.launch_bf16_state(m2, stream));
        EXPECT_OK(stream.synchronize());
        std::vector<uint16_t> pa, pb, ca, cbv, oa, ob2;
        EXPECT_OK(d_pool_a.to_vec(&pa)); EXPECT_OK(d_pool_b.to_vec(&pb));
        EXPECT_OK(d_conv_a.to_vec(&ca)); EXPECT_OK(d_conv_b.to_vec(&cbv));
        EXPECT_OK(d_out.to_vec(&oa)); EXPECT_OK(d_out_b.to_vec(&ob2));
        EXPECT(pa == pb);
        EXPECT(ca == cbv);
        EXPECT(oa == ob2);
        // a verify round cannot advance its windows, and shared windows are rejected
        { ChainBatch x = one; x.ckpt = d_ck; x.state_out = StateOut::skip(); EXPECT_INVALID(x.launch_bf16_state(m2, stream)); }
        BatchMeta m3(0);
        EXPECT_OK(BatchMeta::create(4, &m3));
        EXPECT_OK(m3.set({{4, 0, 2 * n}, {2, 0, 0}}, {4, 2}));
        EXPECT_INVALID(one.launch_bf16_state(m3, stream));
        { ChainBatch x = one; x.advance_conv = false; EXPECT_OK(x.launch_bf16_state(m3, stream)); }
        EXPECT_OK(stream.synchronize());
    }

    // Prefill through the wrapper against the literal recurrence
    PrefillWorkspace ws;
    EXPECT_OK(PrefillWorkspace::within(h, 1, 1 << 20, &ws));
    // the largest whole number of chunks whose workspace fits the budget, by the library's own figure per chunk
    EXPECT(ws.rows_per_pass == ((size_t)(1 << 20) / (size_t)glm53f_kda_prefill_workspace_bytes((int32_t)h, 1, PREFILL_CHUNK)) * PREFILL_CHUNK);
    EXPECT(ws.rows_per_pass >= PREFILL_CHUNK);
    EXPECT_OK(d_state.upload(s0));
    EXPECT_OK(d_conv.upload(enc(conv)));
    Prefill pf;
    pf.weights = &w; pf.rows = rows; pf.p = RowView(d_p, 0, ps); pf.b_off = (int64_t)c; pf.a = RowView::dense(d_a, h * DK);
    pf.g = RowView::dense(d_g, h * DV); pf.conv = d_conv; pf.state = d_state; pf.state_out = StateOut::in_place();
    pf.out = RowView::dense(d_out, h * DV); pf.workspace = &ws;
    EXPECT_OK(pf.launch(stream));
    EXPECT_OK(stream.synchronize());
    kda_literal_chain(&lp, conv.data(), s0.data(), &rw, KDA_FUSED, o_out.data(), o_y.data(), o_state.data(), nullptr, nullptr, nullptr, nullptr, 1);
    EXPECT_OK(d_state.to_vec(&st));
    EXPECT_OK(d_out.to_vec(&out16));
    EXPECT(rel_err(st, o_state) <= 1e-3f);
    EXPECT(rel_err(dec(out16), o_out) <= 1.0f / 128.0f);
    EXPECT_OK(d_conv.to_vec(&cv16));
    kda_conv_shift((int32_t)h, conv.data(), qkv.data(), (int32_t)rows, (int32_t)rows, want_conv.data());
    EXPECT(dec(cv16) == want_conv);
    // a rejected launch leaves an Invalid error, as the launcher's code 1 does
    { Prefill x = pf; x.value_blocks = 3; EXPECT_INVALID(x.launch(stream)); }
    Event e0, e1;
    EXPECT_OK(e0.record(stream)); EXPECT_OK(e1.record(stream)); EXPECT_OK(e1.synchronize());
    float ms = -1; EXPECT_OK(e1.elapsed_since(e0, &ms)); EXPECT(ms >= 0);
    size_t fr = 0, tot = 0; EXPECT_OK(mem_info(&fr, &tot)); EXPECT(tot > 0);
}

int main(int argc, char** argv) {
    const std::string mode = argc > 1 ? argv[1] : "--cpu";
    if (mode == "--cpu") {
        cpu_tests();
    } else {
        if (device_count() == 0) {
            std::printf("no GPU: skipped\n");
            return 77;
        }
        gpu_tests();
    }
    std::printf("%s: %d failure(s)\n", mode.c_str(), failures);
    return failures == 0 ? 0 : 1;
}
