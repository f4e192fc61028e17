// Tests of the KDA layer's call site in C++ (glm53f-afd_amd/host/kda_layer.hpp: the counterpart of the reference's
// GlmForward::kda and the KDA part of GlmForward::commit). `--cpu`: the shape arithmetic. `--gpu`: a verify round and
// its commit against serial decode rounds, bit for bit, on the pool's arenas (as the reference's engine tests hold
// verify + commit to decode: crates/glm53f-forward/tests/gpu_engine.rs), with saves + replay and with checkpoints +
// selection; the chunked prefill against the chain on the same rows.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "kda_layer.hpp"
#include "kda_ref.h"   // the oracle's bf16 conversions and synthetic layers: test infrastructure

using namespace glm53f_forward;
using glm53f_kda::device_count;

static int failures = 0;
#define EXPECT(cond)                                                          \
    do {                                                                      \
        if (!(cond)) {                                                        \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);       \
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
#define EXPECT_INVALID(expr)                                                  \
    do {                                                                      \
        Error e_ = (expr);                                                    \
        if (e_.kind != Error::Invalid) {                                      \
            std::printf("FAIL %s:%d: expected Invalid from %s, got kind %d (%s)\n", __FILE__, __LINE__, #expr, (int)e_.kind, e_.what.c_str()); \
            ++failures;                                                       \
        }                                                                     \
    } while (0)

static void cpu_tests() {
    KdaShape m;   // the model's
    EXPECT(m.width() == 8192 && m.qkv() == 24576 && m.p_cols() == 24640 && m.dim() == 128);
    EXPECT(m.state_elems() == size_t(64) * 128 * 128 && m.conv_elems() == size_t(3) * 24576);
    KdaConfig c;
    EXPECT(c.chunked_prefill && !c.fused_decode_shift && !c.verify_checkpoints);
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
static std::vector<float> values(size_t n, uint32_t seed, float scale) {
    std::vector<float> v(n);
    uint32_t s = seed * 2654435761u + 12345u;
    for (size_t i = 0; i < n; ++i) {
        s = s * 1664525u + 1013904223u;
        v[i] = scale * ((float)(s >> 8) / 8388608.0f - 1.0f);
    }
    return v;
}

struct LayerOnDevice {
    DeviceBuffer qkvb, fga, fgb, o, conv_w, a_log, dt_bias, norm_w;
    KdaW w;
};

static void make_layer(const KdaShape& sh, uint32_t seed, LayerOnDevice* L) {
    const size_t h = sh.heads, c = glm53f_kda::channels(h);
    EXPECT_OK(DeviceBuffer::from_slice(enc(values(sh.p_cols() * sh.hidden, seed + 1, 0.08f)), &L->qkvb));
    EXPECT_OK(DeviceBuffer::from_slice(enc(values(2 * sh.dim() * sh.hidden, seed + 2, 0.08f)), &L->fga));
    EXPECT_OK(DeviceBuffer::from_slice(enc(values(2 * sh.width() * sh.dim(), seed + 3, 0.15f)), &L->fgb));
    EXPECT_OK(DeviceBuffer::from_slice(enc(values(sh.hidden * sh.width(), seed + 4, 0.03f)), &L->o));
    std::vector<float> conv_w(c * glm53f_kda::TAPS), a_log(h), dt_bias(h * glm53f_kda::DK), norm_w(glm53f_kda::DV);
    kda_synth_layer((int32_t)h, seed, conv_w.data(), a_log.data(), dt_bias.data(), norm_w.data());
    EXPECT_OK(DeviceBuffer::from_slice(enc(conv_w), &L->conv_w));
    EXPECT_OK(DeviceBuffer::from_slice(a_log, &L->a_log));
    EXPECT_OK(DeviceBuffer::from_slice(dt_bias, &L->dt_bias));
    EXPECT_OK(DeviceBuffer::from_slice(enc(norm_w), &L->norm_w));
    L->w.qkvb = Bf16Mat{L->qkvb.ptr<uint16_t>(), sh.p_cols(), sh.hidden, sh.hidden};
    L->w.fga = Bf16Mat{L->fga.ptr<uint16_t>(), 2 * sh.dim(), sh.hidden, sh.hidden};
    L->w.fgb = Bf16Mat{L->fgb.ptr<uint16_t>(), sh.width(), sh.dim(), sh.dim(), 2, sh.width() * sh.dim()};
    L->w.o = Bf16Mat{L->o.ptr<uint16_t>(), sh.hidden, sh.width(), sh.width()};
    L->w.core = glm53f_kda::Weights{h, Buf(L->conv_w), Buf(L->a_log), Buf(L->dt_bias), Buf(L->norm_w)};
}

struct Pool {
    DeviceBuffer state, conv;
    KdaPool view;
};
static void make_pool(const KdaShape& sh, size_t slots, const std::vector<uint16_t>& state0, const std::vector<uint16_t>& conv0, Pool* p) {
    EXPECT_OK(DeviceBuffer::from_slice(state0, &p->state));
    EXPECT_OK(DeviceBuffer::from_slice(conv0, &p->conv));
    p->view = KdaPool{Buf(p->state), Buf(p->conv), true, slots};
}

// A verify round of reqs (rows each) and its commit (keep each), against serial decode rounds of the kept rows.
static void verify_commit_equals_decode(bool checkpoints, bool fused_shift) {
    KdaShape sh; sh.hidden = 512; sh.heads = 16; sh.layers = 2;
    const size_t slots = 7, drafts = 4;
    const std::vector<Req> reqs = {{4, drafts}, {1, drafts}, {6, drafts}, {0, drafts}, {3, drafts}};
    const std::vector<size_t> keep = {4, 2, 1, 4, 3};
    const size_t rows = reqs.size() * drafts;
    Stream stream = Stream::null();
    EXPECT_OK(Stream::create(&stream));
    GemmPolicy policy; policy.gemv_max_rows = 0;    // every row count through the GEMM for 9 to 64 rows: one set of bits
    KdaConfig cfg; cfg.verify_checkpoints = checkpoints; cfg.fused_decode_shift = fused_shift;
    KdaEngine ev, ed;
    EXPECT_OK(KdaEngine::create(stream, sh, cfg, policy, 64, 32, 8, &ev));
    EXPECT_OK(KdaEngine::create(stream, sh, cfg, policy, 64, 32, 8, &ed));
    LayerOnDevice layer[2];
    make_layer(sh, 40, &layer[0]);
    make_layer(sh, 50, &layer[1]);
    const std::vector<uint16_t> state0 = enc(values(slots * sh.layers * sh.state_elems(), 3, 0.05f));
    const std::vector<uint16_t> conv0 = enc(values(slots * sh.layers * sh.conv_elems(), 4, 1.0f));
    Pool pv, pd;
    make_pool(sh, slots, state0, conv0, &pv);
    make_pool(sh, slots, state0, conv0, &pd);
    // the rows entering each layer (the test feeds every layer its own rows: what lies between two KDA layers of the
    // model is not this path)
    std::vector<std::vector<uint16_t>> x(sh.layers);
    for (size_t j = 0; j < sh.layers; ++j) x[j] = enc(values(rows * sh.hidden, 60 + (uint32_t)j, 1.0f));

    // the verify round
    std::vector<std::vector<uint16_t>> out_v(sh.layers);
    EXPECT_OK(ev.upload_meta(reqs));
    for (size_t j = 0; j < sh.layers; ++j) {
        EXPECT_OK(ev.s.normed.upload(x[j]));
        EXPECT_OK(ev.kda_layer(j, Mode::Verify, rows, 0, layer[j].w, pv.view, stream));
        EXPECT_OK(stream.synchronize());
        EXPECT_OK(ev.s.attn_out.download<uint16_t>(rows * sh.hidden, &out_v[j]));
    }
    std::vector<uint16_t> st, cv;
    EXPECT_OK(pv.state.to_vec(&st));
    EXPECT_OK(pv.conv.to_vec(&cv));
    EXPECT(st == state0 && cv == conv0);   // a verify round writes neither arena
    EXPECT_OK(ev.commit(reqs, keep, pv.view, stream));
    EXPECT_OK(stream.synchronize());

    // serial decode rounds over the kept rows
    size_t compared = 0;
    for (size_t t = 0; t < drafts; ++t) {
        std::vector<Req> live;
        std::vector<size_t> idx;
        for (size_t i = 0; i < reqs.size(); ++i)
            if (keep[i] > t) { live.push_back({reqs[i].slot, 1}); idx.push_back(i); }
        if (live.empty()) break;
        EXPECT_OK(ed.upload_meta(live));
        for (size_t j = 0; j < sh.layers; ++j) {
            std::vector<uint16_t> xt(live.size() * sh.hidden);
            for (size_t r = 0; r < live.size(); ++r)
                std::memcpy(&xt[r * sh.hidden], &x[j][(idx[r] * drafts + t) * sh.hidden], sh.hidden * 2);
            EXPECT_OK(ed.s.normed.upload(xt));
            EXPECT_OK(ed.kda_layer(j, Mode::Decode, live.size(), 0, layer[j].w, pd.view, stream));
            EXPECT_OK(stream.synchronize());
            std::vector<uint16_t> out_d;
            EXPECT_OK(ed.s.attn_out.download<uint16_t>(live.size() * sh.hidden, &out_d));
            for (size_t r = 0; r < live.size(); ++r) {
                const bool same = std::memcmp(&out_d[r * sh.hidden], &out_v[j][(idx[r] * drafts + t) * sh.hidden], sh.hidden * 2) == 0;
                EXPECT(same);
                ++compared;
            }
        }
    }
    std::vector<uint16_t> st_v, cv_v, st_d, cv_d;
    EXPECT_OK(pv.state.to_vec(&st_v)); EXPECT_OK(pv.conv.to_vec(&cv_v));
    EXPECT_OK(pd.state.to_vec(&st_d)); EXPECT_OK(pd.conv.to_vec(&cv_d));
    EXPECT(st_v == st_d);
    EXPECT(cv_v == cv_d);
    EXPECT(st_v != state0);
    std::printf("verify + commit (%s, %s decode) == serial decode rounds: %zu output rows, states and windows of %zu slots x %zu layers, bit for bit\n",
                checkpoints ? "checkpoints + selection" : "saves + replay", fused_shift ? "one-launch" : "two-launch", compared, slots, sh.layers);

    // host-side rejections of the call site
    EXPECT_INVALID(ev.commit(reqs, {4, 2, 0, 4, 3}, pv.view, stream));
    EXPECT_INVALID(ev.commit(reqs, {4, 2, 1, 5, 3}, pv.view, stream));
    EXPECT_INVALID(ev.commit(reqs, {4, 2}, pv.view, stream));
    EXPECT_OK(ev.upload_meta(reqs));
    EXPECT_INVALID(ev.kda_layer(2, Mode::Decode, rows, 0, layer[0].w, pv.view, stream));
    EXPECT_INVALID(ev.kda_layer(0, Mode::Decode, rows - 1, 0, layer[0].w, pv.view, stream));
    EXPECT_INVALID(ev.kda_layer(0, Mode::Verify, rows, 20, layer[0].w, pv.view, stream));
}

static double rel_err(const std::vector<float>& a, const std::vector<float>& b) {
    double d = 0, m = 0;
    for (size_t i = 0; i < a.size(); ++i) { d = std::fmax(d, std::fabs((double)a[i] - b[i])); m = std::fmax(m, std::fabs((double)b[i])); }
    return d / std::fmax(m, 1e-30);
}

// A prefill pass in the chunked form against the same pass through the chain.
static void prefill_chunked_against_chain() {
    KdaShape sh; sh.hidden = 512; sh.heads = 16; sh.layers = 2;
    const size_t slots = 4;
    const std::vector<Req> reqs = {{2, 100}, {0, 70}, {3, 9}};
    const size_t rows = 179;
    Stream stream = Stream::null();
    EXPECT_OK(Stream::create(&stream));
    KdaConfig chunked, chain;
    chunked.prefill_rows = 64;     // several passes per request
    chain.chunked_prefill = false;
    KdaEngine ec, er;
    EXPECT_OK(KdaEngine::create(stream, sh, chunked, GemmPolicy{}, 256, 8, 4, &ec));
    EXPECT_OK(KdaEngine::create(stream, sh, chain, GemmPolicy{}, 256, 8, 4, &er));
    LayerOnDevice layer;
    make_layer(sh, 70, &layer);
    const std::vector<uint16_t> state0 = enc(values(slots * sh.layers * sh.state_elems(), 5, 0.05f));
    const std::vector<uint16_t> conv0 = enc(values(slots * sh.layers * sh.conv_elems(), 6, 1.0f));
    Pool pc, pr;
    make_pool(sh, slots, state0, conv0, &pc);
    make_pool(sh, slots, state0, conv0, &pr);
    const std::vector<uint16_t> x = enc(values(rows * sh.hidden, 80, 1.0f));
    std::vector<uint16_t> oc, orr, sc, sr, cc, cr;
    EXPECT_OK(ec.upload_meta(reqs)); EXPECT_OK(er.upload_meta(reqs));
    EXPECT_OK(ec.s.normed.upload(x)); EXPECT_OK(er.s.normed.upload(x));
    EXPECT_OK(ec.kda_layer(1, Mode::Prefill, rows, 0, layer.w, pc.view, stream));
    EXPECT_OK(er.kda_layer(1, Mode::Prefill, rows, 0, layer.w, pr.view, stream));
    EXPECT_OK(stream.synchronize());
    EXPECT_OK(ec.s.attn_out.download<uint16_t>(rows * sh.hidden, &oc)); EXPECT_OK(er.s.attn_out.download<uint16_t>(rows * sh.hidden, &orr));
    EXPECT_OK(pc.state.to_vec(&sc)); EXPECT_OK(pr.state.to_vec(&sr));
    EXPECT_OK(pc.conv.to_vec(&cc)); EXPECT_OK(pr.conv.to_vec(&cr));
    const double es = rel_err(dec(sc), dec(sr)), eo = rel_err(dec(oc), dec(orr));
    std::printf("prefill pass, chunked against chain: bf16 states %.2e, attention outputs %.2e (max-abs over max)\n", es, eo);
    EXPECT(es <= 1.0 / 128.0);    // bf16 states rounded after every chunk against after every row
    EXPECT(eo <= 1.0 / 64.0);
    EXPECT(cc == cr);             // the windows hold input rows: exact
    EXPECT(sc != state0);
    // layer 0 of every slot and the slot outside the batch are untouched
    const size_t sn = sh.state_elems();
    EXPECT(std::memcmp(&sc[(1 * sh.layers) * sn], &state0[(1 * sh.layers) * sn], sh.layers * sn * 2) == 0);
    EXPECT(std::memcmp(&sc[(2 * sh.layers) * sn], &state0[(2 * sh.layers) * sn], sn * 2) == 0);
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
        verify_commit_equals_decode(false, false);
        verify_commit_equals_decode(true, true);
        prefill_chunked_against_chain();
    }
    std::printf("%s: %d failure(s)\n", mode.c_str(), failures);
    return failures == 0 ? 0 : 1;
}
