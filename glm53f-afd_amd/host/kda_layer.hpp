// A KDA layer's step and a verify round's commit as the reference's engine issues them, over this library's host
// layer: the C++ counterpart of `GlmForward::kda` (crates/glm53f-forward/src/forward.rs:3469-3767: the three
// projections into the engine's row packing, the core by mode, the output projection) and of the KDA part of
// `GlmForward::commit` (forward.rs:1936-2040: replay of every layer's saves and the conv shift over all layers),
// with the pool's arenas as kv.rs:10-12 lays them out (`[slots][kda layers][...]`: a layer's base is j elements-per-
// layer in, a slot's offset slot * layers * elements-per-layer).
//
// Packing (forward.rs:3486-3542, :3577): projection rows `p` of 3 width + heads columns with the beta logits behind
// q|k|v (b_off = 3 width); the gates' first projection into `fga` [rows][256], the second as a grouped GEMM over its
// two halves into `ag` [rows][2 width] (`a` = ag, `g` = ag + width, both with stride 2 width); the core's output rows
// `kda_out` [rows][width]; the attention output [rows][hidden]. A verify round keeps every layer's `p` rows and
// replay saves `[layers][verify rows][...]` for the commit.
//
// Two switches beyond the reference's call site, both off by default: `fused_decode_shift` issues a decode round's
// chain and conv window advance as one launch (glm53f_kda_chain_shift_batch[_bf16state]); `verify_checkpoints` (bf16
// states) lets a verify round write a checkpoint after every row, and the commit then selects instead of replaying
// (glm53f_kda_verify_batch_bf16state, glm53f_kda_select_batch_bf16state).
#ifndef GLM53F_FORWARD_HOST_KDA_LAYER_HPP
#define GLM53F_FORWARD_HOST_KDA_LAYER_HPP

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "gemm.hpp"
#include "kernel.hpp"

namespace glm53f_forward {

namespace kda = glm53f_kda;
using kda::Buf;
using kda::RowView;

#define GLM53F_FWD_TRY(expr)             \
    do {                                 \
        Error e_try_ = (expr);           \
        if (!e_try_) return e_try_;      \
    } while (0)

/// The sizes a KDA layer's buffers follow from (forward.rs: HIDDEN, KDA_HEADS, KDA_DIM, KDA_WIDTH, KDA_QKV,
/// KDA_P_COLS; the model's are 4096, 64, 128, 8192, 24,576, 24,640).
struct KdaShape {
    size_t hidden = 4096, heads = 64, layers = 34;
    size_t dim() const { return kda::DK; }
    size_t width() const { return heads * kda::DK; }
    size_t qkv() const { return 3 * width(); }
    size_t p_cols() const { return qkv() + heads; }
    size_t state_elems() const { return kda::state_len(heads); }            // per layer and slot
    size_t conv_elems() const { return kda::WINDOW * kda::channels(heads); }
};

/// One KDA layer's weights on the device (forward.rs `KdaW`, BF16 projections).
struct KdaW {
    Bf16Mat qkvb;      // [3 width + heads][hidden]
    Bf16Mat fga;       // [2 dim][hidden]
    Bf16Mat fgb;       // two groups [width][dim]
    Bf16Mat o;         // [hidden][width]
    kda::Weights core; // conv_w, a_log, dt_bias, o_norm
};

enum class Mode { Prefill, Decode, Verify };

/// One request of a pass (forward.rs `Req`): its slot and the rows it owns in the pass's row buffers.
struct Req {
    size_t slot = 0, rows = 0;
};

/// The pool's KDA arenas (kv.rs:10-12, :744-753).
struct KdaPool {
    Buf state, conv;
    bool state_bf16 = true;
    size_t slots = 0;
    kda::StateType state_type() const { return state_bf16 ? kda::StateType::Bf16 : kda::StateType::F32; }
};

/// The per-pass row buffers (forward.rs `Scratch`: normed, p, fga, ag, kda_out, attn_out), sized for `rows` rows.
struct KdaScratch {
    size_t rows = 0;
    DeviceBuffer normed, p, fga, ag, kda_out, attn_out;
    static Error create(const KdaShape& s, size_t rows, KdaScratch* out) {
        out->rows = rows;
        GLM53F_FWD_TRY(DeviceBuffer::zeroed(rows * s.hidden * 2, &out->normed));
        GLM53F_FWD_TRY(DeviceBuffer::zeroed(rows * s.p_cols() * 2, &out->p));
        GLM53F_FWD_TRY(DeviceBuffer::zeroed(rows * 2 * s.dim() * 2, &out->fga));
        GLM53F_FWD_TRY(DeviceBuffer::zeroed(rows * 2 * s.width() * 2, &out->ag));
        GLM53F_FWD_TRY(DeviceBuffer::zeroed(rows * s.width() * 2, &out->kda_out));
        return DeviceBuffer::zeroed(rows * s.hidden * 2, &out->attn_out);
    }
};

/// What a verify round keeps for the commit (forward.rs `VerifyBufs`): every layer's projection rows and replay
/// saves, `[layers][rows][...]`; with checkpoints, every layer's state after every row.
struct KdaVerify {
    size_t rows = 0;   // capacity: rows of one verify round
    DeviceBuffer p, k, v, g, b, ckpt;
    static Error create(const KdaShape& s, size_t rows, bool checkpoints, KdaVerify* out) {
        out->rows = rows;
        const size_t lr = s.layers * rows;
        GLM53F_FWD_TRY(DeviceBuffer::zeroed(lr * s.p_cols() * 2, &out->p));
        GLM53F_FWD_TRY(DeviceBuffer::zeroed(lr * s.width() * 4, &out->k));
        GLM53F_FWD_TRY(DeviceBuffer::zeroed(lr * s.width() * 2, &out->v));
        GLM53F_FWD_TRY(DeviceBuffer::zeroed(lr * s.width() * 4, &out->g));
        GLM53F_FWD_TRY(DeviceBuffer::zeroed(lr * s.heads * 4, &out->b));
        if (checkpoints) GLM53F_FWD_TRY(DeviceBuffer::zeroed(lr * s.state_elems() * 2, &out->ckpt));
        return Error::ok();
    }
};

struct KdaConfig {
    bool chunked_prefill = true;       // forward.rs `kda_chunked_prefill`
    size_t prefill_rows = 1024;        // `kda_prefill_rows`: rows of every request per pass of the chunked prefill
    size_t prefill_value_blocks = 0;   // `kda_prefill_value_blocks`
    bool fused_decode_shift = false;   // chain + conv window advance in one launch
    bool verify_checkpoints = false;   // a checkpoint per verify row; commit by selection
};

class KdaEngine {
  public:
    KdaShape shape;
    KdaConfig cfg;
    Gemm gemm;
    KdaScratch s;
    KdaVerify v;

    static Error create(const Stream& stream, const KdaShape& shape, const KdaConfig& cfg, const GemmPolicy& policy,
                        size_t max_rows, size_t verify_rows, size_t max_requests, KdaEngine* out) {
        out->shape = shape;
        out->cfg = cfg;
        GLM53F_FWD_TRY(Gemm::create(stream, policy, &out->gemm));
        GLM53F_FWD_TRY(KdaScratch::create(shape, max_rows, &out->s));
        GLM53F_FWD_TRY(KdaVerify::create(shape, verify_rows, cfg.verify_checkpoints, &out->v));
        GLM53F_FWD_TRY(kda::BatchMeta::create(max_requests, &out->meta_));
        out->max_requests_ = max_requests;
        return Error::ok();
    }

    /// The pass's batch metadata (forward.rs `upload_meta`, :2266-2336): cu_rows, keep, and every request's offsets
    /// into a layer's view of the arenas.
    Error upload_meta(const std::vector<Req>& reqs, const std::vector<size_t>& keep = {}) {
        std::vector<kda::Request> rq;
        for (const Req& r : reqs)
            rq.push_back({r.rows, r.slot * shape.layers * shape.conv_elems(), r.slot * shape.layers * shape.state_elems()});
        return meta_.set(rq, keep);
    }
    const kda::BatchMeta& meta() const { return meta_; }

    /// KDA layer j of a pass over `rows` rows (`s.normed` holds them): projections, core, output projection into
    /// `s.attn_out` (forward.rs:3469-3767). `base`: the first row of this pass inside the verify round's buffers.
    Error kda_layer(size_t j, Mode mode, size_t rows, size_t base, const KdaW& w, const KdaPool& pool, const Stream& st) {
        const KdaShape& sh = shape;
        if (j >= sh.layers) return Error::invalid("KDA layer " + std::to_string(j) + " of " + std::to_string(sh.layers));
        if (rows == 0 || rows > s.rows || rows != meta_.total_rows())
            return Error::invalid("a pass of " + std::to_string(rows) + " rows against metadata for " +
                                  std::to_string(meta_.total_rows()) + " and scratch for " + std::to_string(s.rows));
        const bool verify = mode == Mode::Verify;
        if (verify && base + rows > v.rows) return Error::invalid("verify rows beyond the verify buffers");
        // Projection rows: per layer for a verify round (the commit's conv shift reads them).
        const Buf pbuf = verify ? Buf(v.p) : Buf(s.p);
        const size_t p_first = verify ? (j * v.rows + base) * sh.p_cols() : 0;
        const uint16_t* x = s.normed.ptr<uint16_t>();
        GLM53F_FWD_TRY(gemm.bf16(x, sh.hidden, 0, w.qkvb, rows, pbuf.ptr<uint16_t>(p_first), sh.p_cols(), 0, false, st));
        GLM53F_FWD_TRY(gemm.bf16(x, sh.hidden, 0, w.fga, rows, s.fga.ptr<uint16_t>(), 2 * sh.dim(), 0, false, st));
        GLM53F_FWD_TRY(gemm.bf16(s.fga.ptr<uint16_t>(), 2 * sh.dim(), sh.dim(), w.fgb, rows, s.ag.ptr<uint16_t>(),
                                 2 * sh.width(), sh.width(), false, st));

        // The layer's view of the arenas: from its base to the arena's end.
        const size_t sn = sh.state_elems(), cn = sh.conv_elems(), es = kda::state_bytes(pool.state_type());
        const Buf state(pool.state.ptr<unsigned char>(j * sn * es), pool.state.bytes - j * sn * es);
        const Buf conv(pool.conv.ptr<unsigned char>(j * cn * 2), pool.conv.bytes - j * cn * 2);
        const RowView p(pbuf, p_first, sh.p_cols());
        const RowView a(Buf(s.ag), 0, 2 * sh.width()), g(Buf(s.ag), sh.width(), 2 * sh.width());
        const RowView out = RowView::dense(Buf(s.kda_out), sh.width());

        if (mode == Mode::Prefill && cfg.chunked_prefill && rows > 8) {
            // The chunked form: it advances the conv windows itself (forward.rs:3581-3663).
            const size_t per = std::max<size_t>(cfg.prefill_rows, 16), n = meta_.requests().size();
            if (ws_.heads != sh.heads || ws_.batch < n)   // (the reference sizes it with the engine: forward.rs:3585-3594)
                GLM53F_FWD_TRY(kda::PrefillWorkspace::create(sh.heads, std::max(n, max_requests_), per, &ws_));
            kda::PrefillBatch pf;
            pf.weights = &w.core; pf.p = p; pf.b_off = (int64_t)sh.qkv(); pf.a = a; pf.g = g;
            pf.conv = conv; pf.state = state; pf.state_out = kda::StateOut::in_place(); pf.out = out;
            pf.value_blocks = cfg.prefill_value_blocks; pf.workspace = &ws_;
            GLM53F_FWD_TRY(pf.launch_as(meta_, st, pool.state_type()));
            return kda_o(rows, w.o, st);
        }
        kda::Saves saves;
        if (verify) {
            const size_t r0 = j * v.rows + base, left = v.rows - base;
            saves = kda::Saves{sh.heads, left, Buf(v.k.ptr<float>(r0 * sh.width()), left * sh.width() * 4),
                               Buf(v.v.ptr<uint16_t>(r0 * sh.width()), left * sh.width() * 2),
                               Buf(v.g.ptr<float>(r0 * sh.width()), left * sh.width() * 4),
                               Buf(v.b.ptr<float>(r0 * sh.heads), left * sh.heads * 4)};
        }
        kda::ChainBatch ch;
        ch.weights = &w.core; ch.p = p; ch.b_off = (int64_t)sh.qkv(); ch.a = a; ch.g = g;
        ch.conv = conv; ch.state = state; ch.out = out;
        ch.state_out = verify ? kda::StateOut::skip() : kda::StateOut::in_place();
        ch.saves = verify ? &saves : nullptr;
        if (verify && cfg.verify_checkpoints) {
            if (!pool.state_bf16) return Error::invalid("checkpoints need bf16 states");
            const size_t r0 = j * v.rows + base;
            ch.ckpt = Buf(v.ckpt.ptr<uint16_t>(r0 * sn), (v.rows - base) * sn * 2);
        }
        ch.advance_conv = !verify && cfg.fused_decode_shift;
        GLM53F_FWD_TRY(ch.launch_as(meta_, st, pool.state_type()));
        if (!verify && !cfg.fused_decode_shift)    // keep = each request's rows (forward.rs:3741-3760)
            GLM53F_FWD_TRY(kda::conv_shift_batch(sh.heads, 1, meta_, conv, 0, RowView(pbuf, p_first, sh.p_cols()), 0, st));
        return kda_o(rows, w.o, st);
    }

    /// KDA's o_proj of the gated norm's output into the attention output (forward.rs:3769-3789, BF16).
    Error kda_o(size_t rows, const Bf16Mat& o, const Stream& st) {
        return gemm.bf16(s.kda_out.ptr<uint16_t>(), shape.width(), 0, o, rows, s.attn_out.ptr<uint16_t>(), shape.hidden, 0,
                         false, st);
    }

    /// The KDA part of the commit of a verify round of `rows` rows (forward.rs:1968-2040): request i keeps its first
    /// keep[i] rows; every layer's states move on by replay (or by selection among the checkpoints) and every
    /// layer's conv windows by the kept rows, two launches for all layers.
    Error commit(const std::vector<Req>& reqs, const std::vector<size_t>& keep, const KdaPool& pool, const Stream& st) {
        if (keep.size() != reqs.size()) return Error::invalid("commit: one keep per request");
        for (size_t i = 0; i < reqs.size(); ++i)
            if (keep[i] == 0 || keep[i] > reqs[i].rows)
                return Error::invalid("commit of " + std::to_string(keep[i]) + " rows does not match the pending verify of slot " +
                                      std::to_string(reqs[i].slot));
        GLM53F_FWD_TRY(upload_meta(reqs, keep));
        const KdaShape& sh = shape;
        const size_t sn = sh.state_elems(), cn = sh.conv_elems(), es = kda::state_bytes(pool.state_type());
        if (meta_.total_rows() > v.rows) return Error::invalid("commit of more rows than the verify buffers hold");
        for (const Req& r : reqs)
            if (r.slot >= pool.slots || (r.slot + 1) * sh.layers * sn * es > pool.state.bytes ||
                (r.slot + 1) * sh.layers * cn * 2 > pool.conv.bytes)
                return Error::invalid("commit: slot " + std::to_string(r.slot) + " outside the pool");
        // The launches go to the C ABI as the reference's engine sends them (forward.rs:1980-2040): the checked
        // wrappers' rule for several layers (a layer's stride beyond every request's offset, kernel.rs:849-861)
        // does not hold in the arenas, where a layer's slots lie `layers` states apart and the layers interleave.
        int32_t h32, l32, n32, c32;
        GLM53F_FWD_TRY(kda::to_i32(sh.heads, "heads", &h32));
        GLM53F_FWD_TRY(kda::to_i32(sh.layers, "layers", &l32));
        GLM53F_FWD_TRY(kda::to_i32(kda::channels(sh.heads), "channels", &c32));
        GLM53F_FWD_TRY(meta_.batch(&n32));
        glm53f_stream_t raw = reinterpret_cast<glm53f_stream_t>(st.raw());
        if (cfg.verify_checkpoints) {
            if (!pool.state_bf16) return Error::invalid("checkpoints need bf16 states");
            GLM53F_FWD_TRY(kda::launched(
                glm53f_kda_select_batch_bf16state(h32, l32, n32, meta_.cu_rows(), meta_.keep_dev(), v.ckpt.ptr<glm53f_bf16>(),
                                                  (int64_t)(v.rows * sn), pool.state.ptr<glm53f_bf16>(), (int64_t)sn,
                                                  meta_.state_off(), raw),
                "glm53f_kda_select_batch_bf16state"));
        } else if (pool.state_bf16) {
            GLM53F_FWD_TRY(kda::launched(
                glm53f_kda_replay_batch_bf16state(h32, l32, n32, meta_.cu_rows(), meta_.keep_dev(), pool.state.ptr<glm53f_bf16>(),
                                                  pool.state.ptr<glm53f_bf16>(), (int64_t)sn, meta_.state_off(), v.k.ptr<float>(),
                                                  v.v.ptr<glm53f_bf16>(), v.g.ptr<float>(), v.b.ptr<float>(),
                                                  (int64_t)(v.rows * sh.width()), (int64_t)(v.rows * sh.heads), raw),
                "glm53f_kda_replay_batch_bf16state"));
        } else {
            GLM53F_FWD_TRY(kda::launched(
                glm53f_kda_replay_batch(h32, l32, n32, meta_.cu_rows(), meta_.keep_dev(), pool.state.ptr<float>(),
                                        pool.state.ptr<float>(), (int64_t)sn, meta_.state_off(), v.k.ptr<float>(),
                                        v.v.ptr<glm53f_bf16>(), v.g.ptr<float>(), v.b.ptr<float>(),
                                        (int64_t)(v.rows * sh.width()), (int64_t)(v.rows * sh.heads), raw),
                "glm53f_kda_replay_batch"));
        }
        return kda::launched(glm53f_kda_conv_shift_batch(c32, l32, n32, meta_.cu_rows(), meta_.keep_dev(),
                                                         pool.conv.ptr<glm53f_bf16>(), (int64_t)cn, meta_.conv_off(),
                                                         v.p.ptr<glm53f_bf16>(), (int64_t)(v.rows * sh.p_cols()),
                                                         (int64_t)sh.p_cols(), raw),
                             "glm53f_kda_conv_shift_batch");
    }

  private:
    kda::BatchMeta meta_{0};
    kda::PrefillWorkspace ws_;
    size_t max_requests_ = 0;
};

}  // namespace glm53f_forward

#endif  // GLM53F_FORWARD_HOST_KDA_LAYER_HPP
