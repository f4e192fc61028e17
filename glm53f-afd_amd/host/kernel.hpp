// Checked wrappers over the KDA kernels' C ABI: the C++ counterpart of the reference's
// crates/glm53f-kda/src/kernel.rs:14-1285, with its names, argument meaning and error behaviour. Every launch
// first checks on the host that each buffer is large enough for the geometry it is given, that written regions do
// not overlap and that the batch metadata is consistent, then makes one call into include/glm53f_kda.h. Launches
// are asynchronous; buffers must outlive the stream's work. Batch metadata is copied to the device
// synchronously when it is set.
//
// The wrappers take `Buf` views (address + size) of device memory; a DeviceBuffer converts to one. Every
// wrapper has check(), which validates and never touches the GPU, and launch(), which is check() followed by the
// C call: the argument checks are testable on a machine without a GPU.
#ifndef GLM53F_KDA_HOST_KERNEL_HPP
#define GLM53F_KDA_HOST_KERNEL_HPP

#include <algorithm>
#include <cstdint>
#include <limits>
#include <string>
#include <vector>

#include "device.hpp"
#include "glm53f_kda.h"

namespace glm53f_kda {

constexpr size_t DK = 128, DV = 128, TAPS = 4, WINDOW = TAPS - 1;
constexpr size_t HEADS = 64, LAYERS = 34;
constexpr float LOWER_BOUND = -5.0f, RMS_EPS = 1e-5f;
/// The gate lower bounds the prefill accepts (kernel.rs:975-986).
constexpr float PREFILL_LOWER_MIN = -5.8f;
/// Rows per chunk of this build's prefill (the reference's kernel uses 16).
constexpr size_t PREFILL_CHUNK = GLM53F_KDA_PREFILL_CHUNK;

inline size_t channels(size_t heads) { return 3 * heads * DK; }
inline size_t state_len(size_t heads) { return heads * DV * DK; }

/// A view of device memory: address and size in bytes.
struct Buf {
    void* p = nullptr;
    size_t bytes = 0;
    Buf() = default;
    Buf(void* p_, size_t b) : p(p_), bytes(b) {}
    Buf(const DeviceBuffer& d) : p(const_cast<void*>(d.as_ptr())), bytes(d.bytes()) {}
    template <typename T>
    T* ptr(size_t offset = 0) const { return reinterpret_cast<T*>(p) + offset; }
};

inline bool same(const Buf& a, const Buf& b) { return a.p == b.p && a.bytes > 0; }
/// Regions [a, a + n) and [b, b + n) either coincide or are disjoint (kernel.rs:217-220).
inline bool coincide_or_disjoint(size_t a, size_t b, size_t n) { return a == b || a + n <= b || b + n <= a; }

inline Error check_region(const char* what, const Buf& buf, size_t size, size_t offset, size_t n) {
    const size_t len = buf.bytes / size;
    if (offset > len || n > len - offset)
        return Error::invalid(std::string(what) + ": elements [" + std::to_string(offset) + ", " + std::to_string(offset) +
                              " + " + std::to_string(n) + ") exceed a buffer of " + std::to_string(len));
    return Error::ok();
}

inline Error to_i32(size_t x, const char* what, int32_t* out) {
    if (x > (size_t)std::numeric_limits<int32_t>::max())
        return Error::invalid(std::string(what) + " = " + std::to_string(x) + " does not fit in 32 bits");
    *out = (int32_t)x;
    return Error::ok();
}

inline Error launched(int code, const char* what) {
    if (code == 0) return Error::ok();
    if (code == 1) return Error::invalid(std::string(what) + ": rejected by the launcher");
    return Error::hip(code, what);
}

#define KDA_TRY(expr)                 \
    do {                              \
        ::glm53f_kda::Error e_ = (expr); \
        if (!e_) return e_;           \
    } while (0)

/// Rows in a device buffer: row r starts at element offset + r * stride (kernel.rs:54-105).
struct RowView {
    Buf buf;
    size_t offset = 0;
    size_t stride = 0;
    RowView() = default;
    RowView(Buf b, size_t off, size_t st) : buf(b), offset(off), stride(st) {}
    static RowView dense(Buf b, size_t width) { return RowView(b, 0, width); }

    /// Rows first .. first + rows have columns [lo, hi) inside the buffer (elements of `size` bytes).
    Error check(const char* what, size_t size, size_t first, size_t rows, int64_t lo, int64_t hi) const {
        if (rows == 0) return Error::ok();
        const __int128 len = (__int128)(buf.bytes / size);
        const __int128 start = (__int128)offset + (__int128)first * stride;
        const __int128 mn = start + lo;
        const __int128 mx = start + (__int128)(rows - 1) * stride + hi;
        if (mn < 0 || mx > len)
            return Error::invalid(std::string(what) + ": rows reach outside a buffer of " + std::to_string((long long)len) +
                                  " elements");
        return Error::ok();
    }
};

/// One layer's weights on the device (kernel.rs:14-52).
struct Weights {
    size_t heads = 0;
    Buf conv_w;   // bf16 [C][TAPS]
    Buf a_log;    // f32 [H]
    Buf dt_bias;  // f32 [H * DK]
    Buf norm_w;   // bf16 [DV]
    float eps = RMS_EPS;
    float lower = LOWER_BOUND;

    Error check() const {
        if (heads < 1 || conv_w.bytes < channels(heads) * TAPS * 2 || a_log.bytes < heads * 4 ||
            dt_bias.bytes < heads * DK * 4 || norm_w.bytes < DV * 2)
            return Error::invalid("layer parameters have the wrong sizes");
        return Error::ok();
    }
};

/// Per-row replay inputs for up to `rows` rows of `heads` heads, one layer (kernel.rs:137-179).
struct Saves {
    size_t heads = 0, rows = 0;
    Buf k;  // f32 [rows][H][DK]
    Buf v;  // bf16 [rows][H][DV]
    Buf g;  // f32 [rows][H][DK]
    Buf b;  // f32 [rows][H]
    Error check(size_t h, size_t need_rows) const {
        if (heads != h || rows < need_rows || k.bytes < rows * heads * DK * 4 || v.bytes < rows * heads * DV * 2 ||
            g.bytes < rows * heads * DK * 4 || b.bytes < rows * heads * 4)
            return Error::invalid("saves hold " + std::to_string(rows) + " rows of " + std::to_string(heads) + " heads");
        return Error::ok();
    }
};

/// Device storage behind a Saves (kernel.rs `Saves::alloc`).
struct SavesStorage {
    DeviceBuffer k, v, g, b;
    Saves view;
    static Error alloc(size_t heads, size_t rows, SavesStorage* out) {
        KDA_TRY(DeviceBuffer::zeroed(rows * heads * DK * 4, &out->k));
        KDA_TRY(DeviceBuffer::zeroed(rows * heads * DV * 2, &out->v));
        KDA_TRY(DeviceBuffer::zeroed(rows * heads * DK * 4, &out->g));
        KDA_TRY(DeviceBuffer::zeroed(rows * heads * 4, &out->b));
        out->view = Saves{heads, rows, out->k, out->v, out->g, out->b};
        return Error::ok();
    }
};

/// Where a chain writes the state after its last row (kernel.rs:181-190).
struct StateOut {
    enum Kind { Skip, InPlace, To };
    Kind kind = InPlace;
    Buf buf;
    size_t offset = 0;
    static StateOut skip() { return {Skip, Buf(), 0}; }
    static StateOut in_place() { return {InPlace, Buf(), 0}; }
    static StateOut to(Buf b, size_t off = 0) { return {To, b, off}; }
};

/// How a batch launch's states are stored (kernel.rs:192-211).
enum class StateType { F32, Bf16 };
inline size_t state_bytes(StateType t) { return t == StateType::F32 ? 4 : 2; }

/// One layer, one request: `rows` rows from the committed state (glm53f_kda_chain; kernel.rs:222-326).
struct Chain {
    const Weights* weights = nullptr;
    size_t rows = 0;
    RowView p;
    int64_t b_off = 0;
    RowView a, g;
    Buf conv;
    size_t conv_offset = 0;
    Buf state;
    size_t state_offset = 0;
    StateOut state_out;
    RowView out;
    const Saves* saves = nullptr;

    Error check(float** state_out_ptr) const {
        KDA_TRY(weights->check());
        const size_t h = weights->heads;
        if (rows == 0) return Error::invalid("a chain needs at least one row");
        const int64_t c = (int64_t)channels(h);
        const int64_t lo = std::min<int64_t>(b_off, 0), hi = std::max<int64_t>(c, b_off + (int64_t)h);
        KDA_TRY(p.check("p", 2, 0, rows, lo, hi));
        KDA_TRY(a.check("a", 2, 0, rows, 0, (int64_t)(h * DK)));
        KDA_TRY(g.check("g", 2, 0, rows, 0, (int64_t)(h * DV)));
        KDA_TRY(out.check("out", 2, 0, rows, 0, (int64_t)(h * DV)));
        if (rows > 1 && out.stride < h * DV) return Error::invalid("out rows overlap");
        KDA_TRY(check_region("conv", conv, 2, conv_offset, WINDOW * channels(h)));
        KDA_TRY(check_region("state", state, 4, state_offset, state_len(h)));
        *state_out_ptr = nullptr;
        if (state_out.kind == StateOut::InPlace) {
            *state_out_ptr = state.ptr<float>(state_offset);
        } else if (state_out.kind == StateOut::To) {
            KDA_TRY(check_region("state_out", state_out.buf, 4, state_out.offset, state_len(h)));
            if (same(state_out.buf, state) && !coincide_or_disjoint(state_out.offset, state_offset, state_len(h)))
                return Error::invalid("state_out partly overlaps the state");
            *state_out_ptr = state_out.buf.ptr<float>(state_out.offset);
        }
        if (saves != nullptr) KDA_TRY(saves->check(h, rows));
        return Error::ok();
    }

    Error launch(const Stream& stream) const {
        float* so = nullptr;
        KDA_TRY(check(&so));
        const Weights& w = *weights;
        int32_t h32, r32;
        KDA_TRY(to_i32(w.heads, "heads", &h32));
        KDA_TRY(to_i32(rows, "rows", &r32));
        const int code = glm53f_kda_chain(
            h32, r32, p.buf.ptr<glm53f_bf16>(p.offset), (int64_t)p.stride, b_off, a.buf.ptr<glm53f_bf16>(a.offset),
            (int64_t)a.stride, g.buf.ptr<glm53f_bf16>(g.offset), (int64_t)g.stride, conv.ptr<glm53f_bf16>(conv_offset),
            w.conv_w.ptr<glm53f_bf16>(), state.ptr<float>(state_offset), so, w.a_log.ptr<float>(),
            w.dt_bias.ptr<float>(), w.norm_w.ptr<glm53f_bf16>(), w.eps, w.lower, out.buf.ptr<glm53f_bf16>(out.offset),
            (int64_t)out.stride, saves ? saves->k.ptr<float>() : nullptr, saves ? saves->v.ptr<glm53f_bf16>() : nullptr,
            saves ? saves->g.ptr<float>() : nullptr, saves ? saves->b.ptr<float>() : nullptr,
            reinterpret_cast<glm53f_stream_t>(stream.raw()));
        return launched(code, "glm53f_kda_chain");
    }
};

/// The state after the first `rows` saved rows (glm53f_kda_replay; kernel.rs:328-365).
inline Error replay(size_t heads, size_t rows, Buf state, size_t state_off, Buf state_out, size_t state_out_off,
                    const Saves& saves, const Stream& stream, bool dry_run = false) {
    KDA_TRY(check_region("state", state, 4, state_off, state_len(heads)));
    KDA_TRY(check_region("state_out", state_out, 4, state_out_off, state_len(heads)));
    if (same(state, state_out) && !coincide_or_disjoint(state_off, state_out_off, state_len(heads)))
        return Error::invalid("state_out partly overlaps the state");
    KDA_TRY(saves.check(heads, rows));
    if (dry_run) return Error::ok();
    int32_t h32, r32;
    KDA_TRY(to_i32(heads, "heads", &h32));
    KDA_TRY(to_i32(rows, "rows", &r32));
    return launched(glm53f_kda_replay(h32, r32, state.ptr<float>(state_off), state_out.ptr<float>(state_out_off),
                                      saves.k.ptr<float>(), saves.v.ptr<glm53f_bf16>(), saves.g.ptr<float>(),
                                      saves.b.ptr<float>(), reinterpret_cast<glm53f_stream_t>(stream.raw())),
                    "glm53f_kda_replay");
}

/// Advance one conv window past `keep` kept rows of p, in place (glm53f_kda_conv_shift; kernel.rs:367-394).
inline Error conv_shift(size_t heads, size_t keep, Buf conv, size_t conv_offset, const RowView& p, const Stream& stream,
                        bool dry_run = false) {
    const size_t c = channels(heads);
    KDA_TRY(check_region("conv", conv, 2, conv_offset, WINDOW * c));
    const size_t first = keep > WINDOW ? keep - WINDOW : 0;   // the shift reads new rows first .. keep
    KDA_TRY(p.check("p", 2, first, keep - first, 0, (int64_t)c));
    if (dry_run) return Error::ok();
    int32_t c32, k32;
    KDA_TRY(to_i32(c, "channels", &c32));
    KDA_TRY(to_i32(keep, "keep", &k32));
    return launched(glm53f_kda_conv_shift(c32, k32, conv.ptr<glm53f_bf16>(conv_offset), p.buf.ptr<glm53f_bf16>(p.offset),
                                          (int64_t)p.stride, reinterpret_cast<glm53f_stream_t>(stream.raw())),
                    "glm53f_kda_conv_shift");
}

/// One request of a batch (kernel.rs:396-405).
struct Request {
    size_t rows = 0;         // it owns the next `rows` rows of the shared row buffers
    size_t conv_offset = 0;  // element offset of its conv window (per layer)
    size_t state_offset = 0; // element offset of its state (per layer)
};

/// Batch metadata on the device, with a host copy for the checks (kernel.rs:407-526).
class BatchMeta {
  public:
    /// Host-only metadata (no device arrays): enough for check(), not for launch().
    explicit BatchMeta(size_t capacity) : capacity_(capacity) {}
    static Error create(size_t capacity, BatchMeta* out) {
        out->capacity_ = capacity;
        KDA_TRY(DeviceBuffer::zeroed((capacity + 1) * 4, &out->cu_rows_));
        KDA_TRY(DeviceBuffer::zeroed(capacity * 4, &out->keep_));
        KDA_TRY(DeviceBuffer::zeroed(capacity * 8, &out->conv_off_));
        KDA_TRY(DeviceBuffer::zeroed(capacity * 8, &out->state_off_));
        out->on_device_ = true;
        return Error::ok();
    }

    /// Set the requests and, for replays and conv shifts, the rows each keeps (empty: all). Copies to the device
    /// synchronously.
    Error set(const std::vector<Request>& requests, const std::vector<size_t>& keep = {}) {
        if (requests.empty() || requests.size() > capacity_)
            return Error::invalid(std::to_string(requests.size()) + " requests for a capacity of " + std::to_string(capacity_));
        std::vector<size_t> kp = keep;
        if (kp.empty()) {
            for (const Request& r : requests) kp.push_back(r.rows);
        } else if (kp.size() != requests.size()) {
            return Error::invalid("one keep per request");
        }
        for (size_t i = 0; i < requests.size(); ++i)
            if (kp[i] > requests[i].rows)
                return Error::invalid("keep " + std::to_string(kp[i]) + " exceeds the request's " +
                                      std::to_string(requests[i].rows) + " rows");
        std::vector<int32_t> cu(requests.size() + 1, 0), keep32(requests.size());
        std::vector<int64_t> conv(requests.size()), state(requests.size());
        for (size_t i = 0; i < requests.size(); ++i) {
            int32_t r32;
            KDA_TRY(to_i32(requests[i].rows, "rows", &r32));
            const int64_t sum = (int64_t)cu[i] + r32;
            if (sum > std::numeric_limits<int32_t>::max()) return Error::invalid("total rows do not fit in 32 bits");
            cu[i + 1] = (int32_t)sum;
            KDA_TRY(to_i32(kp[i], "keep", &keep32[i]));
            conv[i] = (int64_t)requests[i].conv_offset;
            state[i] = (int64_t)requests[i].state_offset;
        }
        if (on_device_) {
            KDA_TRY(cu_rows_.upload(cu));
            KDA_TRY(keep_.upload(keep32));
            KDA_TRY(conv_off_.upload(conv));
            KDA_TRY(state_off_.upload(state));
        }
        requests_ = requests;
        keep_host_ = kp;
        return Error::ok();
    }

    const std::vector<Request>& requests() const { return requests_; }
    const std::vector<size_t>& keep() const { return keep_host_; }
    size_t total_rows() const {
        size_t n = 0;
        for (const Request& r : requests_) n += r.rows;
        return n;
    }
    size_t max_rows() const {
        size_t n = 0;
        for (const Request& r : requests_) n = std::max(n, r.rows);
        return n;
    }
    Error batch(int32_t* out) const {
        if (requests_.empty()) return Error::invalid("batch metadata not set");
        return to_i32(requests_.size(), "batch", out);
    }
    const int32_t* cu_rows() const { return cu_rows_.ptr<int32_t>(); }
    const int32_t* keep_dev() const { return keep_.ptr<int32_t>(); }
    const int64_t* conv_off() const { return conv_off_.ptr<int64_t>(); }
    const int64_t* state_off() const { return state_off_.ptr<int64_t>(); }
    bool on_device() const { return on_device_; }

    /// Each request's region of n elements at base + offset(r) inside the buffer, pairwise disjoint when asked.
    template <typename F>
    Error check_regions(const char* what, const Buf& buf, size_t size, size_t base, size_t n, bool disjoint, F offset) const {
        std::vector<size_t> spans;
        for (const Request& r : requests_) {
            KDA_TRY(check_region(what, buf, size, base + offset(r), n));
            spans.push_back(offset(r));
        }
        if (disjoint) {
            std::sort(spans.begin(), spans.end());
            for (size_t i = 1; i < spans.size(); ++i)
                if (spans[i] < spans[i - 1] + n) return Error::invalid(std::string(what) + ": requests' regions overlap");
        }
        return Error::ok();
    }

  private:
    size_t capacity_ = 0;
    bool on_device_ = false;
    std::vector<Request> requests_;
    std::vector<size_t> keep_host_;
    DeviceBuffer cu_rows_, keep_, conv_off_, state_off_;
};

/// One layer, a batch of requests (glm53f_kda_chain_batch[_bf16state]; kernel.rs:528-679). With `ckpt` set and
/// bf16 states it is the checkpointing verify step (glm53f_kda_verify_batch_bf16state), which never writes the
/// pool. With `advance_conv` the same launch moves every request's conv window past all its rows
/// (glm53f_kda_chain_shift_batch[_bf16state]: what conv_shift_batch with keep = rows would do next); the windows are
/// written then and must not overlap.
struct ChainBatch {
    const Weights* weights = nullptr;
    RowView p;
    int64_t b_off = 0;
    RowView a, g;
    Buf conv;    // conv windows, at each request's conv_offset
    Buf state;   // states, at each request's state_offset
    StateOut state_out;   // To(buf, _) writes at each request's state_offset in buf
    RowView out;
    const Saves* saves = nullptr;
    Buf ckpt;    // bf16 [total rows][H][128][128], or empty
    bool advance_conv = false;

    Error check(const BatchMeta& meta, StateType st, void** state_out_ptr) const {
        KDA_TRY(weights->check());
        const size_t es = state_bytes(st), h = weights->heads;
        int32_t batch;
        KDA_TRY(meta.batch(&batch));
        const size_t total = meta.total_rows();
        const int64_t c = (int64_t)channels(h);
        const int64_t lo = std::min<int64_t>(b_off, 0), hi = std::max<int64_t>(c, b_off + (int64_t)h);
        KDA_TRY(p.check("p", 2, 0, total, lo, hi));
        KDA_TRY(a.check("a", 2, 0, total, 0, (int64_t)(h * DK)));
        KDA_TRY(g.check("g", 2, 0, total, 0, (int64_t)(h * DV)));
        KDA_TRY(out.check("out", 2, 0, total, 0, (int64_t)(h * DV)));
        if (total > 1 && out.stride < h * DV) return Error::invalid("out rows overlap");
        KDA_TRY(meta.check_regions("conv", conv, 2, 0, WINDOW * channels(h), advance_conv, [](const Request& r) { return r.conv_offset; }));
        KDA_TRY(meta.check_regions("state", state, es, 0, state_len(h), true, [](const Request& r) { return r.state_offset; }));
        *state_out_ptr = nullptr;
        if (advance_conv && ckpt.p != nullptr) return Error::invalid("a verify round's windows wait for the commit");
        if (ckpt.p != nullptr) {
            if (st != StateType::Bf16) return Error::invalid("checkpoints need bf16 states");
            if (state_out.kind != StateOut::Skip) return Error::invalid("a checkpointing verify does not write the pool");
            KDA_TRY(check_region("ckpt", ckpt, 2, 0, total * state_len(h)));
        } else if (state_out.kind == StateOut::InPlace) {
            *state_out_ptr = state.p;
        } else if (state_out.kind == StateOut::To) {
            KDA_TRY(meta.check_regions("state_out", state_out.buf, es, 0, state_len(h), true,
                                       [](const Request& r) { return r.state_offset; }));
            if (same(state_out.buf, state)) return Error::invalid("state_out is the state buffer: use InPlace");
            *state_out_ptr = state_out.buf.p;
        }
        if (saves != nullptr) KDA_TRY(saves->check(h, total));
        return Error::ok();
    }

    Error launch(const BatchMeta& meta, const Stream& stream) const { return launch_as(meta, stream, StateType::F32); }
    Error launch_bf16_state(const BatchMeta& meta, const Stream& stream) const { return launch_as(meta, stream, StateType::Bf16); }

    Error launch_as(const BatchMeta& meta, const Stream& stream, StateType st) const {
        void* so = nullptr;
        KDA_TRY(check(meta, st, &so));
        if (!meta.on_device()) return Error::invalid("batch metadata has no device arrays");
        const Weights& w = *weights;
        int32_t h32, batch;
        KDA_TRY(to_i32(w.heads, "heads", &h32));
        KDA_TRY(meta.batch(&batch));
        const glm53f_bf16* pp = p.buf.ptr<glm53f_bf16>(p.offset);
        const glm53f_bf16* ap = a.buf.ptr<glm53f_bf16>(a.offset);
        const glm53f_bf16* gp = g.buf.ptr<glm53f_bf16>(g.offset);
        glm53f_bf16* op = out.buf.ptr<glm53f_bf16>(out.offset);
        float* ks = saves ? saves->k.ptr<float>() : nullptr;
        glm53f_bf16* vs = saves ? saves->v.ptr<glm53f_bf16>() : nullptr;
        float* gs = saves ? saves->g.ptr<float>() : nullptr;
        float* bs = saves ? saves->b.ptr<float>() : nullptr;
        glm53f_stream_t s = reinterpret_cast<glm53f_stream_t>(stream.raw());
        int code;
        if (ckpt.p != nullptr) {
            code = glm53f_kda_verify_batch_bf16state(
                h32, batch, meta.cu_rows(), pp, (int64_t)p.stride, b_off, ap, (int64_t)a.stride, gp, (int64_t)g.stride,
                conv.ptr<glm53f_bf16>(), meta.conv_off(), w.conv_w.ptr<glm53f_bf16>(), state.ptr<glm53f_bf16>(),
                meta.state_off(), w.a_log.ptr<float>(), w.dt_bias.ptr<float>(), w.norm_w.ptr<glm53f_bf16>(), w.eps,
                w.lower, op, (int64_t)out.stride, ckpt.ptr<glm53f_bf16>(), ks, vs, gs, bs, s);
            return launched(code, "glm53f_kda_verify_batch_bf16state");
        }
        if (advance_conv) {
            if (st == StateType::F32)
                code = glm53f_kda_chain_shift_batch(
                    h32, batch, meta.cu_rows(), pp, (int64_t)p.stride, b_off, ap, (int64_t)a.stride, gp, (int64_t)g.stride,
                    conv.ptr<glm53f_bf16>(), meta.conv_off(), w.conv_w.ptr<glm53f_bf16>(), state.ptr<float>(),
                    reinterpret_cast<float*>(so), meta.state_off(), w.a_log.ptr<float>(), w.dt_bias.ptr<float>(),
                    w.norm_w.ptr<glm53f_bf16>(), w.eps, w.lower, op, (int64_t)out.stride, ks, vs, gs, bs, s);
            else
                code = glm53f_kda_chain_shift_batch_bf16state(
                    h32, batch, meta.cu_rows(), pp, (int64_t)p.stride, b_off, ap, (int64_t)a.stride, gp, (int64_t)g.stride,
                    conv.ptr<glm53f_bf16>(), meta.conv_off(), w.conv_w.ptr<glm53f_bf16>(), state.ptr<glm53f_bf16>(),
                    reinterpret_cast<glm53f_bf16*>(so), meta.state_off(), w.a_log.ptr<float>(), w.dt_bias.ptr<float>(),
                    w.norm_w.ptr<glm53f_bf16>(), w.eps, w.lower, op, (int64_t)out.stride, ks, vs, gs, bs, s);
            return launched(code, "glm53f_kda_chain_shift_batch");
        }
        if (st == StateType::F32)
            code = glm53f_kda_chain_batch(h32, batch, meta.cu_rows(), pp, (int64_t)p.stride, b_off, ap, (int64_t)a.stride, gp,
                                          (int64_t)g.stride, conv.ptr<glm53f_bf16>(), meta.conv_off(),
                                          w.conv_w.ptr<glm53f_bf16>(), state.ptr<float>(), reinterpret_cast<float*>(so),
                                          meta.state_off(), w.a_log.ptr<float>(), w.dt_bias.ptr<float>(),
                                          w.norm_w.ptr<glm53f_bf16>(), w.eps, w.lower, op, (int64_t)out.stride, ks, vs, gs,
                                          bs, s);
        else
            code = glm53f_kda_chain_batch_bf16state(
                h32, batch, meta.cu_rows(), pp, (int64_t)p.stride, b_off, ap, (int64_t)a.stride, gp, (int64_t)g.stride,
                conv.ptr<glm53f_bf16>(), meta.conv_off(), w.conv_w.ptr<glm53f_bf16>(), state.ptr<glm53f_bf16>(),
                reinterpret_cast<glm53f_bf16*>(so), meta.state_off(), w.a_log.ptr<float>(), w.dt_bias.ptr<float>(),
                w.norm_w.ptr<glm53f_bf16>(), w.eps, w.lower, op, (int64_t)out.stride, ks, vs, gs, bs, s);
        return launched(code, "glm53f_kda_chain_batch");
    }
};

/// Saves for several layers in one allocation each (kernel.rs:681-737).
struct LayerSaves {
    size_t layers = 0, heads = 0, rows = 0;
    Buf k, v, g, b;
    size_t kv_stride() const { return rows * heads * DK; }
    size_t b_stride() const { return rows * heads; }
    Error check() const {
        if (k.bytes < layers * kv_stride() * 4 || v.bytes < layers * kv_stride() * 2 || g.bytes < layers * kv_stride() * 4 ||
            b.bytes < layers * b_stride() * 4)
            return Error::invalid("layer saves are smaller than layers x rows x heads");
        return Error::ok();
    }
};

/// Replay every layer of one request (glm53f_kda_replay_layers; kernel.rs:739-777).
inline Error replay_layers(size_t rows, Buf state, Buf state_out, size_t state_stride, const LayerSaves& saves,
                           const Stream& stream, bool dry_run = false) {
    const size_t h = saves.heads, l = saves.layers;
    if (l == 0 || rows > saves.rows || state_stride < state_len(h))
        return Error::invalid("replay_layers: no layers, rows beyond the saves, or overlapping layers");
    KDA_TRY(saves.check());
    KDA_TRY(check_region("state", state, 4, (l - 1) * state_stride, state_len(h)));
    KDA_TRY(check_region("state", state_out, 4, (l - 1) * state_stride, state_len(h)));
    if (dry_run) return Error::ok();
    int32_t h32, l32, r32;
    KDA_TRY(to_i32(h, "heads", &h32));
    KDA_TRY(to_i32(l, "layers", &l32));
    KDA_TRY(to_i32(rows, "rows", &r32));
    return launched(glm53f_kda_replay_layers(h32, l32, r32, state.ptr<float>(), state_out.ptr<float>(), (int64_t)state_stride,
                                             saves.k.ptr<float>(), saves.v.ptr<glm53f_bf16>(), saves.g.ptr<float>(),
                                             saves.b.ptr<float>(), (int64_t)saves.kv_stride(), (int64_t)saves.b_stride(),
                                             reinterpret_cast<glm53f_stream_t>(stream.raw())),
                    "glm53f_kda_replay_layers");
}

/// Replay every layer of every request of a batch (glm53f_kda_replay_batch[_bf16state]; kernel.rs:779-905).
inline Error replay_batch_as(const BatchMeta& meta, Buf state, Buf state_out, size_t state_stride, const LayerSaves& saves,
                             const Stream& stream, StateType st, bool dry_run = false) {
    const size_t h = saves.heads, l = saves.layers;
    int32_t batch;
    KDA_TRY(meta.batch(&batch));
    if (l == 0 || meta.total_rows() > saves.rows)
        return Error::invalid("replay_batch: no layers, or more rows than the saves hold");
    KDA_TRY(saves.check());
    auto off = [](const Request& r) { return r.state_offset; };
    KDA_TRY(meta.check_regions("state", state, state_bytes(st), (l - 1) * state_stride, state_len(h), true, off));
    KDA_TRY(meta.check_regions("state", state_out, state_bytes(st), (l - 1) * state_stride, state_len(h), true, off));
    if (l > 1) {
        size_t max_off = 0;
        for (const Request& r : meta.requests()) max_off = std::max(max_off, r.state_offset);
        if (state_stride < max_off + state_len(h)) return Error::invalid("replay_batch: layers' regions overlap");
    }
    if (dry_run) return Error::ok();
    if (!meta.on_device()) return Error::invalid("batch metadata has no device arrays");
    int32_t h32, l32;
    KDA_TRY(to_i32(h, "heads", &h32));
    KDA_TRY(to_i32(l, "layers", &l32));
    glm53f_stream_t s = reinterpret_cast<glm53f_stream_t>(stream.raw());
    int code;
    if (st == StateType::F32)
        code = glm53f_kda_replay_batch(h32, l32, batch, meta.cu_rows(), meta.keep_dev(), state.ptr<float>(),
                                       state_out.ptr<float>(), (int64_t)state_stride, meta.state_off(), saves.k.ptr<float>(),
                                       saves.v.ptr<glm53f_bf16>(), saves.g.ptr<float>(), saves.b.ptr<float>(),
                                       (int64_t)saves.kv_stride(), (int64_t)saves.b_stride(), s);
    else
        code = glm53f_kda_replay_batch_bf16state(h32, l32, batch, meta.cu_rows(), meta.keep_dev(), state.ptr<glm53f_bf16>(),
                                                 state_out.ptr<glm53f_bf16>(), (int64_t)state_stride, meta.state_off(),
                                                 saves.k.ptr<float>(), saves.v.ptr<glm53f_bf16>(), saves.g.ptr<float>(),
                                                 saves.b.ptr<float>(), (int64_t)saves.kv_stride(),
                                                 (int64_t)saves.b_stride(), s);
    return launched(code, "glm53f_kda_replay_batch");
}
inline Error replay_batch(const BatchMeta& meta, Buf state, Buf state_out, size_t state_stride, const LayerSaves& saves,
                          const Stream& stream) {
    return replay_batch_as(meta, state, state_out, state_stride, saves, stream, StateType::F32);
}
inline Error replay_batch_bf16_state(const BatchMeta& meta, Buf state, Buf state_out, size_t state_stride,
                                     const LayerSaves& saves, const Stream& stream) {
    return replay_batch_as(meta, state, state_out, state_stride, saves, stream, StateType::Bf16);
}

/// The commit by selection of a checkpointing verify round (glm53f_kda_select_batch_bf16state): request r keeps
/// keep[r] rows; layer l's checkpoints at l * ckpt_layer_stride, its states at l * state_stride.
inline Error select_batch_bf16_state(size_t heads, size_t layers, const BatchMeta& meta, Buf ckpt, size_t ckpt_layer_stride,
                                     Buf state, size_t state_stride, const Stream& stream, bool dry_run = false) {
    int32_t batch;
    KDA_TRY(meta.batch(&batch));
    if (layers == 0) return Error::invalid("select_batch: no layers");
    const size_t per_layer = meta.total_rows() * state_len(heads);
    if (layers > 1 && ckpt_layer_stride < per_layer) return Error::invalid("select_batch: layers' checkpoints overlap");
    KDA_TRY(check_region("ckpt", ckpt, 2, (layers - 1) * ckpt_layer_stride, per_layer));
    KDA_TRY(meta.check_regions("state", state, 2, (layers - 1) * state_stride, state_len(heads), true,
                               [](const Request& r) { return r.state_offset; }));
    if (layers > 1) {
        size_t max_off = 0;
        for (const Request& r : meta.requests()) max_off = std::max(max_off, r.state_offset);
        if (state_stride < max_off + state_len(heads)) return Error::invalid("select_batch: layers' regions overlap");
    }
    if (dry_run) return Error::ok();
    if (!meta.on_device()) return Error::invalid("batch metadata has no device arrays");
    int32_t h32, l32;
    KDA_TRY(to_i32(heads, "heads", &h32));
    KDA_TRY(to_i32(layers, "layers", &l32));
    return launched(glm53f_kda_select_batch_bf16state(h32, l32, batch, meta.cu_rows(), meta.keep_dev(),
                                                      ckpt.ptr<glm53f_bf16>(), (int64_t)ckpt_layer_stride,
                                                      state.ptr<glm53f_bf16>(), (int64_t)state_stride, meta.state_off(),
                                                      reinterpret_cast<glm53f_stream_t>(stream.raw())),
                    "glm53f_kda_select_batch_bf16state");
}

/// Advance every layer's conv window of every request past its kept rows (glm53f_kda_conv_shift_batch;
/// kernel.rs:907-973).
inline Error conv_shift_batch(size_t heads, size_t layers, const BatchMeta& meta, Buf conv, size_t conv_stride,
                              const RowView& p, size_t p_layer_stride, const Stream& stream, bool dry_run = false) {
    const size_t c = channels(heads);
    int32_t batch;
    KDA_TRY(meta.batch(&batch));
    if (layers == 0) return Error::invalid("conv_shift_batch: no layers");
    size_t max_off = 0;
    for (const Request& r : meta.requests()) max_off = std::max(max_off, r.conv_offset);
    if (layers > 1 && conv_stride < max_off + WINDOW * c) return Error::invalid("conv_shift_batch: layers' windows overlap");
    KDA_TRY(meta.check_regions("conv", conv, 2, (layers - 1) * conv_stride, WINDOW * c, true,
                               [](const Request& r) { return r.conv_offset; }));
    for (size_t l : {(size_t)0, layers - 1}) {
        const RowView view(p.buf, p.offset + l * p_layer_stride, p.stride);
        KDA_TRY(view.check("p", 2, 0, meta.total_rows(), 0, (int64_t)c));
    }
    if (dry_run) return Error::ok();
    if (!meta.on_device()) return Error::invalid("batch metadata has no device arrays");
    int32_t c32, l32;
    KDA_TRY(to_i32(c, "channels", &c32));
    KDA_TRY(to_i32(layers, "layers", &l32));
    return launched(glm53f_kda_conv_shift_batch(c32, l32, batch, meta.cu_rows(), meta.keep_dev(), conv.ptr<glm53f_bf16>(),
                                                (int64_t)conv_stride, meta.conv_off(), p.buf.ptr<glm53f_bf16>(p.offset),
                                                (int64_t)p_layer_stride, (int64_t)p.stride,
                                                reinterpret_cast<glm53f_stream_t>(stream.raw())),
                    "glm53f_kda_conv_shift_batch");
}

inline Error check_lower(float lower) {
    if (!(lower >= PREFILL_LOWER_MIN && lower <= 0.0f))
        return Error::invalid("prefill: gate lower bound " + std::to_string(lower) + " outside [-5.8, 0]");
    return Error::ok();
}

inline Error check_value_blocks(size_t value_blocks, int32_t* out) {
    if (value_blocks == 0 || value_blocks == 1 || value_blocks == 2 || value_blocks == 4) {
        *out = (int32_t)value_blocks;
        return Error::ok();
    }
    return Error::invalid("value_blocks " + std::to_string(value_blocks) + ": 0 (choose), 1, 2 or 4");
}

/// Device workspace of the prefill for rows_per_pass rows of every request at a time (kernel.rs:988-1041).
struct PrefillWorkspace {
    size_t heads = 0, batch = 0, rows_per_pass = 0;
    DeviceBuffer storage;
    Buf buf;   // the memory used: `storage`, or a caller's

    static size_t bytes_for(size_t heads, size_t batch, size_t rows_per_pass) {
        return (size_t)glm53f_kda_prefill_workspace_bytes((int32_t)heads, (int32_t)batch, (int32_t)std::max<size_t>(rows_per_pass, 1));
    }
    /// Room for rows_per_pass rows (rounded up to whole chunks) of `batch` requests of `heads` heads.
    static Error create(size_t heads, size_t batch, size_t rows_per_pass, PrefillWorkspace* out) {
        int32_t tmp;
        KDA_TRY(to_i32(heads, "heads", &tmp));
        KDA_TRY(to_i32(batch, "batch", &tmp));
        KDA_TRY(to_i32(std::max<size_t>(rows_per_pass, 1), "rows_per_pass", &tmp));
        out->heads = heads;
        out->batch = batch;
        out->rows_per_pass = (std::max<size_t>(rows_per_pass, 1) + PREFILL_CHUNK - 1) / PREFILL_CHUNK * PREFILL_CHUNK;
        KDA_TRY(DeviceBuffer::alloc(bytes_for(heads, batch, rows_per_pass), &out->storage));
        out->buf = out->storage;
        return Error::ok();
    }
    /// The rows per pass that keep the workspace within `bytes` (at least one chunk).
    static Error within(size_t heads, size_t batch, size_t bytes, PrefillWorkspace* out) {
        const size_t chunk = std::max<size_t>(bytes_for(heads, batch, PREFILL_CHUNK), 1);
        return create(heads, batch, std::max<size_t>(bytes / chunk, 1) * PREFILL_CHUNK, out);
    }
    Error args(size_t h, size_t b, float** ws, int64_t* ws_bytes) const {
        if (h != heads || b > batch)
            return Error::invalid("workspace for " + std::to_string(heads) + " heads x " + std::to_string(batch) +
                                  " requests used for " + std::to_string(h) + " x " + std::to_string(b));
        *ws = buf.ptr<float>();
        *ws_bytes = (int64_t)buf.bytes;
        return Error::ok();
    }
};

/// One layer, one request: a prompt segment through the chunked prefill (glm53f_kda_prefill; kernel.rs:1052-1141).
struct Prefill {
    const Weights* weights = nullptr;
    size_t rows = 0;
    RowView p;
    int64_t b_off = 0;
    RowView a, g;
    Buf conv;
    size_t conv_offset = 0;
    Buf state;
    size_t state_offset = 0;
    StateOut state_out;   // InPlace or To; the prefill always writes its state
    RowView out;
    size_t value_blocks = 0;
    const PrefillWorkspace* workspace = nullptr;

    Error check(float** state_out_ptr, int32_t* vb, float** ws, int64_t* ws_bytes) const {
        KDA_TRY(weights->check());
        const size_t h = weights->heads;
        KDA_TRY(check_value_blocks(value_blocks, vb));
        KDA_TRY(check_lower(weights->lower));
        const int64_t c = (int64_t)channels(h);
        const int64_t lo = std::min<int64_t>(b_off, 0), hi = std::max<int64_t>(c, b_off + (int64_t)h);
        KDA_TRY(p.check("p", 2, 0, rows, lo, hi));
        KDA_TRY(a.check("a", 2, 0, rows, 0, (int64_t)(h * DK)));
        KDA_TRY(g.check("g", 2, 0, rows, 0, (int64_t)(h * DV)));
        KDA_TRY(out.check("out", 2, 0, rows, 0, (int64_t)(h * DV)));
        if (rows > 1 && out.stride < h * DV) return Error::invalid("out rows overlap");
        KDA_TRY(check_region("conv", conv, 2, conv_offset, WINDOW * channels(h)));
        KDA_TRY(check_region("state", state, 4, state_offset, state_len(h)));
        if (state_out.kind == StateOut::Skip) return Error::invalid("a prefill always writes its state");
        if (state_out.kind == StateOut::InPlace) {
            *state_out_ptr = state.ptr<float>(state_offset);
        } else {
            KDA_TRY(check_region("state_out", state_out.buf, 4, state_out.offset, state_len(h)));
            if (same(state_out.buf, state) && !coincide_or_disjoint(state_out.offset, state_offset, state_len(h)))
                return Error::invalid("state_out partly overlaps the state");
            *state_out_ptr = state_out.buf.ptr<float>(state_out.offset);
        }
        return workspace->args(h, 1, ws, ws_bytes);
    }

    Error launch(const Stream& stream) const {
        float *so = nullptr, *ws = nullptr;
        int32_t vb = 0;
        int64_t wsb = 0;
        KDA_TRY(check(&so, &vb, &ws, &wsb));
        const Weights& w = *weights;
        int32_t h32, r32;
        KDA_TRY(to_i32(w.heads, "heads", &h32));
        KDA_TRY(to_i32(rows, "rows", &r32));
        return launched(
            glm53f_kda_prefill(h32, r32, p.buf.ptr<glm53f_bf16>(p.offset), (int64_t)p.stride, b_off,
                               a.buf.ptr<glm53f_bf16>(a.offset), (int64_t)a.stride, g.buf.ptr<glm53f_bf16>(g.offset),
                               (int64_t)g.stride, conv.ptr<glm53f_bf16>(conv_offset), w.conv_w.ptr<glm53f_bf16>(),
                               state.ptr<float>(state_offset), so, w.a_log.ptr<float>(), w.dt_bias.ptr<float>(),
                               w.norm_w.ptr<glm53f_bf16>(), w.eps, w.lower, out.buf.ptr<glm53f_bf16>(out.offset),
                               (int64_t)out.stride, vb, ws, wsb, reinterpret_cast<glm53f_stream_t>(stream.raw())),
            "glm53f_kda_prefill");
    }
};

/// One layer, a batch of prompt segments (glm53f_kda_prefill_batch[_bf16state]; kernel.rs:1143-1285).
struct PrefillBatch {
    const Weights* weights = nullptr;
    RowView p;
    int64_t b_off = 0;
    RowView a, g;
    Buf conv;
    Buf state;
    StateOut state_out;   // InPlace, or To(buf, _): each request's state at its state_offset in buf
    RowView out;
    size_t value_blocks = 0;
    const PrefillWorkspace* workspace = nullptr;

    Error check(const BatchMeta& meta, StateType st, void** state_out_ptr, int32_t* vb, float** ws, int64_t* ws_bytes) const {
        KDA_TRY(weights->check());
        const size_t es = state_bytes(st), h = weights->heads;
        KDA_TRY(check_value_blocks(value_blocks, vb));
        KDA_TRY(check_lower(weights->lower));
        int32_t batch;
        KDA_TRY(meta.batch(&batch));
        const size_t total = meta.total_rows();
        const int64_t c = (int64_t)channels(h);
        const int64_t lo = std::min<int64_t>(b_off, 0), hi = std::max<int64_t>(c, b_off + (int64_t)h);
        KDA_TRY(p.check("p", 2, 0, total, lo, hi));
        KDA_TRY(a.check("a", 2, 0, total, 0, (int64_t)(h * DK)));
        KDA_TRY(g.check("g", 2, 0, total, 0, (int64_t)(h * DV)));
        KDA_TRY(out.check("out", 2, 0, total, 0, (int64_t)(h * DV)));
        if (total > 1 && out.stride < h * DV) return Error::invalid("out rows overlap");
        // The windows are written: they must not overlap.
        KDA_TRY(meta.check_regions("conv", conv, 2, 0, WINDOW * channels(h), true, [](const Request& r) { return r.conv_offset; }));
        KDA_TRY(meta.check_regions("state", state, es, 0, state_len(h), true, [](const Request& r) { return r.state_offset; }));
        if (state_out.kind == StateOut::Skip) return Error::invalid("a prefill always writes its state");
        if (state_out.kind == StateOut::InPlace) {
            *state_out_ptr = state.p;
        } else {
            KDA_TRY(meta.check_regions("state_out", state_out.buf, es, 0, state_len(h), true,
                                       [](const Request& r) { return r.state_offset; }));
            if (same(state_out.buf, state)) return Error::invalid("state_out is the state buffer: use InPlace");
            *state_out_ptr = state_out.buf.p;
        }
        return workspace->args(h, (size_t)batch, ws, ws_bytes);
    }

    Error launch(const BatchMeta& meta, const Stream& stream) const { return launch_as(meta, stream, StateType::F32); }
    Error launch_bf16_state(const BatchMeta& meta, const Stream& stream) const { return launch_as(meta, stream, StateType::Bf16); }

    Error launch_as(const BatchMeta& meta, const Stream& stream, StateType st) const {
        void* so = nullptr;
        float* ws = nullptr;
        int32_t vb = 0;
        int64_t wsb = 0;
        KDA_TRY(check(meta, st, &so, &vb, &ws, &wsb));
        if (!meta.on_device()) return Error::invalid("batch metadata has no device arrays");
        const Weights& w = *weights;
        int32_t h32, batch, max_rows;
        KDA_TRY(to_i32(w.heads, "heads", &h32));
        KDA_TRY(meta.batch(&batch));
        KDA_TRY(to_i32(meta.max_rows(), "max_rows", &max_rows));
        const glm53f_bf16* pp = p.buf.ptr<glm53f_bf16>(p.offset);
        const glm53f_bf16* ap = a.buf.ptr<glm53f_bf16>(a.offset);
        const glm53f_bf16* gp = g.buf.ptr<glm53f_bf16>(g.offset);
        glm53f_bf16* op = out.buf.ptr<glm53f_bf16>(out.offset);
        glm53f_stream_t s = reinterpret_cast<glm53f_stream_t>(stream.raw());
        int code;
        if (st == StateType::F32)
            code = glm53f_kda_prefill_batch(h32, batch, meta.cu_rows(), max_rows, pp, (int64_t)p.stride, b_off, ap,
                                            (int64_t)a.stride, gp, (int64_t)g.stride, conv.ptr<glm53f_bf16>(), meta.conv_off(),
                                            w.conv_w.ptr<glm53f_bf16>(), state.ptr<float>(), reinterpret_cast<float*>(so),
                                            meta.state_off(), w.a_log.ptr<float>(), w.dt_bias.ptr<float>(),
                                            w.norm_w.ptr<glm53f_bf16>(), w.eps, w.lower, op, (int64_t)out.stride, vb, ws, wsb, s);
        else
            code = glm53f_kda_prefill_batch_bf16state(
                h32, batch, meta.cu_rows(), max_rows, pp, (int64_t)p.stride, b_off, ap, (int64_t)a.stride, gp,
                (int64_t)g.stride, conv.ptr<glm53f_bf16>(), meta.conv_off(), w.conv_w.ptr<glm53f_bf16>(),
                state.ptr<glm53f_bf16>(), reinterpret_cast<glm53f_bf16*>(so), meta.state_off(), w.a_log.ptr<float>(),
                w.dt_bias.ptr<float>(), w.norm_w.ptr<glm53f_bf16>(), w.eps, w.lower, op, (int64_t)out.stride, vb, ws, wsb, s);
        return launched(code, "glm53f_kda_prefill_batch");
    }
};

}  // namespace glm53f_kda

#endif  // GLM53F_KDA_HOST_KERNEL_HPP
