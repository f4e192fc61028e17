// The forward's BF16 weight GEMM engine over the C ABI of this library: the C++ counterpart of the BF16 half of the
// reference's crates/glm53f-forward/src/gemm.rs:33-43 (Bf16Mat), :93-143 (GemmPolicy, scratch sizes), :150-325 (Gemm:
// new, bytes, gemv_ksplit, bf16, gemv, cublas) and of src/cublas.rs:98-245 (GemmDesc, Blas), with hipBLAS where the
// reference binds cuBLAS. One dispatch more than the reference's: between the GEMV (up to 8 rows) and the vendor GEMM
// sits this library's weight-streaming GEMM for 9 to 64 rows (glm53f_fwd_gemm_bf16_skinny); `skinny_max_rows = 0`
// gives the reference's dispatch. The FP8 and MXFP8 paths of gemm.rs are not part of the KDA layers' BF16 projections
// and are not mirrored. Header only; link with the kernel library, amdhip64 and hipblas.
#ifndef GLM53F_FORWARD_HOST_GEMM_HPP
#define GLM53F_FORWARD_HOST_GEMM_HPP

#include <hipblas/hipblas.h>

#include <climits>
#include <cstddef>
#include <cstdint>
#include <string>
#include <utility>

#include "device.hpp"
#include "glm53f_fwd_gemv.h"

namespace glm53f_forward {

using glm53f_kda::DeviceBuffer;
using glm53f_kda::Error;
using glm53f_kda::Stream;

/// A BF16 weight [groups][n][k] on the device: row o of group g at ptr + g * gstride + o * ld (gemm.rs:33-43).
struct Bf16Mat {
    const uint16_t* ptr = nullptr;
    size_t n = 0, k = 0, ld = 0, groups = 1, gstride = 0;
    size_t bytes() const { return groups * n * k * 2; }
};

/// Which kernel each BF16 GEMM uses (gemm.rs:93-120, its BF16 field, and the one added here).
struct GemmPolicy {
    /// GEMMs with at most this many rows run the GEMV (8 at most; 0 sends none there).
    size_t gemv_max_rows = 8;
    /// GEMMs with more rows than that, up to this many (64 at most), run the library's GEMM for 9 to 64 rows where
    /// its shape rules allow; 0: never, everything above the GEMV goes to the vendor GEMM as in the reference.
    size_t skinny_max_rows = 64;
};

constexpr size_t kPartialFloats = size_t(1) << 20;   // split-K partial sums (gemm.rs:143)
constexpr size_t kSyncCounters = size_t(1) << 16;    // one zeroed counter per 8 outputs of a split GEMV (gemm.rs:144)
constexpr size_t kBlasWorkspace = size_t(32) << 20;  // the vendor library's workspace (gemm.rs:146)

/// One BF16 GEMM, row-major Y [rows][n] = X [rows][k] . W^T with W [n][k], possibly batched over `groups` with
/// element strides between them (cublas.rs:98-117).
struct GemmDesc {
    size_t rows = 0, n = 0, k = 0;
    const uint16_t* x = nullptr; size_t ldx = 0;
    const uint16_t* w = nullptr; size_t ldw = 0;
    void* out = nullptr; size_t ldo = 0;
    bool out_f32 = false;
    size_t groups = 1, x_gstride = 0, w_gstride = 0, o_gstride = 0;
};

/// A hipBLAS handle bound to one stream, with its own workspace (cublas.rs:119-245). In the library's
/// column-major terms the row-major product above is C (n x rows, ldc = ldo) = W^T-read (lda = ldw) times X (ldb = ldx).
class Blas {
  public:
    Blas() = default;
    Blas(const Blas&) = delete;
    Blas& operator=(const Blas&) = delete;
    Blas(Blas&& o) noexcept : handle_(o.handle_), workspace_(std::move(o.workspace_)) { o.handle_ = nullptr; }
    Blas& operator=(Blas&& o) noexcept {
        if (this != &o) {
            release();
            handle_ = o.handle_; workspace_ = std::move(o.workspace_);
            o.handle_ = nullptr;
        }
        return *this;
    }
    ~Blas() { release(); }

    static Error create(const Stream& stream, size_t workspace_bytes, Blas* out) {
        Blas b;
        Error e = status(hipblasCreate(&b.handle_), "hipblasCreate");
        if (!e) return e;
        if (!(e = DeviceBuffer::alloc(workspace_bytes, &b.workspace_))) return e;
        if (!(e = status(hipblasSetStream(b.handle_, stream.raw()), "hipblasSetStream"))) return e;
        if (workspace_bytes > 0 &&
            !(e = status(hipblasSetWorkspace(b.handle_, b.workspace_.ptr<unsigned char>(), workspace_bytes), "hipblasSetWorkspace")))
            return e;
        *out = std::move(b);
        return Error::ok();
    }

    /// Launch `d` (BF16 inputs, f32 accumulation, BF16 or f32 output) on the handle's stream.
    Error gemm(const GemmDesc& d) const {
        if (handle_ == nullptr) return Error::invalid("Blas::gemm on an empty handle");
        const float alpha = 1.0f, beta = 0.0f;
        const hipDataType ctype = d.out_f32 ? HIP_R_32F : HIP_R_16BF;
        int m, n, k, lda, ldb, ldc, groups;
        Error e;
        if (!(e = to_int(d.n, "n", &m)) || !(e = to_int(d.rows, "rows", &n)) || !(e = to_int(d.k, "k", &k)) ||
            !(e = to_int(d.ldw, "ldw", &lda)) || !(e = to_int(d.ldx, "ldx", &ldb)) || !(e = to_int(d.ldo, "ldo", &ldc)) ||
            !(e = to_int(d.groups, "groups", &groups)))
            return e;
        if (d.groups <= 1)
            return status(hipblasGemmEx(handle_, HIPBLAS_OP_T, HIPBLAS_OP_N, m, n, k, &alpha, d.w, HIP_R_16BF, lda, d.x,
                                        HIP_R_16BF, ldb, &beta, d.out, ctype, ldc, HIPBLAS_COMPUTE_32F, HIPBLAS_GEMM_DEFAULT),
                          "hipblasGemmEx");
        return status(hipblasGemmStridedBatchedEx(handle_, HIPBLAS_OP_T, HIPBLAS_OP_N, m, n, k, &alpha, d.w, HIP_R_16BF, lda,
                                                  (hipblasStride)d.w_gstride, d.x, HIP_R_16BF, ldb, (hipblasStride)d.x_gstride,
                                                  &beta, d.out, ctype, ldc, (hipblasStride)d.o_gstride, groups,
                                                  HIPBLAS_COMPUTE_32F, HIPBLAS_GEMM_DEFAULT),
                      "hipblasGemmStridedBatchedEx");
    }

  private:
    static Error status(hipblasStatus_t s, const char* what) {
        if (s == HIPBLAS_STATUS_SUCCESS) return Error::ok();
        return Error::hip((int)s, std::string(what) + ": hipblasStatus " + std::to_string((int)s));
    }
    static Error to_int(size_t v, const char* what, int* out) {
        if (v > (size_t)INT_MAX) return Error::invalid(std::string(what) + " = " + std::to_string(v) + " does not fit in 32 bits");
        *out = (int)v;
        return Error::ok();
    }
    void release() {
        if (handle_ != nullptr) (void)hipblasDestroy(handle_);
        handle_ = nullptr;
    }
    hipblasHandle_t handle_ = nullptr;
    DeviceBuffer workspace_;
};

inline Error launched(int code, const char* what) {
    if (code == 0) return Error::ok();
    if (code == 1) return Error::invalid(std::string(what) + " rejected its arguments");
    return Error::hip(code, std::string(what) + ": " + hipGetErrorString((hipError_t)code));
}

/// The GEMM engine: a vendor-library handle and the split-K scratch the GEMV launches share (one stream: launches
/// run one after another, and the kernel leaves the counters zeroed) (gemm.rs:150-180).
class Gemm {
  public:
    GemmPolicy policy;

    Gemm() = default;
    Gemm(Gemm&&) noexcept = default;
    Gemm& operator=(Gemm&&) noexcept = default;

    /// The policy is checked before anything is allocated (gemm.rs:162-165; the second check is this mirror's).
    static Error check(const GemmPolicy& p) {
        if (p.gemv_max_rows > 8) return Error::invalid("the GEMV takes at most 8 rows");
        if (p.skinny_max_rows > 64) return Error::invalid("the GEMM for 9 to 64 rows takes at most 64 rows");
        return Error::ok();
    }
    static Error create(const Stream& stream, const GemmPolicy& policy, Gemm* out) {
        Error e = check(policy);
        if (!e) return e;
        Gemm g;
        g.policy = policy;
        if (!(e = Blas::create(stream, kBlasWorkspace, &g.blas_))) return e;
        if (!(e = DeviceBuffer::alloc(kPartialFloats * 4, &g.partials_))) return e;
        if (!(e = DeviceBuffer::zeroed(kSyncCounters * 4, &g.sync_))) return e;
        *out = std::move(g);
        return Error::ok();
    }

    /// Device bytes of its scratch (gemm.rs:182-189).
    size_t bytes() const { return kBlasWorkspace + partials_.bytes() + sync_.bytes(); }

    /// The GEMV's K splits for `w` (shape only; gemm.rs:199-203).
    static size_t gemv_ksplit(const Bf16Mat& w) {
        return (size_t)glm53f_fwd_gemv_ksplit((int32_t)w.groups, (int32_t)w.n, (int32_t)w.k);
    }

    /// Whether the split-K scratch holds a GEMV of `rows` rows of `w` (gemm.rs:254-260).
    static bool gemv_scratch_holds(const Bf16Mat& w, size_t rows) {
        const size_t ksplit = gemv_ksplit(w);
        return ksplit <= 1 || (w.groups * ksplit * rows * w.n <= kPartialFloats && w.groups * w.n / 8 <= kSyncCounters);
    }

    /// The shapes glm53f_fwd_gemm_bf16_skinny accepts; others go to the vendor GEMM.
    static bool skinny_takes(const Bf16Mat& w, size_t ldx, size_t x_gstride, size_t ldo, size_t o_gstride, bool out_f32) {
        return w.n >= 16 && w.n % 16 == 0 && w.k >= 128 && w.k % 128 == 0 && w.ld % 8 == 0 && w.gstride % 8 == 0 &&
               ldx % 8 == 0 && x_gstride % 8 == 0 && (reinterpret_cast<uintptr_t>(w.ptr) & 15u) == 0 && w.groups <= 65535 &&
               (out_f32 || (ldo % 2 == 0 && o_gstride % 2 == 0));
    }

    /// out[g][m][o] = x[g][m] . w[g][o] for `rows` rows: BF16 inputs, f32 accumulation, BF16 (or f32) output.
    /// x rows are ldx apart and groups x_gstride; out rows ldo and groups o_gstride (gemm.rs:205-236). The pointers
    /// name live device buffers of those shapes that stay alive until the stream's work completes.
    Error bf16(const uint16_t* x, size_t ldx, size_t x_gstride, const Bf16Mat& w, size_t rows, void* out, size_t ldo,
               size_t o_gstride, bool out_f32, const Stream& stream) const {
        if (rows == 0) return Error::ok();
        if (rows <= policy.gemv_max_rows) return gemv(x, ldx, x_gstride, w, rows, out, ldo, o_gstride, out_f32, stream);
        if (rows <= policy.skinny_max_rows && skinny_takes(w, ldx, x_gstride, ldo, o_gstride, out_f32) &&
            (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(out) & 3u) == 0)
            return skinny(x, ldx, x_gstride, w, rows, out, ldo, o_gstride, out_f32, stream);
        return blas(x, ldx, x_gstride, w, rows, out, ldo, o_gstride, out_f32);
    }

    /// The GEMV (1..8 rows), whatever the policy (gemm.rs:238-291).
    Error gemv(const uint16_t* x, size_t ldx, size_t x_gstride, const Bf16Mat& w, size_t rows, void* out, size_t ldo,
               size_t o_gstride, bool out_f32, const Stream& stream) const {
        if (!gemv_scratch_holds(w, rows)) return Error::invalid("GEMV split-K scratch too small for the weight");
        return launched(glm53f_fwd_gemv_bf16(x, (int64_t)ldx, (int64_t)x_gstride, w.ptr, (int64_t)w.ld, (int64_t)w.gstride,
                                             (int32_t)w.groups, (int32_t)rows, (int32_t)w.n, (int32_t)w.k,
                                             (int32_t)gemv_ksplit(w), partials_.ptr<float>(), sync_.ptr<uint32_t>(), out,
                                             out_f32 ? 1 : 0, (int64_t)ldo, (int64_t)o_gstride, stream.raw()),
                        "glm53f_fwd_gemv_bf16");
    }

    /// The weight-streaming GEMM for up to 64 rows, whatever the policy (no counterpart in the reference, which calls
    /// cuBLAS here: gemm.rs:228-234).
    Error skinny(const uint16_t* x, size_t ldx, size_t x_gstride, const Bf16Mat& w, size_t rows, void* out, size_t ldo,
                 size_t o_gstride, bool out_f32, const Stream& stream) const {
        return launched(glm53f_fwd_gemm_bf16_skinny(x, (int64_t)ldx, (int64_t)x_gstride, w.ptr, (int64_t)w.ld,
                                                    (int64_t)w.gstride, (int32_t)w.groups, (int32_t)rows, (int32_t)w.n,
                                                    (int32_t)w.k, out, out_f32 ? 1 : 0, (int64_t)ldo, (int64_t)o_gstride,
                                                    stream.raw()),
                        "glm53f_fwd_gemm_bf16_skinny");
    }

    /// The vendor GEMM, whatever the policy, on the stream the engine was created on (gemm.rs:293-325).
    Error blas(const uint16_t* x, size_t ldx, size_t x_gstride, const Bf16Mat& w, size_t rows, void* out, size_t ldo,
               size_t o_gstride, bool out_f32) const {
        GemmDesc d;
        d.rows = rows; d.n = w.n; d.k = w.k;
        d.x = x; d.ldx = ldx;
        d.w = w.ptr; d.ldw = w.ld;
        d.out = out; d.ldo = ldo; d.out_f32 = out_f32;
        d.groups = w.groups; d.x_gstride = x_gstride; d.w_gstride = w.gstride; d.o_gstride = o_gstride;
        return blas_.gemm(d);
    }

  private:
    Blas blas_;
    DeviceBuffer partials_, sync_;
};

}  // namespace glm53f_forward

#endif  // GLM53F_FORWARD_HOST_GEMM_HPP
