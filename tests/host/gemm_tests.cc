// Tests of the C++ GEMM engine (glm53f-afd_amd/host/gemm.hpp). `--cpu`: the policy and shape rules, without touching
// a GPU. `--gpu`: the three dispatch targets (GEMV, the GEMM for 9 to 64 rows, the vendor GEMM) on the same inputs
// against exact arithmetic over the bf16 values, within f32 rounding - what the reference's tests/gemv.rs:180-226
// asks of its GEMV and cuBLAS.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "gemm.hpp"
#include "kda_ref.h"   // the oracle's bf16 conversions and generator: test infrastructure

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
    GemmPolicy p;
    EXPECT(p.gemv_max_rows == 8 && p.skinny_max_rows == 64);
    EXPECT_OK(Gemm::check(p));
    p.gemv_max_rows = 9;
    EXPECT_INVALID(Gemm::check(p));
    p.gemv_max_rows = 0; p.skinny_max_rows = 65;
    EXPECT_INVALID(Gemm::check(p));
    p.skinny_max_rows = 0;
    EXPECT_OK(Gemm::check(p));

    // the split rule is the library's (shape only): the KDA layer's four projections
    const uint16_t* wp = reinterpret_cast<const uint16_t*>(uintptr_t(0x10000));
    Bf16Mat qkvb{wp, 24640, 4096, 4096}, fga{wp, 256, 4096, 4096}, fgb{wp, 8192, 128, 128, 2, 8192 * 128}, o{wp, 4096, 8192, 8192};
    EXPECT(Gemm::gemv_ksplit(qkvb) == 1 && Gemm::gemv_ksplit(fga) == 4 && Gemm::gemv_ksplit(fgb) == 1 && Gemm::gemv_ksplit(o) == 1);
    EXPECT(qkvb.bytes() == size_t(24640) * 4096 * 2 && fgb.bytes() == size_t(2) * 8192 * 128 * 2);
    EXPECT(Gemm::gemv_scratch_holds(fga, 8));
    Bf16Mat wide{wp, size_t(1) << 20, 1024, 1024};            // no split: no scratch needed
    EXPECT(Gemm::gemv_ksplit(wide) == 1 && Gemm::gemv_scratch_holds(wide, 8));
    Bf16Mat deep{wp, 8, size_t(1) << 20, size_t(1) << 20};    // the deepest split the rule gives still fits the scratch
    EXPECT(Gemm::gemv_ksplit(deep) > 1 && Gemm::gemv_scratch_holds(deep, 8));

    // what the GEMM for 9 to 64 rows takes
    EXPECT(Gemm::skinny_takes(qkvb, 4096, 0, 24640, 0, false));
    EXPECT(Gemm::skinny_takes(fgb, 256, 128, 16384, 8192, false));
    Bf16Mat n24{wp, 24, 4096, 4096}, k192{wp, 64, 192, 192}, ld{wp, 64, 256, 260}, odd{wp + 1, 64, 256, 256};
    EXPECT(!Gemm::skinny_takes(n24, 4096, 0, 24, 0, false) && !Gemm::skinny_takes(k192, 192, 0, 64, 0, false));
    EXPECT(!Gemm::skinny_takes(ld, 256, 0, 64, 0, false) && !Gemm::skinny_takes(odd, 256, 0, 64, 0, false));
    Bf16Mat ok{wp, 64, 256, 256};
    EXPECT(Gemm::skinny_takes(ok, 256, 0, 65, 0, true) && !Gemm::skinny_takes(ok, 256, 0, 65, 0, false));
    EXPECT(!Gemm::skinny_takes(ok, 260, 0, 64, 0, false));

    EXPECT(launched(0, "x").is_ok() && launched(1, "x").kind == Error::Invalid && launched(700, "x").kind == Error::Hip);
    Blas empty;
    EXPECT_INVALID(empty.gemm(GemmDesc{}));
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
// deterministic values in (-1, 1)
static std::vector<float> values(size_t n, uint32_t seed, float scale) {
    std::vector<float> v(n);
    uint32_t s = seed * 2654435761u + 12345u;
    for (size_t i = 0; i < n; ++i) {
        s = s * 1664525u + 1013904223u;
        v[i] = scale * ((float)(s >> 8) / 8388608.0f - 1.0f);
    }
    return v;
}

// One shape through Gemm::bf16 for several row counts, against f64 over the bf16 values.
static void shape(const Gemm& gemm, const Stream& stream, size_t groups, size_t n, size_t k, size_t ldx, size_t x_gs, size_t ldo,
                  size_t o_gs, const std::vector<size_t>& row_counts, bool out_f32) {
    const size_t max_rows = 100;
    std::vector<uint16_t> w16 = enc(values(groups * n * k, 7, 0.05f)), x16 = enc(values(max_rows * ldx, 9, 1.0f));
    std::vector<float> wf = dec(w16), xf = dec(x16);
    DeviceBuffer d_w, d_x, d_o;
    EXPECT_OK(DeviceBuffer::from_slice(w16, &d_w));
    EXPECT_OK(DeviceBuffer::from_slice(x16, &d_x));
    const size_t es = out_f32 ? 4 : 2;
    EXPECT_OK(DeviceBuffer::alloc(max_rows * ldo * es, &d_o));
    Bf16Mat w{d_w.ptr<uint16_t>(), n, k, k, groups, n * k};
    for (size_t rows : row_counts) {
        EXPECT_OK(glm53f_kda::check_hip(hipMemset(d_o.ptr<unsigned char>(), 0xff, max_rows * ldo * es), "hipMemset"));
        EXPECT_OK(gemm.bf16(d_x.ptr<uint16_t>(), ldx, x_gs, w, rows, d_o.ptr<unsigned char>(), ldo, o_gs, out_f32, stream));
        EXPECT_OK(stream.synchronize());
        std::vector<float> got;
        if (out_f32) {
            EXPECT_OK(d_o.to_vec(&got));
        } else {
            std::vector<uint16_t> g16;
            EXPECT_OK(d_o.to_vec(&g16));
            got = dec(g16);
        }
        double worst = 0;
        for (size_t g = 0; g < groups; ++g)
            for (size_t m = 0; m < rows; ++m)
                for (size_t o = 0; o < n; ++o) {
                    double ref = 0, mag = 0;
                    for (size_t i = 0; i < k; ++i) {
                        const double t = (double)xf[g * x_gs + m * ldx + i] * (double)wf[(g * n + o) * k + i];
                        ref += t; mag += std::fabs(t);
                    }
                    const double tol = 16 * std::ldexp(mag, -24) + (out_f32 ? 0.0 : std::ldexp(std::fabs(ref), -8)) + 1e-30;
                    worst = std::fmax(worst, std::fabs((double)got[g * o_gs + m * ldo + o] - ref) / tol);
                }
        std::printf("groups %zu n %zu k %zu rows %zu %s out: worst error / tolerance %.3f\n", groups, n, k, rows, out_f32 ? "f32" : "bf16", worst);
        EXPECT(worst <= 1.0);
    }
}

static void gpu_tests() {
    Stream stream = Stream::null();
    EXPECT_OK(Stream::create(&stream));
    Gemm gemm;
    EXPECT_OK(Gemm::create(stream, GemmPolicy{}, &gemm));
    EXPECT(gemm.bytes() == kBlasWorkspace + kPartialFloats * 4 + kSyncCounters * 4);
    // rows 1..8 the GEMV, 9..64 the GEMM for 9 to 64 rows, more the vendor GEMM
    shape(gemm, stream, 1, 96, 1024, 1024, 0, 96, 0, {1, 8, 9, 16, 40, 64, 65, 100}, true);
    shape(gemm, stream, 1, 96, 1024, 1024, 0, 96, 0, {3, 20, 70}, false);
    // two groups with the engine's strides for the gates' second projection (activations side by side, outputs interleaved)
    shape(gemm, stream, 2, 64, 128, 256, 128, 128, 64, {2, 16, 33, 80}, false);
    // a shape the GEMM for 9 to 64 rows does not take (n % 16 != 0) goes to the vendor GEMM at 16 rows
    shape(gemm, stream, 1, 40, 256, 256, 0, 40, 0, {8, 16}, true);
    // the reference's dispatch
    Gemm plain;
    GemmPolicy ref_policy; ref_policy.skinny_max_rows = 0;
    EXPECT_OK(Gemm::create(stream, ref_policy, &plain));
    shape(plain, stream, 1, 96, 1024, 1024, 0, 96, 0, {8, 16, 64}, true);
    // a rejected launch comes back as Invalid
    Bf16Mat bad{nullptr, 96, 1024, 1024};
    EXPECT_INVALID(gemm.gemv(nullptr, 1024, 0, bad, 4, nullptr, 96, 0, true, stream));
    EXPECT_INVALID(gemm.skinny(nullptr, 1024, 0, bad, 16, nullptr, 96, 0, true, stream));
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
