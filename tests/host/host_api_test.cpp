// Tests of the C++ host layer (torsh_amd/host/include/torsh_hipq/*.hpp).  The first group
// restates the reference's own unit tests against the mirrored API
// (crates/torsh-quantization/src/algorithms.rs:736-893, simd_ops.rs:475-582,
//  crates/torsh-backend/src/quantization/params.rs tests); the second group compares the
// device results with the CPU oracle on seeded random inputs, bit for bit.
//
// Output: one line per case, "ok <name>", "FAIL <name>: <why>" or "skip <name>"; exit status 1
// if any case failed.  `--cpu-only` runs the cases that never reach the device.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <random>
#include <sstream>

#include "torsh_hipq/backend.hpp"
#include "torsh_hipq/calibration.hpp"
#include "torsh_hipq/fake_quantize.hpp"
#include "torsh_hipq/hardware.hpp"
#include "torsh_hipq/models.hpp"
#include "torsh_hipq/nn.hpp"
#include "torsh_hipq/nn_quantization.hpp"
#include "torsh_hipq/quantization.hpp"
#include "torsh_hipq/serialize.hpp"
#include "torsh_calib_oracle.h"
#include "torsh_quant_oracle.h"

using namespace torsh;
using namespace torsh::quantization;
namespace bq = torsh::backend::quantization;
namespace mq = torsh::models::quantization;

namespace {

struct Case {
    const char *name;
    bool needs_gpu;
    std::function<void()> fn;
};
std::vector<Case> &cases() {
    static std::vector<Case> c;
    return c;
}
struct Reg {
    Reg(const char *n, bool g, std::function<void()> f) { cases().push_back({n, g, std::move(f)}); }
};
struct Failure {
    std::string why;
};
#define CPU_TEST(name) \
    void name();       \
    Reg reg_##name(#name, false, name); \
    void name()
#define GPU_TEST(name) \
    void name();       \
    Reg reg_##name(#name, true, name); \
    void name()
#define CHECK(cond)                                                                    \
    do {                                                                               \
        if (!(cond)) {                                                                 \
            std::ostringstream o;                                                      \
            o << __LINE__ << ": " #cond;                                               \
            throw Failure{o.str()};                                                    \
        }                                                                              \
    } while (0)
#define CHECK_EQ(a, b)                                                                 \
    do {                                                                               \
        if (!((a) == (b))) {                                                           \
            std::ostringstream o;                                                      \
            o << __LINE__ << ": " #a " == " #b " (" << (a) << " vs " << (b) << ")";    \
            throw Failure{o.str()};                                                    \
        }                                                                              \
    } while (0)

std::vector<float> normal(size_t n, unsigned seed, float sigma = 1.0f, bool relu = false) {
    std::mt19937 g(seed);
    std::normal_distribution<float> d(0.0f, sigma);
    std::vector<float> v(n);
    for (auto &x : v) {
        x = d(g);
        if (relu && x < 0) x = 0;
    }
    return v;
}
template <typename A, typename B>
void check_same(const std::vector<A> &a, const std::vector<B> &b, int line) {
    if (a.size() != b.size()) throw Failure{std::to_string(line) + ": size mismatch"};
    for (size_t i = 0; i < a.size(); ++i)
        if (!(static_cast<double>(a[i]) == static_cast<double>(b[i]))) {
            std::ostringstream o;
            o << line << ": element " << i << ": " << static_cast<double>(a[i]) << " vs " << static_cast<double>(b[i]);
            throw Failure{o.str()};
        }
}
#define CHECK_SAME(a, b) check_same(a, b, __LINE__)
// As check_same for f32 carriers that may hold NaN: a NaN must face a NaN.
void check_same_bits(const std::vector<float> &a, const std::vector<float> &b, int line) {
    if (a.size() != b.size()) throw Failure{std::to_string(line) + ": size mismatch"};
    for (size_t i = 0; i < a.size(); ++i)
        if (!(a[i] == b[i] || (std::isnan(a[i]) && std::isnan(b[i])))) {
            std::ostringstream o;
            o << line << ": element " << i << ": " << a[i] << " vs " << b[i];
            throw Failure{o.str()};
        }
}

// ---------------------------------------------------------------- host logic (no device)

CPU_TEST(test_calculate_affine_quantization_params) {  // algorithms.rs:742-760
    auto [scale, zp] = calculate_affine_quantization_params(-1.0f, 1.0f, DType::I8).unwrap();
    CHECK(scale > 0.0f);
    CHECK(zp >= -128 && zp <= 127);
    float s_ref;
    int32_t z_ref;
    CHECK_EQ(tq_calculate_affine_params(-1.0f, 1.0f, TQ_DTYPE_I8, &s_ref, &z_ref), 0);
    CHECK_EQ(scale, s_ref);
    CHECK_EQ(zp, z_ref);
    auto [s2, z2] = calculate_affine_quantization_params(1.0f, 1.0f, DType::I8).unwrap();
    CHECK_EQ(s2, 1.0f);
    CHECK_EQ(z2, -128);
    CHECK(calculate_affine_quantization_params(2.0f, 1.0f, DType::I8).is_err());
    CHECK(calculate_affine_quantization_params(NAN, 1.0f, DType::I8).is_err());
}

CPU_TEST(test_calculate_symmetric_quantization_params) {  // algorithms.rs:763-776
    auto [scale, zp] = calculate_symmetric_quantization_params(-2.0f, 1.0f, DType::I8).unwrap();
    CHECK_EQ(scale, 2.0f / 127.0f);
    CHECK_EQ(zp, 0);
    auto [s0, z0] = calculate_symmetric_quantization_params(0.0f, 0.0f, DType::I8).unwrap();
    CHECK_EQ(s0, 1.0f);
    CHECK_EQ(z0, 0);
    auto [su, zu] = calculate_symmetric_quantization_params(-2.0f, 1.0f, DType::U8).unwrap();
    CHECK_EQ(su, 2.0f / 255.0f);  // qmax of the dtype, algorithms.rs:417-419
    CHECK_EQ(zu, 0);
    CHECK(calculate_symmetric_quantization_params(-INFINITY, 1.0f, DType::I8).is_err());
}

CPU_TEST(test_params_match_oracle_on_random_ranges) {
    std::mt19937 g(5);
    std::uniform_real_distribution<float> d(-50.0f, 50.0f);
    for (int i = 0; i < 2000; ++i) {
        float a = d(g), b = d(g);
        if (a > b) std::swap(a, b);
        for (int dt = 0; dt < 2; ++dt) {
            const DType dtype = dt ? DType::U8 : DType::I8;
            float s;
            int32_t z;
            CHECK_EQ(tq_calculate_affine_params(a, b, dt, &s, &z), 0);
            auto p = calculate_affine_quantization_params(a, b, dtype).unwrap();
            CHECK_EQ(p.first, s);
            CHECK_EQ(p.second, z);
            CHECK_EQ(tq_calculate_symmetric_params(a, b, dt, &s, &z), 0);
            auto q = calculate_symmetric_quantization_params(a, b, dtype).unwrap();
            CHECK_EQ(q.first, s);
            CHECK_EQ(q.second, z);
            bq::QuantizationParams bp;
            bp.dtype = dt ? bq::QuantizedDType::UInt8 : bq::QuantizedDType::Int8;
            bp.scheme = bq::QuantizationScheme::Asymmetric;
            CHECK(bp.from_statistics(a, b).is_ok());
            CHECK_EQ(tq_backend_params_asymmetric(a, b, dt ? 0 : -128, dt ? 255 : 127, &s, &z), 0);
            CHECK_EQ(bp.scale[0], s);
            CHECK_EQ(bp.zero_point[0], z);
            bp.scheme = bq::QuantizationScheme::Symmetric;
            CHECK(bp.from_statistics(a, b).is_ok());
            CHECK_EQ(tq_backend_params_symmetric(a, b, dt ? 0 : -128, dt ? 255 : 127, &s, &z), 0);
            CHECK_EQ(bp.scale[0], s);
            CHECK_EQ(bp.zero_point[0], z);
        }
    }
}

CPU_TEST(test_get_dtype_range) {  // algorithms.rs:779-784
    CHECK(get_dtype_range(DType::I8) == std::make_pair(-128, 127));
    CHECK(get_dtype_range(DType::U8) == std::make_pair(0, 255));
    CHECK(get_dtype_range(DType::I16) == std::make_pair(-32768, 32767));
}

CPU_TEST(test_quant_config) {  // config.rs:158-409
    CHECK(QuantConfig::int8().validate().is_ok());
    CHECK(QuantConfig::int8().scheme == QScheme::PerTensorAffine);
    CHECK(QuantConfig::int8().get_qint_range() == std::make_pair(-128, 127));
    CHECK(QuantConfig::uint8().get_qint_range() == std::make_pair(0, 255));
    CHECK(QuantConfig::int8().with_reduce_range(ReduceRange::Reduce).get_qint_range() == std::make_pair(-63, 63));
    QuantConfig c;
    c.scheme = QScheme::PerChannelSymmetric;
    CHECK(c.validate().is_err());  // no channel axis
    CHECK(QuantConfig::int8().with_scheme(QScheme::PerChannelSymmetric).validate().is_ok());
    CHECK(*QuantConfig::int8().with_scheme(QScheme::PerChannelSymmetric).ch_axis == 0);
    c = QuantConfig::int8();
    c.eps = 0.0f;
    CHECK(c.validate().is_err());
    c = QuantConfig::int8();
    c.averaging_constant = 1.0f;
    CHECK(c.validate().is_err());
    c = QuantConfig::int8().with_scheme(QScheme::MixedPrecision);
    CHECK(c.validate().is_err());  // needs a KL / entropy observer
}

CPU_TEST(test_error_cases_before_the_device) {  // algorithms.rs:876-893, simd_ops.rs:538-552
    auto tensor = tensor_1d({1.0f, 2.0f}).unwrap();
    auto r = quantize_per_tensor_affine(tensor, -1.0f, 0);
    CHECK(r.is_err());
    CHECK(r.unwrap_err().kind == TorshError::InvalidArgument);
    CHECK_EQ(r.unwrap_err().message, std::string("Scale must be positive"));
    CHECK(dequantize_per_tensor_affine(tensor, 0.0f, 0).is_err());
    CHECK(quantize_per_tensor_affine_i8(tensor, 0.0f, 0).is_err());
    auto empty = tensor_1d({}).unwrap();
    auto e = quantize_tensor_auto(empty, DType::I8, QScheme::PerTensorAffine);
    CHECK(e.is_err());
    CHECK_EQ(e.unwrap_err().message, std::string("Cannot quantize empty tensor"));
    std::vector<float> in{1.0f, 2.0f}, out(1);
    CHECK(quantize_per_tensor_affine_simd(in, 0.1f, 0, out).is_err());  // length mismatch
    out.resize(2);
    CHECK(quantize_per_tensor_affine_simd(in, -0.1f, 0, out).is_err());
    CHECK(dequantize_per_tensor_affine_simd(in, 0.0f, 0, out).is_err());
    CHECK(find_min_max_simd({}).is_err());
    auto t3 = Tensor::from_data(std::vector<float>(24, 1.0f), {2, 3, 4}).unwrap();
    auto ax = quantize_per_channel_auto(t3, 3, DType::I8, QScheme::PerChannelSymmetric);
    CHECK(ax.is_err());
    CHECK_EQ(ax.unwrap_err().message, std::string("Axis out of bounds"));
    CHECK(quantize_per_channel_auto(t3, 0, DType::I8, QScheme::PerTensorAffine).is_err());
    CHECK(Tensor::from_data({1.0f, 2.0f}, {3}).is_err());
    QuantConfig bad;
    bad.scheme = QScheme::PerChannelAffine;
    CHECK(quantize_with_config(tensor, bad).is_err());
}

CPU_TEST(test_backend_params_and_tensor) {  // params.rs / tensor.rs tests
    auto p = bq::QuantizationParams{};
    CHECK(p.dtype == bq::QuantizedDType::UInt8 && p.scale[0] == 1.0f && p.zero_point[0] == 0);
    CHECK(bq::QuantizationParams::int8_symmetric().validate().is_ok());
    CHECK(bq::QuantizationParams::uint8_asymmetric().zero_point[0] == 128);
    auto bad = bq::QuantizationParams::int8_symmetric();
    bad.zero_point[0] = 3;
    CHECK(bad.validate().is_err());
    bad = bq::QuantizationParams::int8_symmetric();
    bad.scale[0] = 0.0f;
    CHECK(bad.validate().is_err());
    bad = bq::QuantizationParams::uint8_asymmetric();
    bad.zero_point[0] = 300;
    CHECK(bad.validate().is_err());
    CHECK(bq::QuantizationParams::channel_wise(1, bq::QuantizedDType::Int8).validate().is_err());
    CHECK(bq::QuantizationParams::channel_wise(4, bq::QuantizedDType::Int8).validate().is_ok());
    auto u = bq::QuantizationParams::uint8_asymmetric();
    CHECK(u.from_statistics(2.0f, 1.0f).is_err());
    CHECK(u.from_statistics(0.0f, INFINITY).is_err());
    CHECK(u.from_statistics(-1.0f, 1.0f).is_ok());
    CHECK_EQ(u.scale[0], 2.0f / 255.0f);
    CHECK(u.zero_point[0] == 127 || u.zero_point[0] == 128);
    CHECK(u.from_statistics(3.0f, 3.0f).is_ok());
    CHECK(u.scale[0] == 1.0f && u.zero_point[0] == 0);
    auto s = bq::QuantizationParams::int8_symmetric();
    CHECK(s.from_statistics(-2.0f, 1.0f).is_ok());
    CHECK_EQ(s.scale[0], 4.0f / 255.0f);  // 2*max_range/(qmax-qmin), params.rs:331-337
    CHECK(bq::QuantizedTensor::from_data(std::vector<uint8_t>(5), {2, 3}, bq::QuantizationParams{}).is_err());
    CHECK(bq::QuantizedTensor::from_data(std::vector<uint8_t>(6), {2, 3}, bq::QuantizationParams{}).is_ok());
    bq::HipQuantizationOps ops;
    auto a = bq::QuantizedTensor::from_data(std::vector<uint8_t>(6), {2, 3}, bq::QuantizationParams::int8_symmetric()).unwrap();
    auto b = bq::QuantizedTensor::from_data(std::vector<uint8_t>(8), {4, 2}, bq::QuantizationParams::int8_symmetric()).unwrap();
    CHECK(ops.qmatmul(a, b).is_err());            // K mismatch
    CHECK(ops.vnni_qmatmul_int8(a, b).is_err());
    CHECK(ops.vnni_qmatmul_int8(a, b).unwrap_err().kind == TorshError::BackendError);
    auto v = bq::QuantizedTensor::from_data(std::vector<uint8_t>(6), {6}, bq::QuantizationParams::int8_symmetric()).unwrap();
    CHECK(ops.qmatmul(v, b).is_err());            // not 2D
    CHECK(ops.qconv2d(a, b, nullptr, {1, 1}, {0, 0}).is_err());
    CHECK(ops.calibrate({}, bq::QuantizedDType::UInt8).is_err());
    CHECK(ops.quantize_f32({}, bq::QuantizationParams::int8_symmetric()).unwrap().empty());
    CHECK(ops.quantize_f32({1.0f}, bad).is_err());
    CHECK(ops.qadd(a, b).unwrap_err().kind == TorshError::InvalidArgument);  // shape mismatch, before the device
}

CPU_TEST(test_module_shapes_before_the_device) {
    nn::Linear lin(4, 3, true);
    CHECK(lin.parameters().count("weight") == 1 && lin.parameters().count("bias") == 1);
    CHECK(lin.parameters().at("weight").shape().dims() == (std::vector<size_t>{4, 3}));
    CHECK(lin.set_weight(Tensor::from_data(std::vector<float>(12, 0.f), {3, 4}).unwrap()).is_err());
    CHECK(lin.training());
    lin.eval();
    CHECK(!lin.training());
    auto w1 = tensor_1d({1.0f, 2.0f}).unwrap();
    CHECK(nn::QuantizedLinear::from_weight_nk(w1, nullptr).is_err());
    CHECK(nn::QuantizedConv2d::from_weight(w1, nullptr, {1, 1}, {0, 0}, 0.1f, 0).is_err());
    auto w4 = Tensor::from_data(std::vector<float>(2 * 3 * 1 * 1, 0.5f), {2, 3, 1, 1}).unwrap();
    CHECK(nn::QuantizedConv2d::from_weight(w4, nullptr, {1, 1}, {0, 0}, 0.0f, 0).is_err());
    CHECK(nn::QuantizedConv2d::from_weight(w4, nullptr, {0, 1}, {0, 0}, 0.1f, 0).is_err());
}

// ---------------------------------------------------------------- the reference's tests, on the device

GPU_TEST(test_quantize_per_tensor_affine) {  // algorithms.rs:787-800
    auto tensor = tensor_1d({1.0f, 2.0f, 3.0f, 4.0f}).unwrap();
    auto [quantized, scale, zero_point] = quantize_per_tensor_affine(tensor, 0.1f, 0).unwrap();
    auto q = quantized.data().unwrap();
    CHECK_EQ(q[0], 10.0f);
    CHECK_EQ(q[1], 20.0f);
    CHECK_EQ(q[2], 30.0f);
    CHECK_EQ(q[3], 40.0f);
    CHECK_EQ(scale, 0.1f);
    CHECK_EQ(zero_point, 0);
    auto [q8, s8, z8] = quantize_per_tensor_affine_i8(tensor, 0.1f, 0).unwrap();  // simd_ops.rs:525-535 values
    CHECK_SAME(q8.as_slice(), (std::vector<int>{10, 20, 30, 40}));
    CHECK_EQ(s8, 0.1f);
    CHECK_EQ(z8, 0);
}

GPU_TEST(test_dequantize_per_tensor_affine) {  // algorithms.rs:803-813
    auto qt = tensor_1d({10.0f, 20.0f, 30.0f, 40.0f}).unwrap();
    auto d = dequantize_per_tensor_affine(qt, 0.1f, 0).unwrap().data().unwrap();
    for (int i = 0; i < 4; ++i) CHECK(std::fabs(d[i] - float(i + 1)) < 1e-6f);
}

GPU_TEST(test_quantize_tensor_auto) {  // algorithms.rs:816-829
    auto tensor = tensor_1d({-1.0f, 0.0f, 1.0f, 2.0f}).unwrap();
    auto [quantized, scale, zp] = quantize_tensor_auto(tensor, DType::I8, QScheme::PerTensorAffine).unwrap();
    CHECK(scale > 0.0f);
    CHECK(zp >= -128 && zp <= 127);
    CHECK_EQ(quantized.data().unwrap().size(), size_t(4));
}

GPU_TEST(test_quantize_with_config) {  // algorithms.rs:832-845
    auto tensor = tensor_1d({1.0f, 2.0f, 3.0f, 4.0f}).unwrap();
    auto result = quantize_with_config(tensor, QuantConfig::int8());
    CHECK(result.is_ok());
    auto [quantized, scale, zp] = result.unwrap();
    CHECK(scale > 0.0f);
    CHECK(zp >= -128 && zp <= 127);
    CHECK(quantized.shape().dims() == tensor.shape().dims());
}

GPU_TEST(test_dequantize) {  // algorithms.rs:847-859
    auto qt = tensor_1d({64.0f, 128.0f, -64.0f, 0.0f}).unwrap();
    auto d = dequantize(qt, 0.5f, 0).unwrap().data().unwrap();
    CHECK(std::fabs(d[0] - 32.0f) < 1e-6f);
    CHECK(std::fabs(d[1] - 64.0f) < 1e-6f);
    CHECK(std::fabs(d[2] + 32.0f) < 1e-6f);
    CHECK(std::fabs(d[3] - 0.0f) < 1e-6f);
}

GPU_TEST(test_quantize_auto) {  // algorithms.rs:862-873
    auto tensor = tensor_1d({0.5f, 1.0f, 1.5f, 2.0f}).unwrap();
    auto result = quantize_auto(tensor, QuantConfig::int8());
    CHECK(result.is_ok());
    CHECK(std::get<1>(result.unwrap()) > 0.0f);
}

GPU_TEST(test_simd_slice_functions) {  // simd_ops.rs:479-511, 570-582
    std::vector<float> in{1.0f, 2.0f, 3.0f, 4.0f}, out(4);
    CHECK(quantize_per_tensor_affine_simd(in, 0.1f, 0, out).is_ok());
    CHECK_SAME(out, (std::vector<float>{10, 20, 30, 40}));
    std::vector<float> deq(4);
    CHECK(dequantize_per_tensor_affine_simd(out, 0.1f, 0, deq).is_ok());
    for (int i = 0; i < 4; ++i) CHECK(std::fabs(deq[i] - in[i]) < 1e-6f);
    auto mm = find_min_max_simd({-1.5f, 0.0f, 2.3f, -0.8f, 4.7f, 1.2f}).unwrap();
    CHECK_EQ(mm.first, -1.5f);
    CHECK_EQ(mm.second, 4.7f);
    std::vector<float> mob{1.0f, 2.0f, 3.0f, 4.0f, -1.0f, -2.0f};
    std::vector<int8_t> q8(6);
    CHECK(quantize_to_int8_simd(mob, 0.1f, 0, q8).is_ok());
    CHECK_SAME(q8, (std::vector<int>{10, 20, 30, 40, -10, -20}));
}

// ---------------------------------------------------------------- parity with the oracle

GPU_TEST(parity_quantize_tensor_auto_and_round_trip) {
    for (size_t n : {size_t(7), size_t(64), size_t(65), size_t(5000), size_t(1 << 18)}) {
        auto x = normal(n, 11 + unsigned(n));
        auto t = tensor_1d(x).unwrap();
        for (int dt = 0; dt < 2; ++dt)
            for (int sch = 0; sch < 2; ++sch) {
                std::vector<float> want(n);
                float s;
                int32_t z;
                CHECK_EQ(tq_quantize_tensor_auto(x.data(), n, dt, sch ? TQ_PER_TENSOR_SYMMETRIC : TQ_PER_TENSOR_AFFINE,
                                                 want.data(), &s, &z), 0);
                auto [q, scale, zp] = quantize_tensor_auto(t, dt ? DType::U8 : DType::I8,
                                                           sch ? QScheme::PerTensorSymmetric : QScheme::PerTensorAffine)
                                          .unwrap();
                CHECK_EQ(scale, s);
                CHECK_EQ(zp, z);
                CHECK_SAME(q.as_slice(), want);
                std::vector<float> back(n);
                CHECK_EQ(tq_dequantize_per_tensor_affine(want.data(), n, s, z, back.data()), 0);
                CHECK_SAME(dequantize(q, scale, zp).unwrap().as_slice(), back);
            }
    }
}

GPU_TEST(parity_quantize_per_channel_auto) {
    const std::vector<size_t> shape{6, 5, 7};
    auto x = normal(6 * 5 * 7, 3);
    auto t = Tensor::from_data(x, shape).unwrap();
    for (size_t axis = 0; axis < 3; ++axis)
        for (int sch = 0; sch < 2; ++sch) {
            std::vector<float> want(x.size()), ws(shape[axis]);
            std::vector<int32_t> wz(shape[axis]);
            CHECK_EQ(tq_quantize_per_channel_auto(x.data(), shape.data(), 3, axis, TQ_DTYPE_I8,
                                                  sch ? TQ_PER_CHANNEL_SYMMETRIC : TQ_PER_CHANNEL_AFFINE, want.data(),
                                                  ws.data(), wz.data()), 0);
            auto [q, s, z] = quantize_per_channel_auto(t, axis, DType::I8,
                                                       sch ? QScheme::PerChannelSymmetric : QScheme::PerChannelAffine)
                                 .unwrap();
            CHECK_SAME(s, ws);
            CHECK_SAME(z, wz);
            CHECK_SAME(q.as_slice(), want);
        }
    auto cfg = QuantConfig::int8().with_scheme(QScheme::PerChannelSymmetric);
    auto [q, s0, z0] = quantize_with_config(t, cfg).unwrap();
    float mn, mx, s_ref;
    int32_t z_ref;
    tq_find_min_max(x.data(), 35, &mn, &mx);  // channel 0 of axis 0 is the first 35 values
    tq_calculate_symmetric_params(mn, mx, TQ_DTYPE_I8, &s_ref, &z_ref);
    CHECK_EQ(s0, s_ref);
    CHECK_EQ(z0, 0);
}

GPU_TEST(parity_backend_quantize_dequantize) {
    bq::HipQuantizationOps ops;
    const size_t n = 4096 + 12;
    auto x = normal(n, 21, 3.0f);
    for (int dt = 0; dt < 2; ++dt) {
        bq::QuantizationParams p = dt ? bq::QuantizationParams::uint8_asymmetric() : bq::QuantizationParams::int8_symmetric();
        if (dt) p.from_statistics(-7.5f, 9.0f).unwrap();
        else p.from_statistics(-9.0f, 9.0f).unwrap();
        std::vector<uint8_t> want(n);
        CHECK_EQ(tq_backend_quantize_f32(x.data(), n, p.scale.data(), p.zero_point.data(), 1, dt ? 0 : -128,
                                         dt ? 255 : 127, want.data()), 0);
        auto got = ops.quantize_f32(x, p).unwrap();
        CHECK_SAME(got, want);
        std::vector<float> back(n);
        CHECK_EQ(tq_backend_dequantize_f32(want.data(), n, p.scale.data(), p.zero_point.data(), 1, dt ? 0 : 1,
                                           back.data()), 0);
        CHECK_SAME(ops.dequantize_f32(got, p).unwrap(), back);
    }
    // channel-wise: contiguous equal chunks
    const size_t ch = 8, m = 8 * 515;
    auto y = normal(m, 22);
    for (int dt = 0; dt < 2; ++dt) {
        auto p = bq::QuantizationParams::channel_wise(ch, dt ? bq::QuantizedDType::UInt8 : bq::QuantizedDType::Int8);
        for (size_t c = 0; c < ch; ++c) {
            p.scale[c] = 0.01f * float(c + 1);
            p.zero_point[c] = dt ? int32_t(100 + c) : int32_t(c) - 4;
        }
        std::vector<uint8_t> want(m);
        CHECK_EQ(tq_backend_quantize_f32(y.data(), m, p.scale.data(), p.zero_point.data(), ch, dt ? 0 : -128,
                                         dt ? 255 : 127, want.data()), 0);
        auto got = ops.quantize_f32(y, p).unwrap();
        CHECK_SAME(got, want);
        std::vector<float> back(m);
        CHECK_EQ(tq_backend_dequantize_f32(want.data(), m, p.scale.data(), p.zero_point.data(), ch, dt ? 0 : 1,
                                           back.data()), 0);
        CHECK_SAME(ops.dequantize_f32(got, p).unwrap(), back);
    }
    auto cal = ops.calibrate({normal(1000, 1), normal(3000, 2, 2.0f)}, bq::QuantizedDType::UInt8).unwrap();
    float mn = INFINITY, mx = -INFINITY;
    for (auto &s : {normal(1000, 1), normal(3000, 2, 2.0f)})
        for (float v : s) mn = std::fmin(mn, v), mx = std::fmax(mx, v);
    float s_ref;
    int32_t z_ref;
    tq_backend_params_asymmetric(mn, mx, 0, 255, &s_ref, &z_ref);
    CHECK_EQ(cal.scale[0], s_ref);
    CHECK_EQ(cal.zero_point[0], z_ref);
}

GPU_TEST(parity_backend_matmul) {
    bq::HipQuantizationOps ops;
    for (auto [m, k, n] : {std::make_tuple(size_t(5), size_t(7), size_t(3)), std::make_tuple(size_t(33), size_t(256), size_t(70)),
                           std::make_tuple(size_t(128), size_t(512), size_t(64))}) {
        std::mt19937 g(unsigned(m * 31 + k));
        std::uniform_int_distribution<int> d(-128, 127);
        std::vector<uint8_t> a(m * k), b(k * n);
        for (auto &v : a) v = uint8_t(int8_t(d(g)));
        for (auto &v : b) v = uint8_t(int8_t(d(g)));
        auto pa = bq::QuantizationParams::int8_symmetric(), pb = bq::QuantizationParams::int8_symmetric();
        pa.scale[0] = 0.031f;
        pb.scale[0] = 0.0007f;
        auto ta = bq::QuantizedTensor::from_data(a, {m, k}, pa).unwrap();
        auto tb = bq::QuantizedTensor::from_data(b, {k, n}, pb).unwrap();
        std::vector<int32_t> acc(m * n);
        std::vector<uint8_t> clamped(m * n);
        CHECK_EQ(tq_backend_matmul_i32(a.data(), b.data(), m, k, n, acc.data(), clamped.data()), 0);
        CHECK_SAME(ops.qmatmul_i32(ta, tb).unwrap(), acc);
        auto v = ops.vnni_qmatmul_int8(ta, tb).unwrap();
        CHECK_SAME(v.data, clamped);
        CHECK(v.shape == (std::vector<size_t>{m, n}));
        CHECK_EQ(v.params.scale[0], pa.scale[0]);
        // qmatmul: acc * (s_a * s_b) -> range -> symmetric params of `a`'s kind -> requantize
        std::vector<float> out_f(m * n);
        const float sab = pa.scale[0] * pb.scale[0];
        float mn = INFINITY, mx = -INFINITY;
        for (size_t i = 0; i < m * n; ++i) {
            out_f[i] = float(acc[i]) * sab;
            mn = std::fmin(mn, out_f[i]);
            mx = std::fmax(mx, out_f[i]);
        }
        float s_out;
        int32_t z_out;
        tq_backend_params_symmetric(mn, mx, -128, 127, &s_out, &z_out);
        std::vector<uint8_t> want(m * n);
        tq_backend_quantize_f32(out_f.data(), m * n, &s_out, &z_out, 1, -128, 127, want.data());
        auto r = ops.qmatmul(ta, tb).unwrap();
        CHECK_EQ(r.params.scale[0], s_out);
        CHECK_EQ(r.params.zero_point[0], 0);
        CHECK_SAME(r.data, want);
        // and against the reference's own f32 loop (dequantize, accumulate in k order): the two
        // differ only by f32 summation error, at most one output step
        std::vector<float> af(m * k), bf(k * n);
        tq_backend_dequantize_f32(a.data(), m * k, pa.scale.data(), pa.zero_point.data(), 1, 1, af.data());
        tq_backend_dequantize_f32(b.data(), k * n, pb.scale.data(), pb.zero_point.data(), 1, 1, bf.data());
        for (size_t i = 0; i < m; ++i)
            for (size_t j = 0; j < n; ++j) {
                float s = 0.0f;
                for (size_t l = 0; l < k; ++l) s += af[i * k + l] * bf[l * n + j];
                CHECK(std::fabs(s - out_f[i * n + j]) <= 1e-4f * std::fmax(1.0f, std::fabs(s)) + 0.51f * s_out);
            }
    }
}

GPU_TEST(parity_backend_qconv2d) {
    bq::HipQuantizationOps ops;
    struct G { size_t nb, c, h, w, oc, k, stride, pad; };
    for (G g : {G{2, 3, 8, 8, 4, 3, 1, 1}, G{1, 128, 7, 7, 16, 3, 1, 1}, G{1, 16, 9, 9, 6, 3, 2, 1}}) {
        auto xf = normal(g.nb * g.c * g.h * g.w, unsigned(g.c), 1.0f, true);
        auto in_p = bq::QuantizationParams::uint8_asymmetric();
        float mn, mx;
        tq_find_min_max(xf.data(), xf.size(), &mn, &mx);
        in_p.from_statistics(mn, mx).unwrap();
        auto xq = ops.quantize_f32(xf, in_p).unwrap();
        const size_t per = g.c * g.k * g.k;
        auto wf = normal(g.oc * per, 77, 0.02f);
        auto w_p = bq::QuantizationParams::channel_wise(g.oc, bq::QuantizedDType::Int8);
        for (size_t o = 0; o < g.oc; ++o) {
            float a = 0.0f;
            for (size_t i = 0; i < per; ++i) a = std::fmax(a, std::fabs(wf[o * per + i]));
            w_p.scale[o] = a / 127.0f;
        }
        auto wq = ops.quantize_f32(wf, w_p).unwrap();
        auto bias_f = normal(g.oc, 5, 0.01f);
        auto b_p = bq::QuantizationParams::int8_symmetric();
        b_p.scale[0] = 0.0005f;
        auto bq8 = ops.quantize_f32(bias_f, b_p).unwrap();
        auto tin = bq::QuantizedTensor::from_data(xq, {g.nb, g.c, g.h, g.w}, in_p).unwrap();
        auto tw = bq::QuantizedTensor::from_data(wq, {g.oc, g.c, g.k, g.k}, w_p).unwrap();
        auto tb = bq::QuantizedTensor::from_data(bq8, {g.oc}, b_p).unwrap();
        const size_t ho = (g.h + 2 * g.pad - g.k) / g.stride + 1, wo = (g.w + 2 * g.pad - g.k) / g.stride + 1;
        std::vector<int32_t> acc(g.nb * g.oc * ho * wo);
        CHECK_EQ(tq_backend_conv2d_i32(xq.data(), 0, in_p.zero_point[0], reinterpret_cast<const int8_t *>(wq.data()), g.nb,
                                       g.c, g.h, g.w, g.oc, g.k, g.k, g.stride, g.stride, g.pad, g.pad, acc.data()), 0);
        std::vector<float> bias_dq(g.oc);
        tq_backend_dequantize_f32(bq8.data(), g.oc, b_p.scale.data(), b_p.zero_point.data(), 1, 1, bias_dq.data());
        std::vector<float> out_f(acc.size());
        mn = INFINITY, mx = -INFINITY;
        for (size_t i = 0; i < acc.size(); ++i) {
            const size_t oc = (i / (ho * wo)) % g.oc;
            out_f[i] = float(acc[i]) * (in_p.scale[0] * w_p.scale[oc]) + bias_dq[oc];
            mn = std::fmin(mn, out_f[i]);
            mx = std::fmax(mx, out_f[i]);
        }
        float s_out;
        int32_t z_out;
        tq_backend_params_asymmetric(mn, mx, 0, 255, &s_out, &z_out);
        std::vector<uint8_t> want(acc.size());
        tq_backend_quantize_f32(out_f.data(), out_f.size(), &s_out, &z_out, 1, 0, 255, want.data());
        auto r = ops.qconv2d(tin, tw, &tb, {g.stride, g.stride}, {g.pad, g.pad}).unwrap();
        CHECK(r.shape == (std::vector<size_t>{g.nb, g.oc, ho, wo}));
        CHECK_EQ(r.params.scale[0], s_out);
        CHECK_EQ(r.params.zero_point[0], z_out);
        CHECK_SAME(r.data, want);
    }
}

GPU_TEST(parity_quantized_linear_module) {
    for (int per_token = 0; per_token < 2; ++per_token) {
        const size_t m = 48, k = 256, n = 96;
        nn::Linear lin(k, n, true);
        auto w_in_out = normal(k * n, 31, 0.02f);
        auto bias = normal(n, 32, 0.01f);
        lin.set_weight(Tensor::from_data(w_in_out, {k, n}).unwrap()).unwrap();
        lin.set_bias(Tensor::from_data(bias, {n}).unwrap()).unwrap();
        auto qlin = nn::QuantizedLinear::from_linear(lin, per_token ? nn::ActivationQuant::PerToken
                                                                    : nn::ActivationQuant::PerTensor)
                        .unwrap();
        auto x = normal(m * k, 33);
        auto y = qlin.forward(Tensor::from_data(x, {4, 12, k}).unwrap()).unwrap();
        CHECK(y.shape().dims() == (std::vector<size_t>{4, 12, n}));
        // oracle composition
        std::vector<float> wnk(n * k);
        for (size_t i = 0; i < k; ++i)
            for (size_t j = 0; j < n; ++j) wnk[j * k + i] = w_in_out[i * n + j];
        const size_t wshape[2] = {n, k};
        std::vector<float> wq_f(n * k), sw(n);
        std::vector<int32_t> wz(n);
        tq_quantize_per_channel_auto(wnk.data(), wshape, 2, 0, TQ_DTYPE_I8, TQ_PER_CHANNEL_SYMMETRIC, wq_f.data(),
                                     sw.data(), wz.data());
        std::vector<int8_t> wq(n * k), aq(m * k);
        for (size_t i = 0; i < n * k; ++i) wq[i] = int8_t(wq_f[i]);
        std::vector<float> sa(per_token ? m : 1), aq_f(m * k);
        if (per_token) {
            const size_t ashape[2] = {m, k};
            std::vector<int32_t> az(m);
            tq_quantize_per_channel_auto(x.data(), ashape, 2, 0, TQ_DTYPE_I8, TQ_PER_CHANNEL_SYMMETRIC, aq_f.data(),
                                         sa.data(), az.data());
        } else {
            int32_t z;
            tq_quantize_tensor_auto(x.data(), m * k, TQ_DTYPE_I8, TQ_PER_TENSOR_SYMMETRIC, aq_f.data(), &sa[0], &z);
        }
        for (size_t i = 0; i < m * k; ++i) aq[i] = int8_t(aq_f[i]);
        std::vector<int32_t> acc(m * n);
        tq_gemm_i8_nk(aq.data(), wq.data(), m, n, k, acc.data());
        std::vector<float> want(m * n);
        tq_linear_dequant_epilogue(acc.data(), m, n, sa.data(), per_token, sw.data(), bias.data(), want.data());
        CHECK_SAME(y.as_slice(), want);
        auto params = qlin.parameters();
        CHECK(params.count("weight") && params.count("bias") && params.count("weight_scale"));
        CHECK_SAME(params.at("weight").as_slice(), wq_f);
        CHECK_SAME(params.at("weight_scale").as_slice(), sw);
        CHECK(qlin.forward(Tensor::from_data(std::vector<float>(10, 0.f), {2, 5}).unwrap()).is_err());
        // Static quantization: a calibrated per-tensor activation scale (MinMax observer over the same
        // data, symmetric int8) replaces the range pass.  Per-token layers refuse it.
        if (per_token) {
            CHECK(qlin.set_static_activation_scale(0.05f).is_err());
        } else {
            quantization::Observer ob(quantization::ObserverType::MinMax);
            CHECK(ob.update(Tensor::from_data(x, {m, k}).unwrap()).is_ok());
            const auto [mn, mx] = ob.get_min_max();
            float s_cal;
            int32_t z_cal;
            tq_calculate_symmetric_params(mn, mx, TQ_DTYPE_I8, &s_cal, &z_cal);
            CHECK(qlin.set_static_activation_scale(s_cal, 1).is_err());
            CHECK(qlin.set_static_activation_scale(s_cal, 0).is_ok());
            CHECK(qlin.static_activation_scale() == s_cal);
            auto ys = qlin.forward(Tensor::from_data(x, {m, k}).unwrap()).unwrap();
            // with the scale of this very tensor the static path reproduces the dynamic one bit for bit
            CHECK_SAME(ys.as_slice(), want);
            // and with another scale it follows the oracle's per-tensor quantize (x * (1/scale) above 64 elements)
            const float s2 = 3.0f / 127.0f;
            CHECK(qlin.set_static_activation_scale(s2).is_ok());
            auto y2 = qlin.forward(Tensor::from_data(x, {m, k}).unwrap()).unwrap();
            std::vector<int8_t> aq2(m * k);
            tq_quantize_to_int8_simd(x.data(), m * k, s2, 0, aq2.data());
            tq_gemm_i8_nk(aq2.data(), wq.data(), m, n, k, acc.data());
            std::vector<float> want2(m * n);
            tq_linear_dequant_epilogue(acc.data(), m, n, &s2, 0, sw.data(), bias.data(), want2.data());
            CHECK_SAME(y2.as_slice(), want2);
            CHECK(qlin.set_static_activation_scale(0.0f).is_ok());  // back to dynamic
            auto y3 = qlin.forward(Tensor::from_data(x, {m, k}).unwrap()).unwrap();
            CHECK_SAME(y3.as_slice(), want);
        }
    }
}

GPU_TEST(parity_quantized_conv2d_module) {
    const size_t nb = 2, c = 128, h = 9, w = 9, oc = 24, k = 3, pad = 1;
    auto wf = normal(oc * c * k * k, 41, 0.02f);
    auto bias = normal(oc, 42, 0.01f);
    auto x = normal(nb * c * h * w, 43, 1.0f, true);
    const float s_out = 0.013f;
    const int32_t zp_out = -3;
    auto bt = Tensor::from_data(bias, {oc}).unwrap();
    auto conv = nn::QuantizedConv2d::from_weight(Tensor::from_data(wf, {oc, c, k, k}).unwrap(), &bt, {1, 1}, {pad, pad},
                                                 s_out, zp_out)
                    .unwrap();
    auto xt = Tensor::from_data(x, {nb, c, h, w}).unwrap();
    auto q = conv.forward_quantized(xt).unwrap();
    // oracle composition
    float mn, mx, s_in;
    int32_t zp_in;
    tq_find_min_max(x.data(), x.size(), &mn, &mx);
    tq_backend_params_asymmetric(mn, mx, 0, 255, &s_in, &zp_in);
    std::vector<uint8_t> xq(x.size());
    tq_backend_quantize_f32(x.data(), x.size(), &s_in, &zp_in, 1, 0, 255, xq.data());
    const size_t wshape[2] = {oc, c * k * k};
    std::vector<float> wq_f(wf.size()), sw(oc);
    std::vector<int32_t> wz(oc);
    tq_quantize_per_channel_auto(wf.data(), wshape, 2, 0, TQ_DTYPE_I8, TQ_PER_CHANNEL_SYMMETRIC, wq_f.data(), sw.data(),
                                 wz.data());
    std::vector<int8_t> wq(wf.size());
    for (size_t i = 0; i < wf.size(); ++i) wq[i] = int8_t(wq_f[i]);
    std::vector<int32_t> acc(nb * oc * h * w);
    tq_backend_conv2d_i32(xq.data(), 0, zp_in, wq.data(), nb, c, h, w, oc, k, k, 1, 1, pad, pad, acc.data());
    std::vector<int8_t> want(acc.size());
    // rows of the [nb*oc, h*w] view cycle through the output channels
    tq_requantize_epilogue(acc.data(), nb * oc, h * w, &s_in, 0, sw.data(), bias.data(), s_out, zp_out, -128, 127, 1, oc,
                           want.data());
    CHECK(q.shape().dims() == (std::vector<size_t>{nb, oc, h, w}));
    CHECK_SAME(q.as_slice(), want);
    auto y = conv.forward(xt).unwrap();
    for (size_t i = 0; i < want.size(); ++i) CHECK_EQ(y.as_slice()[i], float(int(want[i]) - zp_out) * s_out);
    CHECK(conv.forward(Tensor::from_data(std::vector<float>(6, 0.f), {2, 3}).unwrap()).is_err());
    CHECK(conv.forward(Tensor::from_data(std::vector<float>(2 * 3 * 4 * 4, 0.f), {2, 3, 4, 4}).unwrap()).is_err());
}


// ---- calibration, metrics, model quantizer, persistence ----------------------------------------

bool close_rel(double a, double b, double rel, double abs_tol = 1e-9) {
    if (std::isinf(a) || std::isinf(b)) return a == b;
    return std::fabs(a - b) <= abs_tol + rel * std::fabs(b);
}

CPU_TEST(test_observer_creation_and_host_logic) {  // observers.rs:577-591, 654-662, 706-716
    CHECK(Observer::min_max().observer_type() == ObserverType::MinMax);
    Observer h = Observer::histogram_with_bins(128);
    CHECK(h.observer_type() == ObserverType::Histogram);
    CHECK_EQ(h.num_bins(), size_t(128));
    Observer p = Observer::percentile_with_value(95.0f);
    CHECK(p.observer_type() == ObserverType::Percentile);
    CHECK_EQ(p.percentile_value(), 95.0f);
    auto [cleaned, removed] = Observer::min_max().detect_outliers({1.f, 2.f, 3.f, 4.f, 5.f, 100.f}, 1.5f);
    CHECK(removed > 0 && cleaned.size() < 6);
    CHECK(std::find(cleaned.begin(), cleaned.end(), 100.0f) == cleaned.end());
    CHECK(Observer::min_max().calculate_qparams(DType::F32).is_err());
    // an empty batch is counted and touches nothing else (observers.rs:694-703)
    Observer e = Observer::min_max();
    CHECK(e.update(Tensor::from_data({}, {0}).unwrap()).is_ok());
    CHECK_EQ(e.num_batches(), size_t(1));
    CHECK(std::isinf(e.get_min_max().first) && e.get_min_max().first > 0);
}

CPU_TEST(test_config_json_round_trip) {  // utils.rs:322-347
    QuantConfig c = QuantConfig::per_channel(1).with_reduce_range(ReduceRange::Reduce);
    c.dtype = DType::U8;
    c.observer_type = ObserverType::Histogram;
    c.qint_min = -5;
    c.eps = 1e-6f;
    c.averaging_constant = 0.05f;
    const std::string json = export_config_to_json(c).unwrap();
    CHECK(json.find("\"scheme\": \"PerChannelAffine\"") != std::string::npos);
    CHECK(json.find("\"qint_max\": null") != std::string::npos);
    CHECK(json.find("\"ch_axis\": 1") != std::string::npos);
    const QuantConfig d = import_config_from_json(json).unwrap();
    CHECK(d.dtype == c.dtype && d.scheme == c.scheme && d.observer_type == c.observer_type);
    CHECK(d.reduce_range == c.reduce_range && d.backend == c.backend && d.enable_fake_quant == c.enable_fake_quant);
    CHECK(d.qint_min == c.qint_min && !d.qint_max && d.ch_axis == c.ch_axis && !d.group_size);
    CHECK_EQ(d.eps, c.eps);
    CHECK_EQ(d.averaging_constant, c.averaging_constant);
    // compact single-line form, as serde_json::to_string writes it
    const char *compact =
        "{\"dtype\":\"I8\",\"scheme\":\"PerTensorSymmetric\",\"enable_fake_quant\":true,\"observer_type\":\"MinMax\","
        "\"backend\":\"Native\",\"reduce_range\":\"None\",\"qint_min\":null,\"qint_max\":null,\"eps\":1e-8,"
        "\"averaging_constant\":0.01,\"ch_axis\":null,\"group_size\":64}";
    const QuantConfig g = import_config_from_json(compact).unwrap();
    CHECK(g.scheme == QScheme::PerTensorSymmetric && g.enable_fake_quant && g.group_size == size_t(64));
    CHECK(import_config_from_json("{\"dtype\":\"I8\"}").is_err());          // missing fields
    CHECK(import_config_from_json("not json").is_err());
    CHECK(import_config_from_json(std::string(compact).replace(10, 2, "Q9")).is_err());  // unknown variant
}

CPU_TEST(test_weight_file_round_trip_and_corruption) {
    QuantizedWeights w;
    w.kind = QuantizedWeights::Conv2d;
    w.dims = {3, 2, 2, 2};
    for (int i = 0; i < 24; ++i) w.weight.push_back(static_cast<int8_t>(i * 11 - 128));
    w.scales = {0.5f, 0.25f, 1e-3f};
    w.bias = {1.f, -2.f, 3.f};
    const std::string path = "/tmp/torsh_hipq_weights_test.bin";
    CHECK(save_quantized_weights(w, path).is_ok());
    const QuantizedWeights r = load_quantized_weights(path).unwrap();
    CHECK(r.kind == w.kind && r.dims == w.dims && r.weight == w.weight && r.scales == w.scales && r.bias == w.bias);
    // flipped payload byte -> checksum error; truncated file -> length error; wrong sections -> validate error
    std::vector<char> bytes;
    {
        std::ifstream f(path, std::ios::binary);
        bytes.assign((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    }
    CHECK(bytes.size() % 256 == 0 && bytes.size() >= 1024);
    auto write = [&](const std::vector<char> &b) {
        std::ofstream f(path, std::ios::binary | std::ios::trunc);
        f.write(b.data(), static_cast<std::streamsize>(b.size()));
    };
    auto flipped = bytes;
    flipped[256 + 5] ^= 1;
    write(flipped);
    CHECK(load_quantized_weights(path).is_err());
    CHECK(load_quantized_weights(path).unwrap_err().message.find("checksum") != std::string::npos);
    write(std::vector<char>(bytes.begin(), bytes.begin() + 512));
    CHECK(load_quantized_weights(path).is_err());
    write(std::vector<char>(300, 'x'));
    CHECK(load_quantized_weights(path).is_err());
    // a damaged header field is caught by the checksum, which covers the header
    auto header = bytes;
    header[16] ^= 4;  // dims[0]
    write(header);
    CHECK(load_quantized_weights(path).unwrap_err().message.find("checksum") != std::string::npos);
    // a crafted header with a consistent checksum: offsets and dims near 2^64 must not wrap the bounds checks
    auto craft = [&](size_t field_off, uint64_t value) {
        auto b = bytes;
        std::memcpy(b.data() + field_off, &value, 8);
        std::memset(b.data() + 80, 0, 8);
        const uint64_t sum = torsh::quantization::detail::fnv1a64(reinterpret_cast<const unsigned char *>(b.data()), b.size());
        std::memcpy(b.data() + 80, &sum, 8);
        write(b);
        return load_quantized_weights(path);
    };
    CHECK(craft(48, ~uint64_t(0) - 15).unwrap_err().message.find("section outside") != std::string::npos);  // weights
    CHECK(craft(56, ~uint64_t(0) - 3).unwrap_err().message.find("section outside") != std::string::npos);   // scales
    CHECK(craft(64, uint64_t(1) << 63).unwrap_err().message.find("section outside") != std::string::npos);  // bias
    CHECK(craft(48, 8).is_err());                                                                          // inside the header
    CHECK(craft(16, uint64_t(1) << 62).unwrap_err().message.find("implausible") != std::string::npos);      // rows
    CHECK(craft(24, ~uint64_t(0)).unwrap_err().message.find("implausible") != std::string::npos);           // a dim
    QuantizedWeights bad = w;
    bad.scales.pop_back();
    CHECK(save_quantized_weights(bad, path).is_err());
    std::remove(path.c_str());
    CHECK(load_quantized_weights(path).is_err());
}

CPU_TEST(test_model_quantizer_scalar_logic) {  // crates/torsh-models/src/quantization.rs:726-822
    mq::ModelQuantizer quantizer{mq::QuantizationConfig{}};
    const mq::QuantizationParams p = quantizer.calculate_quantization_params(-1.0f, 1.0f, mq::QuantizationDType::Int8);
    CHECK(p.scale > 0.0f && p.zero_point >= -128 && p.zero_point <= 127);
    CHECK(quantizer.get_quantization_range(mq::QuantizationDType::Int8) == std::make_pair(-128, 127));
    CHECK(quantizer.get_quantization_range(mq::QuantizationDType::Uint8) == std::make_pair(0, 255));
    std::mt19937 g(3);
    std::uniform_real_distribution<float> d(-50.f, 50.f);
    for (int i = 0; i < 2000; ++i) {
        float a = d(g), b = i % 17 == 0 ? a : d(g);
        if (a > b) std::swap(a, b);
        const auto got = quantizer.calculate_quantization_params(a, b, i % 2 ? mq::QuantizationDType::Int8
                                                                             : mq::QuantizationDType::Uint8);
        float s, amin, amax;
        int32_t z;
        tq_model_calculate_quantization_params(a, b, i % 2 ? -128 : 0, i % 2 ? 127 : 255, &s, &z, &amin, &amax);
        CHECK(got.scale == s && got.zero_point == z && got.min_val == amin && got.max_val == amax);
    }
    const auto [ratio, savings] = mq::quantization_utils::calculate_memory_savings(1000, 250);
    CHECK_EQ(ratio, 4.0);
    CHECK_EQ(savings, 75.0);
    CHECK(mq::quantization_utils::estimate_inference_speedup(mq::QuantizationDType::Int8, "cpu") > 1.0);
    CHECK(mq::quantization_utils::post_training_quantization_config(mq::QuantizationDType::Int8).strategy.kind ==
          mq::QuantizationStrategyKind::PostTraining);
    // layer filter by substring and by type (quantization.rs:411-457)
    std::map<std::string, Tensor> params;
    for (const char *n : {"encoder.fc1.weight", "encoder.conv.weight", "embed.weight", "attn.q.weight"})
        params.emplace(n, Tensor::from_data({1.f}, {1}).unwrap());
    mq::QuantizationConfig cfg;
    cfg.layer_filter.kind = mq::LayerQuantizationFilter::Exclude;
    cfg.layer_filter.names = {"embed"};
    CHECK_EQ(mq::ModelQuantizer{cfg}.filter_parameters(params).size(), size_t(3));
    cfg.layer_filter.kind = mq::LayerQuantizationFilter::LayerTypes;
    cfg.layer_filter.types = {mq::QuantizableLayerType::Linear, mq::QuantizableLayerType::Attention};
    const auto kept = mq::ModelQuantizer{cfg}.filter_parameters(params);
    CHECK(kept.size() == 2 && kept.count("encoder.fc1.weight") && kept.count("attn.q.weight"));
}

GPU_TEST(test_calculate_quantization_metrics) {  // metrics.rs:588-621
    const Tensor original = tensor_1d({1.0f, 2.0f, 3.0f, 4.0f}).unwrap();
    const Tensor quantized = tensor_1d({1.1f, 2.1f, 2.9f, 3.9f}).unwrap();
    const QuantizationMetrics m = calculate_quantization_metrics(original, quantized, 32, 8).unwrap();
    CHECK(m.mse > 0.0f && m.mse < 1.0f && m.mae > 0.0f && m.mae < 1.0f && m.psnr > 0.0f && m.snr > 0.0f);
    CHECK(m.max_error >= 0.0f && m.zero_error_percentage >= 0.0f && m.zero_error_percentage <= 100.0f);
    CHECK(m.cosine_similarity > 0.8f);
    CHECK_EQ(m.compression_ratio, 4.0f);
    const QuantizationMetrics p = calculate_quantization_metrics(original, original, 32, 16).unwrap();
    CHECK(p.mse == 0.0f && p.mae == 0.0f && p.max_error == 0.0f && p.zero_error_percentage == 100.0f);
    CHECK(std::fabs(p.cosine_similarity - 1.0f) < 1e-6f && std::isinf(p.psnr) && std::isinf(p.snr));
    CHECK_EQ(p.compression_ratio, 2.0f);
    CHECK(calculate_quantization_metrics(original, tensor_1d({1.f, 2.f}).unwrap(), 32, 8).is_err());
    const Tensor empty = Tensor::from_data({}, {0}).unwrap();
    CHECK_EQ(calculate_quantization_metrics(empty, empty, 32, 8).unwrap().zero_error_percentage, 100.0f);
}

GPU_TEST(test_compare_quantization_configs) {  // metrics.rs:623-661
    const Tensor tensor = tensor_1d({1.0f, 2.0f, 3.0f, 4.0f, 5.0f}).unwrap();
    const std::vector<QuantConfig> configs{QuantConfig::int8(), QuantConfig::binary(), QuantConfig::ternary()};
    const auto results = compare_quantization_configs(tensor, configs).unwrap();
    CHECK_EQ(results.size(), size_t(3));
    for (const auto &r : results) {
        bool known = false;
        for (const auto &c : configs) known = known || c.scheme == r.config.scheme;
        CHECK(known && r.seconds >= 0.0);
        if (std::isfinite(r.metrics.psnr))
            CHECK(r.metrics.psnr > 0.0f && r.metrics.compression_ratio >= 1.0f && r.metrics.mae >= 0.0f &&
                  r.metrics.mse >= 0.0f);
    }
    for (size_t i = 1; i < results.size(); ++i) {
        const float a = results[i - 1].metrics.psnr, b = results[i].metrics.psnr;
        if (std::isfinite(a) && std::isfinite(b)) CHECK(a >= b);
    }
    // a configuration that cannot be quantized gets the worst-case record and sorts last (metrics.rs:231-245)
    QuantConfig mixed;
    mixed.scheme = QScheme::MixedPrecision;
    const auto with_bad = compare_quantization_configs(tensor, {mixed, QuantConfig::int8()}).unwrap();
    CHECK(with_bad.back().config.scheme == QScheme::MixedPrecision && std::isinf(with_bad.back().metrics.mse));
    CHECK(with_bad.back().metrics.psnr < 0 && with_bad.back().metrics.zero_error_percentage == 0.0f);
}

GPU_TEST(test_auto_calibrate_quantization) {  // metrics.rs:663-686
    const Tensor t1 = tensor_1d({1.0f, 2.0f, 3.0f, 4.0f}).unwrap(), t2 = tensor_1d({2.0f, 3.0f, 4.0f, 5.0f}).unwrap(),
                 t3 = tensor_1d({0.5f, 1.5f, 2.5f, 3.5f}).unwrap();
    const std::vector<const Tensor *> calibration{&t1, &t2, &t3};
    const auto result = auto_calibrate_quantization(calibration, 20.0f, 10.0f);
    CHECK(result.is_ok());
    CHECK(result.unwrap().validate().is_ok());
    CHECK(auto_calibrate_quantization(calibration, 100.0f, 1.1f).is_ok());  // impossible thresholds still yield a config
    const auto none = auto_calibrate_quantization({}, 20.0f, 10.0f);
    CHECK(none.is_err());
    CHECK_EQ(none.unwrap_err().message, std::string("No calibration tensors provided"));
    // the score rule, recomputed from compare_quantization_configs on one tensor: every candidate has
    // compression ratio 4 (int8 carrier), so with both thresholds met the highest PSNR wins
    const Tensor big = Tensor::from_data(normal(64 * 32, 97, 1.0f), {64, 32}).unwrap();
    const QuantConfig chosen = auto_calibrate_quantization({&big}, 10.0f, 10.0f).unwrap();
    const std::vector<QuantConfig> candidates{
        QuantConfig::int8(),           QuantConfig::int8().with_observer(ObserverType::Histogram),
        QuantConfig::per_channel(0),   QuantConfig::per_channel(1),
        QuantConfig::group_wise(0, 8), QuantConfig::group_wise(1, 16),
        QuantConfig::int4(),           QuantConfig::ternary()};
    float best = -INFINITY;
    size_t best_i = 0;
    for (size_t i = 0; i < candidates.size(); ++i) {
        const auto cmp = compare_quantization_configs(big, {candidates[i]}).unwrap();
        const QuantizationMetrics &m = cmp.front().metrics;
        if (!std::isfinite(m.psnr)) continue;
        const float score = (m.psnr >= 10.0f && m.compression_ratio <= 10.0f) ? m.compression_ratio + m.psnr / 100.0f
                                                                              : m.psnr / m.compression_ratio;
        if (score > best) best = score, best_i = i;
    }
    CHECK(chosen.scheme == candidates[best_i].scheme && chosen.observer_type == candidates[best_i].observer_type);
    CHECK(chosen.ch_axis == candidates[best_i].ch_axis && chosen.group_size == candidates[best_i].group_size);
}

GPU_TEST(parity_metrics_and_compare_configs) {
    const std::vector<float> x = normal(200003, 31, 1.7f);
    const Tensor tx = tensor_1d(x).unwrap();
    for (QScheme scheme : {QScheme::PerTensorAffine, QScheme::PerTensorSymmetric}) {
        const QuantConfig cfg = QuantConfig::int8().with_scheme(scheme);
        const auto res = compare_quantization_configs(tx, {cfg}).unwrap();
        // oracle: quantize_tensor_auto -> dequantize -> metrics
        std::vector<float> q(x.size()), y(x.size());
        float s;
        int32_t z;
        CHECK_EQ(tq_quantize_tensor_auto(x.data(), x.size(), TQ_DTYPE_I8,
                                         scheme == QScheme::PerTensorAffine ? TQ_PER_TENSOR_AFFINE : TQ_PER_TENSOR_SYMMETRIC,
                                         q.data(), &s, &z), 0);
        CHECK_EQ(tq_dequantize_per_tensor_affine(q.data(), q.size(), s, z, y.data()), 0);
        double want[8];
        tq_calculate_quantization_metrics_f64(x.data(), y.data(), x.size(), 32, 8, want);
        const QuantizationMetrics &m = res[0].metrics;
        CHECK(close_rel(m.mse, want[0], 1e-6) && close_rel(m.psnr, want[1], 1e-6) && close_rel(m.snr, want[2], 1e-6));
        CHECK(close_rel(m.mae, want[3], 1e-6) && m.max_error == static_cast<float>(want[4]));
        CHECK(m.zero_error_percentage == static_cast<float>(want[5]) && close_rel(m.cosine_similarity, want[6], 1e-6));
        // and the two-tensor form on the materialised image
        const QuantizationMetrics two = calculate_quantization_metrics(tx, tensor_1d(y).unwrap(), 32, 8).unwrap();
        CHECK(close_rel(two.mse, m.mse, 1e-6) && two.max_error == m.max_error);
    }
}

GPU_TEST(test_observers) {  // observers.rs:594-651, 665-703
    Observer mm = Observer::min_max();
    CHECK(mm.update(tensor_1d({1.0f, 2.0f, 3.0f, 4.0f}).unwrap()).is_ok());
    CHECK(mm.get_min_max() == std::make_pair(1.0f, 4.0f));
    CHECK(mm.update(tensor_1d({0.5f, 5.0f}).unwrap()).is_ok());
    CHECK(mm.get_min_max() == std::make_pair(0.5f, 5.0f));
    Observer h = Observer::histogram_with_bins(10);
    CHECK(h.update(tensor_1d({1.0f, 2.0f, 3.0f, 4.0f, 5.0f}).unwrap()).is_ok());
    auto stats = h.get_statistics();
    CHECK_EQ(stats.at("total_samples"), 5.0f);
    CHECK_EQ(stats.at("num_bins"), 10.0f);
    Observer p = Observer::percentile_with_value(90.0f);
    std::vector<float> ramp(100);
    for (int i = 0; i < 100; ++i) ramp[i] = static_cast<float>(i);
    CHECK(p.update(tensor_1d(ramp).unwrap()).is_ok());
    CHECK_EQ(p.get_statistics().at("total_values"), 100.0f);
    CHECK_EQ(p.get_statistics().at("percentile"), 90.0f);
    Observer q = Observer::min_max();
    CHECK(q.update(tensor_1d({-2.0f, -1.0f, 0.0f, 1.0f, 2.0f}).unwrap()).is_ok());
    const auto qp = q.calculate_qparams(DType::I8).unwrap();
    CHECK(qp.first > 0.0f && qp.second >= -128 && qp.second <= 127);
    Observer r = Observer::min_max();
    CHECK(r.update(tensor_1d({1.0f, 2.0f, 3.0f}).unwrap()).is_ok());
    CHECK_EQ(r.num_batches(), size_t(1));
    r.reset();
    CHECK_EQ(r.num_batches(), size_t(0));
    CHECK(std::isinf(r.get_min_max().first) && r.get_min_max().first > 0 && r.get_min_max().second < 0);
    Observer bad = Observer::min_max();
    auto err = bad.update(tensor_1d({NAN, 1.0f, 2.0f}).unwrap());
    CHECK(err.is_err() && err.unwrap_err().kind == TorshError::InvalidArgument);
    CHECK_EQ(bad.num_batches(), size_t(1));
}

GPU_TEST(parity_observers_against_the_oracle) {
    struct Kind {
        ObserverType type;
        int tq;
    };
    for (Kind k : {Kind{ObserverType::MinMax, TQ_OBS_MINMAX}, Kind{ObserverType::MovingAverage, TQ_OBS_MOVING_AVERAGE},
                   Kind{ObserverType::Histogram, TQ_OBS_HISTOGRAM}, Kind{ObserverType::Percentile, TQ_OBS_PERCENTILE}}) {
        Observer ob(k.type);
        tq_observer *ref = tq_observer_new(k.tq, 0, 0.0f);
        for (unsigned b = 0; b < 4; ++b) {
            const std::vector<float> x = normal(60000 + 1111 * b, 900 + b, 0.5f + b);
            CHECK(ob.update(tensor_1d(x).unwrap()).is_ok());
            CHECK_EQ(tq_observer_update(ref, x.data(), x.size()), 0);
            float mn, mx;
            tq_observer_get_min_max(ref, &mn, &mx);
            CHECK(ob.get_min_max() == std::make_pair(mn, mx));
            for (DType dt : {DType::I8, DType::U8}) {
                float s;
                int32_t z;
                CHECK_EQ(tq_observer_calculate_qparams(ref, dt == DType::I8 ? 0 : 1, &s, &z), 0);
                const auto got = ob.calculate_qparams(dt).unwrap();
                CHECK(got.first == s && got.second == z);
            }
        }
        float a, b;
        tq_observer_get_avg(ref, &a, &b);
        CHECK(ob.get_moving_average() == std::make_pair(a, b));
        tq_observer_get_hist_range(ref, &a, &b);
        CHECK(ob.get_histogram_bounds() == std::make_pair(a, b));
        if (k.type == ObserverType::Histogram) {
            const uint64_t *h = tq_observer_histogram(ref);
            check_same(ob.histogram_counts(), std::vector<uint64_t>(h, h + 256), __LINE__);
            tq_observer_histogram_range(ref, &a, &b);
            CHECK(ob.calculate_histogram_range() == std::make_pair(a, b));
        }
        if (k.type == ObserverType::Percentile) {
            const float *v = tq_observer_values(ref);
            check_same(ob.values(), std::vector<float>(v, v + tq_observer_num_values(ref)), __LINE__);
            CHECK(ob.values().size() < 60000u * 4 + 7000);  // sampling kicked in above 100k values
            tq_observer_percentile_range(ref, &a, &b);
            CHECK(ob.calculate_percentile_range() == std::make_pair(a, b));
        }
        tq_observer_free(ref);
    }
}

GPU_TEST(parity_quantize_batch_consistent) {  // utils.rs:153-180
    const std::vector<float> a = normal(5000, 41, 1.0f), b = normal(300, 42, 3.0f), c = normal(70, 43, 0.2f);
    const Tensor ta = tensor_1d(a).unwrap(), tb = tensor_1d(b).unwrap(), tc = tensor_1d(c).unwrap();
    const auto res = quantize_batch_consistent({&ta, &tb, &tc}, QuantConfig::int8()).unwrap();
    CHECK_EQ(res.size(), size_t(3));
    tq_observer *ref = tq_observer_new(TQ_OBS_MINMAX, 0, 0.0f);
    for (const auto *v : {&a, &b, &c}) tq_observer_update(ref, v->data(), v->size());
    float s;
    int32_t z;
    tq_observer_calculate_qparams(ref, 0, &s, &z);
    tq_observer_free(ref);
    const std::vector<float> *inputs[3] = {&a, &b, &c};
    for (int i = 0; i < 3; ++i) {
        CHECK(std::get<1>(res[i]) == s && std::get<2>(res[i]) == z);
        std::vector<float> want(inputs[i]->size());
        CHECK_EQ(tq_quantize_per_tensor_affine(inputs[i]->data(), want.size(), s, z, want.data()), 0);
        check_same(std::get<0>(res[i]).as_slice(), want, __LINE__);
    }
    CHECK(quantize_batch_consistent({}, QuantConfig::int8()).unwrap().empty());
}

CPU_TEST(test_slice_variant_errors_before_the_device) {  // algorithms.rs:997-1020, 984-994; simd_ops.rs:620-628
    const CacheAwareParams cp;
    CHECK_EQ(cp.cache_line_size, size_t(64));
    CHECK_EQ(cp.l1_cache_size, size_t(32 * 1024));
    CHECK_EQ(cp.l2_cache_size, size_t(256 * 1024));
    CHECK_EQ(cp.l3_cache_size, size_t(8 * 1024 * 1024));
    CHECK_EQ(cp.prefetch_distance, size_t(16));
    CHECK(cp.enable_chunking);
    std::vector<float> in{1.0f, 2.0f}, out(3);
    auto r = quantize_per_tensor_affine_cache_aware(in, 0.1f, 0, out, cp);
    CHECK(r.is_err());
    CHECK_EQ(r.unwrap_err().message, std::string("Input and output length mismatch"));
    out.resize(2);
    r = quantize_per_tensor_affine_cache_aware(in, -0.1f, 0, out, cp);
    CHECK(r.is_err());
    CHECK_EQ(r.unwrap_err().message, std::string("Scale must be positive"));
    CHECK(quantize_streaming_with_prefetch(in, 0.0f, 0, out, cp).is_err());
    CHECK(quantize_with_cache_optimization(in, -1.0f, 0, out).is_err());
    auto m = quantize_matrix_cache_friendly(in, 2, 2, 0.1f, 0, out, cp);
    CHECK(m.is_err());
    CHECK_EQ(m.unwrap_err().message, std::string("Matrix dimensions don't match buffer sizes"));
    auto st = calculate_tensor_stats_cache_optimized({}, cp);
    CHECK(st.is_err());
    CHECK_EQ(st.unwrap_err().message, std::string("Cannot calculate stats of empty tensor"));
    CHECK(calculate_tensor_stats_simd({}).is_err());
    std::vector<int8_t> q8(1);
    CHECK(quantize_mobile_optimized(in, 0.1f, 0, q8, false).is_err());
    q8.resize(2);
    CHECK(quantize_mobile_optimized(in, 0.0f, 0, q8, true).is_err());
    std::vector<std::vector<float> *> outs;
    auto b = quantize_batch_consistent_simd({&in}, 0.1f, 0, outs);
    CHECK(b.is_err());
    CHECK_EQ(b.unwrap_err().message, std::string("Number of input tensors must match output tensors"));
}

GPU_TEST(test_slice_variants) {  // algorithms.rs:897-982, simd_ops.rs:513-522, 569-618
    const CacheAwareParams cp;
    std::vector<float> in8{1, 2, 3, 4, 5, 6, 7, 8}, out8(8);
    CHECK(quantize_per_tensor_affine_cache_aware(in8, 0.1f, 0, out8, cp).is_ok());
    CHECK_EQ(out8[0], 10.0f);
    CHECK_EQ(out8[7], 80.0f);
    std::fill(out8.begin(), out8.end(), 0.0f);
    CHECK(quantize_neon_optimized(in8, 0.1f, 0, out8).is_ok());
    CHECK(out8[0] == 10.0f && out8[1] == 20.0f && out8[7] == 80.0f);
    std::vector<float> m9{1, 2, 3, 4, 5, 6, 7, 8, 9}, o9(9);
    CHECK(quantize_matrix_cache_friendly(m9, 3, 3, 0.1f, 0, o9, cp).is_ok());
    CHECK(o9[0] == 10.0f && o9[8] == 90.0f);
    std::vector<float> s5{0.1f, 0.2f, 0.3f, 0.4f, 0.5f}, o5(5);
    CHECK(quantize_streaming_with_prefetch(s5, 0.01f, 10, o5, cp).is_ok());
    CHECK_EQ(o5[0], 20.0f);
    std::vector<float> in4{1, 2, 3, 4}, o4(4);
    CHECK(quantize_with_cache_optimization(in4, 0.1f, 0, o4).is_ok());
    CHECK(o4[0] == 10.0f && o4[3] == 40.0f);
    const auto st10 = calculate_tensor_stats_cache_optimized({1, 2, 3, 4, 5, 6, 7, 8, 9, 10}, cp).unwrap();
    CHECK(std::get<0>(st10) == 1.0f && std::get<1>(st10) == 10.0f);
    CHECK(std::fabs(std::get<2>(st10) - 5.5f) < 0.001f && std::get<3>(st10) > 0.0f);
    const TensorStats st5 = calculate_tensor_stats_simd({1, 2, 3, 4, 5}).unwrap();
    CHECK(st5.min == 1.0f && st5.max == 5.0f && st5.mean == 3.0f);
    CHECK(std::fabs(st5.std_dev - static_cast<float>(std::sqrt(2.0))) < 1e-4f);
    std::vector<float> mob{1, 2, 3, 4, -1, -2};
    std::vector<int8_t> q6(6);
    CHECK(quantize_mobile_optimized(mob, 0.1f, 0, q6, false).is_ok());
    CHECK_SAME(q6, (std::vector<int>{10, 20, 30, 40, -10, -20}));
    std::vector<int8_t> q4(4);
    CHECK(quantize_mobile_optimized(in4, 0.1f, 0, q4, true).is_ok());
    CHECK(std::abs(q4[0] - 10) <= 1 && std::abs(q4[1] - 20) <= 1);
    const auto mm = find_min_max_neon({-1.5f, 0.0f, 2.3f, -0.8f, 4.7f, 1.2f, 9.5f, -2.1f}).unwrap();
    CHECK(mm.first == -2.1f && mm.second == 9.5f);
}

GPU_TEST(parity_slice_variants) {
    const CacheAwareParams cp;
    for (size_t n : {size_t(7), size_t(256), size_t(257), size_t(100003)}) {
        std::vector<float> x = normal(n, 300 + static_cast<uint32_t>(n), 2.5f);
        if (n > 300) {
            x[5] = 1.25f, x[6] = -1.25f, x[7] = 0.24999999f;  // ties and the 0.49999997 edge at scale 0.5
            x[8] = 1e9f, x[9] = -1e9f, x[10] = NAN;
        }
        std::vector<float> want(n), got(n);
        CHECK_EQ(tq_quantize_cache_aware(x.data(), n, 0.5f, -7, want.data()), 0);
        CHECK(quantize_per_tensor_affine_cache_aware(x, 0.5f, -7, got, cp).is_ok());
        check_same_bits(got, want, __LINE__);
        CHECK(quantize_streaming_with_prefetch(x, 0.5f, -7, got, cp).is_ok());
        check_same_bits(got, want, __LINE__);
        CHECK(quantize_with_cache_optimization(x, 0.5f, -7, got, &cp).is_ok());
        check_same_bits(got, want, __LINE__);
        for (bool reduced : {false, true}) {
            std::vector<int8_t> q(n), wq(n);
            CHECK_EQ(tq_quantize_mobile_optimized(x.data(), n, 0.5f, 3, reduced ? 1 : 0, wq.data()), 0);
            CHECK(quantize_mobile_optimized(x, 0.5f, 3, q, reduced).is_ok());
            CHECK_SAME(q, wq);
        }
        if (n > 300) x[8] = 3.0f, x[9] = -3.0f, x[10] = 0.0f;  // finite data for the statistics
        for (float &v : x) v += 4.0f;
        float w5[5], w4[4];
        CHECK_EQ(tq_calculate_tensor_stats_simd(x.data(), n, w5), 0);
        CHECK_EQ(tq_calculate_tensor_stats_cache_optimized(x.data(), n, w4), 0);
        const TensorStats st = calculate_tensor_stats_simd(x).unwrap();
        CHECK(st.min == w5[0] && st.max == w5[1]);
        CHECK(std::fabs(st.mean - w5[2]) <= 1e-6f * std::fabs(w5[2]));
        CHECK(std::fabs(st.std_dev - w5[3]) <= 1e-6f * w5[3] && std::fabs(st.variance - w5[4]) <= 1e-6f * w5[4]);
        const auto co = calculate_tensor_stats_cache_optimized(x, cp).unwrap();
        CHECK(std::get<0>(co) == w4[0] && std::get<1>(co) == w4[1]);
        CHECK(std::fabs(std::get<2>(co) - w4[2]) <= 1e-6f * std::fabs(w4[2]));
        CHECK(std::fabs(std::get<3>(co) - w4[3]) <= 2e-5f * w4[3]);  // raw moments cancel: E[x^2] - mean^2
    }
    std::vector<float> a = normal(1000, 311, 1.0f), b = normal(70, 312, 3.0f), oa(1000), ob(70), wa(1000), wb(70);
    std::vector<std::vector<float> *> outs{&oa, &ob};
    CHECK(quantize_batch_consistent_simd({&a, &b}, 0.02f, 4, outs).is_ok());
    CHECK_EQ(tq_quantize_per_tensor_affine_simd(a.data(), a.size(), 0.02f, 4, wa.data()), 0);
    CHECK_EQ(tq_quantize_per_tensor_affine_simd(b.data(), b.size(), 0.02f, 4, wb.data()), 0);
    check_same_bits(oa, wa, __LINE__);
    check_same_bits(ob, wb, __LINE__);
}

GPU_TEST(parity_model_quantizer) {  // crates/torsh-models/src/quantization.rs:260-332, 491-566
    std::map<std::string, Tensor> params;
    params.emplace("block.fc1.weight", Tensor::from_data(normal(64 * 48, 51, 0.05f), {64, 48}).unwrap());
    params.emplace("block.fc1.bias", Tensor::from_data(normal(64, 52, 0.01f), {64}).unwrap());
    params.emplace("block.conv.weight", Tensor::from_data(normal(8 * 4 * 3 * 3, 53, 0.2f), {8, 4, 3, 3}).unwrap());
    params.emplace("norm.gamma", Tensor::from_data(std::vector<float>(48, 1.0f), {48}).unwrap());  // constant tensor
    for (mq::QuantizationDType dt : {mq::QuantizationDType::Int8, mq::QuantizationDType::Uint8}) {
        mq::QuantizationConfig cfg = mq::quantization_utils::post_training_quantization_config(dt);
        mq::ModelQuantizer quantizer{cfg};
        const mq::QuantizationStats stats = quantizer.quantize_parameters(params).unwrap();
        size_t total = 0;
        for (const auto &[name, t] : params) total += t.numel();
        CHECK_EQ(stats.original_size, total * 4);
        CHECK_EQ(stats.quantized_size, total);
        CHECK_EQ(stats.compression_ratio, 4.0);
        CHECK_EQ(stats.theoretical_speedup, 2.0);
        const int32_t qmin = dt == mq::QuantizationDType::Int8 ? -128 : 0, qmax = qmin + 255;
        for (const auto &[name, t] : params) {
            const std::vector<float> &x = t.as_slice();
            float mn, mx, s, amin, amax;
            int32_t z;
            tq_min_max_fold(x.data(), x.size(), &mn, &mx);
            tq_model_calculate_quantization_params(mn, mx, qmin, qmax, &s, &z, &amin, &amax);
            const mq::QuantizationParams &p = quantizer.quantization_params().at(name);
            CHECK(p.scale == s && p.zero_point == z && p.min_val == amin && p.max_val == amax);
            std::vector<float> want(x.size());
            tq_model_fake_quantize(x.data(), x.size(), s, z, qmin, qmax, want.data());
            check_same(quantizer.quantize_tensor(t, p).unwrap().as_slice(), want, __LINE__);
            CHECK(close_rel(stats.layer_stats.at(name).quantization_error, tq_model_mse_error(x.data(), want.data(), x.size()), 1e-5, 1e-12));
            CHECK_EQ(stats.layer_stats.at(name).original_params, x.size());
            CHECK_EQ(int(stats.layer_stats.at(name).bits_per_param), 8);
        }
        // parameters survive a save / load through JSON bit for bit
        const std::string path = "/tmp/torsh_hipq_qparams_test.json";
        CHECK(quantizer.save_quantization_params(path).is_ok());
        mq::ModelQuantizer other{cfg};
        CHECK(other.load_quantization_params(path).is_ok());
        CHECK_EQ(other.quantization_params().size(), params.size());
        for (const auto &[name, p] : quantizer.quantization_params()) {
            const mq::QuantizationParams &o = other.quantization_params().at(name);
            CHECK(o.scale == p.scale && o.zero_point == p.zero_point && o.min_val == p.min_val &&
                  o.max_val == p.max_val && o.dtype == p.dtype);
        }
        std::remove(path.c_str());
    }
    // the layer filter restricts calibration, not the size statistics
    mq::QuantizationConfig cfg;
    cfg.layer_filter.kind = mq::LayerQuantizationFilter::Include;
    cfg.layer_filter.names = {"fc1"};
    mq::ModelQuantizer filtered{cfg};
    const auto st = filtered.quantize_parameters(params).unwrap();
    CHECK_EQ(filtered.quantization_params().size(), size_t(2));
    CHECK_EQ(st.layer_stats.size(), size_t(4));
    CHECK_EQ(st.layer_stats.at("norm.gamma").quantization_error, 0.0);
    mq::MinMaxObserver obs;  // quantization.rs:756-768
    CHECK(obs.observe(Tensor::from_data({1.f, 2.f, 3.f}, {3}).unwrap()).is_ok());
    CHECK(obs.observe(Tensor::from_data({-1.f, 0.f, 4.f}, {3}).unwrap()).is_ok());
    CHECK(obs.get_min_max() == std::make_pair(-1.0f, 4.0f));
}

GPU_TEST(test_quantized_modules_survive_a_weight_file) {
    const size_t n = 96, k = 256, m = 7;
    const Tensor w = Tensor::from_data(normal(n * k, 61, 0.03f), {n, k}).unwrap();
    const Tensor b = Tensor::from_data(normal(n, 62, 0.01f), {n}).unwrap();
    const Tensor x = Tensor::from_data(normal(m * k, 63), {m, k}).unwrap();
    auto lin = nn::QuantizedLinear::from_weight_nk(w, &b, nn::ActivationQuant::PerToken).unwrap();
    const std::string path = "/tmp/torsh_hipq_linear_test.bin";
    CHECK(lin.save(path).is_ok());
    auto back = nn::QuantizedLinear::load(path, nn::ActivationQuant::PerToken).unwrap();
    CHECK(back.in_features() == k && back.out_features() == n);
    check_same(back.forward(x).unwrap().as_slice(), lin.forward(x).unwrap().as_slice(), __LINE__);
    // the file holds exactly what quantize_per_channel_auto produces on axis 0
    const QuantizedWeights file = load_quantized_weights(path).unwrap();
    std::vector<float> carrier(n * k), scales(n);
    std::vector<int32_t> zps(n);
    const size_t shape[2] = {n, k};
    CHECK_EQ(tq_quantize_per_channel_auto(w.as_slice().data(), shape, 2, 0, TQ_DTYPE_I8, TQ_PER_CHANNEL_SYMMETRIC,
                                          carrier.data(), scales.data(), zps.data()), 0);
    check_same(file.scales, scales, __LINE__);
    for (size_t i = 0; i < n * k; ++i) CHECK(static_cast<float>(file.weight[i]) == carrier[i]);
    check_same(file.bias, b.as_slice(), __LINE__);
    std::remove(path.c_str());
    // The prepared blob: the rows in the operand order of the matrix cores.  The file's payload is the layout
    // written out on the host from the row-major codes (ragged shape: 96 rows are three row blocks, K = 304 pads
    // to 12 k blocks), a layer loaded from it forwards the same bits without a packing pass, and its row-major
    // view (rebuilt from the prepared bytes) is the row-major file's.
    {
        const size_t n2 = 70, k2 = 304;
        const Tensor w2 = Tensor::from_data(normal(n2 * k2, 66, 0.03f), {n2, k2}).unwrap();
        const Tensor x2 = Tensor::from_data(normal(m * k2, 67), {m, k2}).unwrap();
        auto lin2 = nn::QuantizedLinear::from_weight_nk(w2, nullptr, nn::ActivationQuant::PerTensor).unwrap();
        CHECK(lin2.save_prepared(path).is_ok());
        const QuantizedWeights prepared = load_quantized_weights(path).unwrap();
        const QuantizedWeights plain = lin2.to_quantized_weights().unwrap();
        CHECK(prepared.packed.size() == packed_layout::bytes(n2, k2) && prepared.packed.size() == 3 * 12 * 1024);
        CHECK_SAME(prepared.weight, plain.weight);
        std::vector<int8_t> want(prepared.packed.size(), 0);
        for (size_t r = 0; r < n2; ++r)
            for (size_t kk = 0; kk < k2; ++kk) want[packed_layout::offset(r, kk, k2)] = plain.weight[r * k2 + kk];
        CHECK_SAME(prepared.packed, want);
        auto back2 = nn::QuantizedLinear::load(path).unwrap();
        check_same(back2.forward(x2).unwrap().as_slice(), lin2.forward(x2).unwrap().as_slice(), __LINE__);
        CHECK_SAME(back2.to_quantized_weights(true).unwrap().packed, want);
        // a damaged prepared section is caught by the checksum
        {
            std::fstream f(path, std::ios::in | std::ios::out | std::ios::binary);
            f.seekp(256 + 1000);
            const char flip = 0x55;
            f.write(&flip, 1);
        }
        CHECK(load_quantized_weights(path).is_err());
        std::remove(path.c_str());
    }
    // conv: same round trip
    const Tensor cw = Tensor::from_data(normal(8 * 4 * 3 * 3, 64, 0.1f), {8, 4, 3, 3}).unwrap();
    const Tensor cx = Tensor::from_data(normal(2 * 4 * 6 * 6, 65, 1.0f, true), {2, 4, 6, 6}).unwrap();
    auto conv = nn::QuantizedConv2d::from_weight(cw, nullptr, {1, 1}, {1, 1}, 0.05f, 3).unwrap();
    CHECK(conv.save(path).is_ok());
    auto conv2 = nn::QuantizedConv2d::from_quantized(load_quantized_weights(path).unwrap(), {1, 1}, {1, 1}, 0.05f, 3).unwrap();
    check_same(conv2.forward_quantized(cx).unwrap().as_slice(), conv.forward_quantized(cx).unwrap().as_slice(), __LINE__);
    CHECK(nn::QuantizedLinear::load(path).is_err());  // a conv file is not a linear layer
    std::remove(path.c_str());
}


CPU_TEST(test_fake_quantize_errors_before_the_device) {  // fake_quantize.rs:120-128, 152-156
    auto t = tensor_1d({-2.0f, -1.0f, 0.0f, 1.0f, 2.0f}).unwrap();
    auto r = fake_quantize_auto(t, DType::F32, QScheme::PerTensorAffine);
    CHECK(r.is_err() && r.unwrap_err().message == "Unsupported quantization dtype");
    auto r2 = fake_quantize_auto(t, DType::I8, QScheme::PerChannelAffine);
    CHECK(r2.is_err() && r2.unwrap_err().message == "Quantization scheme not yet implemented");
    // an empty tensor needs no device either: its range folds to (0, 0), the scale becomes 1
    auto e = Tensor::from_data(std::vector<float>{}, {0}).unwrap();
    auto p = fake_quantize_auto_params(e, DType::U8, QScheme::PerTensorAffine).unwrap();
    CHECK(p.first == 1.0f && p.second == 0);
    CHECK(fake_quantize_auto(e, DType::I8, QScheme::PerTensorSymmetric).unwrap().numel() == 0);
    auto fq = FakeQuantize::uint8(0.25f, 7);
    fq.disable();
    CHECK(!fq.enabled());
    CHECK_SAME(fq.forward(t).unwrap().as_slice(), t.as_slice());  // passthrough needs no device
    fq.update_params(0.5f, 9);
    CHECK(fq.scale() == 0.5f && fq.zero_point() == 9);
}

GPU_TEST(test_fake_quantize) {  // fake_quantize.rs:173-244
    {  // test_fake_quantize_per_tensor_affine
        std::vector<float> data{0.0f, 1.0f, 2.0f, 3.0f};
        const float scale = 0.1f;
        auto y = fake_quantize_per_tensor_affine(tensor_1d(data).unwrap(), scale, 0, -128, 127).unwrap();
        for (size_t i = 0; i < data.size(); ++i) CHECK(std::fabs(y.as_slice()[i] - data[i]) <= scale);
    }
    {  // test_fake_quantize_symmetric
        auto y = fake_quantize_per_tensor_symmetric(tensor_1d({-1.0f, 0.0f, 1.0f, 2.0f}).unwrap(), 0.1f, -128, 127).unwrap();
        CHECK(y.numel() == 4);
    }
    {  // test_fake_quantize_module
        auto fq = FakeQuantize::int8(0.1f, 0);
        std::vector<float> data{0.5f, 1.5f, 2.5f, 3.5f};
        auto t = tensor_1d(data).unwrap();
        CHECK(fq.forward(t).unwrap().numel() == data.size());
        fq.disable();
        auto pass = fq.forward(t).unwrap();
        for (size_t i = 0; i < data.size(); ++i) CHECK(std::fabs(pass.as_slice()[i] - data[i]) <= 1e-5f);
    }
    {  // test_fake_quantize_auto (ignored in the reference: "test hangs"; its assertions hold here)
        auto y = fake_quantize_auto(tensor_1d({-2.0f, -1.0f, 0.0f, 1.0f, 2.0f}).unwrap(), DType::I8, QScheme::PerTensorAffine).unwrap();
        CHECK(y.numel() == 5);
        for (float v : y.as_slice()) CHECK(v >= -2.1f && v <= 2.1f);
    }
    CHECK(fake_quantize(tensor_1d({1.0f}).unwrap(), 0.0f, 0).is_err());
}

GPU_TEST(parity_fake_quantize) {
    auto x = normal(5000, 71, 2.0f);
    x[0] = NAN, x[1] = INFINITY, x[2] = -INFINITY, x[3] = 0.25f, x[4] = -0.25f, x[5] = 1e9f;
    auto t = tensor_1d(x).unwrap();
    std::vector<float> want(x.size());
    tq_fake_quantize_per_tensor_affine(x.data(), x.size(), 0.5f, 3, -128, 127, want.data());
    CHECK_SAME(fake_quantize(t, 0.5f, 3).unwrap().as_slice(), want);
    tq_fake_quantize_per_tensor_affine(x.data(), x.size(), 0.0173f, 10, 0, 255, want.data());
    CHECK_SAME(FakeQuantize::uint8(0.0173f, 10).forward(t).unwrap().as_slice(), want);
    // auto: parameters and image against the oracle, both schemes and both dtypes (finite data)
    auto xf = normal(3000, 72, 1.5f);
    xf[7] = 4.0f;
    auto tf = tensor_1d(xf).unwrap();
    for (int dtype = 0; dtype < 2; ++dtype)
        for (int scheme = 0; scheme < 2; ++scheme) {
            float s;
            int32_t z;
            CHECK(tq_fake_quantize_auto(xf.data(), xf.size(), dtype, scheme, want.data(), &s, &z) == 0);
            const DType dt = dtype ? DType::U8 : DType::I8;
            const QScheme sc = scheme ? QScheme::PerTensorSymmetric : QScheme::PerTensorAffine;
            auto p = fake_quantize_auto_params(tf, dt, sc).unwrap();
            CHECK(p.first == s && p.second == z);
            std::vector<float> w3(want.begin(), want.begin() + xf.size());
            CHECK_SAME(fake_quantize_auto(tf, dt, sc).unwrap().as_slice(), w3);
        }
}

GPU_TEST(test_special_schemes) {  // specialized.rs:577-654, 743-761
    {
        const std::vector<float> data{1.0f, 2.0f, 3.0f, 4.0f, 5.0f};
        const auto [q, scale, zp] = quantize_int4_per_tensor(tensor_1d(data).unwrap(), QuantConfig::int4()).unwrap();
        CHECK(scale > 0.0f && zp >= -8 && zp <= 7);
        CHECK_EQ(q.numel(), data.size());
        for (float v : q.as_slice()) CHECK(v >= -8.0f && v <= 7.0f);
    }
    {
        const auto [q, scale, zp] = quantize_binary(tensor_1d({-2.0f, -1.0f, 0.0f, 1.0f, 2.0f}).unwrap()).unwrap();
        CHECK(scale > 0.0f && zp == 0);
        for (float v : q.as_slice()) CHECK(v == -1.0f || v == 1.0f);
    }
    {
        const auto [q, scale, zp] = quantize_ternary(tensor_1d({-3.0f, -1.0f, 0.1f, 1.0f, 3.0f}).unwrap()).unwrap();
        CHECK(scale > 0.0f && zp == 0);
        for (float v : q.as_slice()) CHECK(v == -1.0f || v == 0.0f || v == 1.0f);
    }
    {
        const Tensor t = Tensor::from_data({1.0f, 2.0f, 3.0f, 4.0f, 5.0f, 6.0f}, {2, 3}).unwrap();
        const auto [q, scale, zp] = quantize_group_wise(t, 1, 2, QuantConfig::group_wise(1, 2)).unwrap();
        CHECK(scale > 0.0f && q.shape().dims() == t.shape().dims());
    }
    const Tensor empty = tensor_1d({}).unwrap();
    CHECK(quantize_binary(empty).is_err() && quantize_ternary(empty).is_err());
    const Tensor t3 = tensor_1d({1.0f, 2.0f, 3.0f}).unwrap();
    CHECK(quantize_group_wise(t3, 5, 2, QuantConfig::group_wise(0, 2)).is_err());
    CHECK(quantize_group_wise(t3, 0, 0, QuantConfig::group_wise(0, 2)).is_err());
    // through the dispatcher (algorithms.rs:47-57)
    CHECK(quantize_with_config(t3, QuantConfig::int4()).is_ok());
    CHECK(quantize_with_config(t3, QuantConfig::binary()).is_ok());
    CHECK(quantize_with_config(t3, QuantConfig::ternary()).is_ok());
    CHECK(quantize_with_config(t3, QuantConfig::group_wise(0, 2)).is_ok());
}

GPU_TEST(test_searched_thresholds_and_mixed_precision) {  // specialized.rs:655-740
    {
        const std::vector<float> data{-2.0f, -0.1f, 0.1f, 0.5f, 2.0f};
        const auto [q, scale, zp, threshold] = quantize_binary_learned_threshold(tensor_1d(data).unwrap(), 0.3f).unwrap();
        CHECK(scale > 0.0f && zp == 0);
        CHECK_EQ(threshold, 0.3f);
        for (size_t i = 0; i < data.size(); ++i) {
            const float expected = std::fabs(data[i]) <= 0.3f ? 0.0f : (data[i] >= 0.0f ? 1.0f : -1.0f);
            CHECK_EQ(q.as_slice()[i], expected);
        }
    }
    {
        const std::vector<float> data{-3.0f, -0.5f, 0.0f, 0.5f, 3.0f};
        const auto [q, scale, zp, threshold] = quantize_ternary_adaptive(tensor_1d(data).unwrap()).unwrap();
        CHECK(scale > 0.0f && zp == 0 && threshold > 0.0f);
        CHECK_EQ(q.numel(), data.size());
        for (float v : q.as_slice()) CHECK(v == -1.0f || v == 0.0f || v == 1.0f);
    }
    std::map<std::string, Tensor> tensors;
    tensors.emplace("embedding", tensor_1d({1.0f, 2.0f, 3.0f}).unwrap());
    tensors.emplace("attention", tensor_1d({4.0f, 5.0f, 6.0f}).unwrap());
    const MixedPrecisionConfig config;
    const auto results = quantize_mixed_precision(tensors, config).unwrap();
    CHECK_EQ(results.size(), size_t(2));
    CHECK(results.count("embedding") == 1 && results.count("attention") == 1);
    // specialized.rs:678-690
    CHECK(determine_layer_precision("layer.embedding.weight", config) == DType::I8);
    CHECK(determine_layer_precision("layer.attention.query", config) == DType::F16);
    CHECK(determine_layer_precision("layer.unknown.weight", config) == DType::I8);  // default
    CHECK(determine_layer_precision("head.output", config) == DType::F32);
    CHECK(create_precision_config(DType::U8).dtype == DType::U8 && create_precision_config(DType::I32).dtype == DType::I8);
    CHECK(create_precision_config(DType::F16).dtype == DType::F16 && !create_precision_config(DType::F32).enable_fake_quant);
    const Tensor empty = tensor_1d({}).unwrap();
    CHECK(quantize_binary_learned_threshold(empty).is_err() && quantize_ternary_adaptive(empty).is_err());
}

GPU_TEST(parity_searched_thresholds_and_mixed_precision) {
    const std::vector<float> x = normal(20011, 91, 1.2f);
    const Tensor t = tensor_1d(x).unwrap();
    std::vector<float> want(x.size());
    float s32, thr;
    double s64;
    for (int given = 0; given < 2; ++given) {
        CHECK_EQ(tq_quantize_binary_learned_threshold(x.data(), x.size(), given, 0.45f, 1, want.data(), &s32, &s64, &thr), 0);
        const auto [q, scale, zp, threshold] =
            quantize_binary_learned_threshold(t, given ? std::optional<float>(0.45f) : std::nullopt).unwrap();
        check_same(q.as_slice(), want, __LINE__);
        CHECK(zp == 0 && threshold == thr);
        CHECK(std::fabs(scale - s64) <= 1e-6 * s64);
    }
    CHECK_EQ(tq_quantize_ternary_adaptive(x.data(), x.size(), 1, want.data(), &s32, &s64, &thr, nullptr, nullptr), 0);
    {
        const auto [q, scale, zp, threshold] = quantize_ternary_adaptive(t).unwrap();
        check_same(q.as_slice(), want, __LINE__);
        CHECK(zp == 0 && threshold == thr);
        CHECK(std::fabs(scale - s64) <= 1e-6 * s64);
    }
    // mixed precision = quantize_with_config per tensor: int8 per-tensor affine for all three default precisions
    std::map<std::string, Tensor> tensors;
    tensors.emplace("model.embedding.weight", Tensor::from_data(normal(600, 92, 0.7f), {20, 30}).unwrap());
    tensors.emplace("block0.attention.q", Tensor::from_data(normal(500, 93, 0.2f), {500}).unwrap());
    tensors.emplace("head.output", Tensor::from_data(normal(70, 94, 2.0f), {70}).unwrap());
    const auto results = quantize_mixed_precision(tensors, MixedPrecisionConfig{}).unwrap();
    for (const auto &[name, tensor] : tensors) {
        const std::vector<float> &v = tensor.as_slice();
        std::vector<float> wq(v.size());
        float ws;
        int32_t wz;
        CHECK_EQ(tq_quantize_tensor_auto(v.data(), v.size(), TQ_DTYPE_I8, TQ_PER_TENSOR_AFFINE, wq.data(), &ws, &wz), 0);
        const QuantizedTriple &r = results.at(name);
        check_same(std::get<0>(r).as_slice(), wq, __LINE__);
        CHECK(std::get<1>(r) == ws && std::get<2>(r) == wz);
    }
}

GPU_TEST(parity_special_schemes) {
    const std::vector<float> x = normal(24 * 50 * 6, 71, 1.3f);
    const std::vector<size_t> dims{24, 50, 6};
    const Tensor t = Tensor::from_data(x, dims).unwrap();
    std::vector<float> want(x.size());
    float s;
    int32_t z;
    {
        const auto [q, scale, zp] = quantize_int4_per_tensor(t, QuantConfig::int4()).unwrap();
        CHECK_EQ(tq_quantize_int4_per_tensor(x.data(), x.size(), want.data(), &s, &z), 0);
        CHECK(scale == s && zp == z);
        check_same(q.as_slice(), want, __LINE__);
    }
    for (size_t axis : {size_t(0), size_t(1), size_t(2)}) {
        std::vector<float> scales(dims[axis]);
        std::vector<int32_t> zps(dims[axis]);
        const auto [q, scale, zp] = quantize_int4_per_channel(t, axis, QuantConfig::int4()).unwrap();
        CHECK_EQ(tq_quantize_int4_per_channel(x.data(), dims.data(), 3, axis, want.data(), scales.data(), zps.data(), &s, &z), 0);
        CHECK(scale == s && zp == z);
        check_same(q.as_slice(), want, __LINE__);
    }
    {
        double s64;
        const auto [q, scale, zp] = quantize_binary(t).unwrap();
        CHECK_EQ(tq_quantize_binary(x.data(), x.size(), want.data(), &s, &s64), 0);
        check_same(q.as_slice(), want, __LINE__);
        CHECK(close_rel(scale, s64, 1e-6) && close_rel(scale, s, 1e-4) && zp == 0);
    }
    {
        double s64;
        float thr;
        const auto [q, scale, zp] = quantize_ternary(t).unwrap();
        CHECK_EQ(tq_quantize_ternary(x.data(), x.size(), want.data(), &s, &s64, &thr), 0);
        check_same(q.as_slice(), want, __LINE__);
        CHECK(close_rel(scale, s64, 1e-6) && close_rel(scale, s, 1e-4) && zp == 0);
    }
    struct G {
        size_t axis, group;
    };
    for (G g : {G{0, 4}, G{0, 5}, G{0, 24}, G{0, 100}, G{1, 10}, G{1, 50}, G{1, 7}, G{2, 3}, G{2, 1}, G{2, 4}}) {
        const QuantConfig cfg = QuantConfig::group_wise(g.axis, g.group);
        const size_t groups = (dims[g.axis] + g.group - 1) / g.group;
        std::vector<float> gs(groups);
        std::vector<int32_t> gz(groups);
        const auto [q, scale, zp] = quantize_group_wise(t, g.axis, g.group, cfg).unwrap();
        CHECK_EQ(tq_quantize_group_wise(x.data(), dims.data(), 3, g.axis, g.group, -128, 127, want.data(), gs.data(),
                                        gz.data(), &s, &z), 0);
        CHECK(scale == s && zp == z);
        check_same(q.as_slice(), want, __LINE__);
    }
    // reduced integer range through the configuration (config.rs:304-328)
    const QuantConfig reduced = QuantConfig::group_wise(0, 4).with_reduce_range(ReduceRange::Reduce);
    const auto [qmin, qmax] = reduced.get_qint_range();
    std::vector<float> gs(6);
    std::vector<int32_t> gz(6);
    const auto [q, scale, zp] = quantize_group_wise(t, 0, 4, reduced).unwrap();
    CHECK_EQ(tq_quantize_group_wise(x.data(), dims.data(), 3, 0, 4, qmin, qmax, want.data(), gs.data(), gz.data(), &s, &z), 0);
    CHECK(scale == s && zp == z);
    check_same(q.as_slice(), want, __LINE__);
}


GPU_TEST(parity_backend_qadd_qrelu) {  // crates/torsh-backend/src/quantization/ops.rs:582-624
    bq::HipQuantizationOps ops;
    std::mt19937 g(91);
    std::uniform_int_distribution<int> byte(0, 255);
    for (auto dtype : {bq::QuantizedDType::Int8, bq::QuantizedDType::UInt8}) {
        for (auto scheme : {bq::QuantizationScheme::Asymmetric, bq::QuantizationScheme::Symmetric}) {
            const size_t n = 70001;
            std::vector<uint8_t> a(n), b(n);
            for (auto &v : a) v = static_cast<uint8_t>(byte(g));
            for (auto &v : b) v = static_cast<uint8_t>(byte(g));
            bq::QuantizationParams pa, pb;
            pa.dtype = pb.dtype = dtype;
            pa.scheme = pb.scheme = scheme;
            const bool is_signed = dtype == bq::QuantizedDType::Int8;
            const bool sym = scheme == bq::QuantizationScheme::Symmetric;  // validate() demands zero point 0 then
            pa.scale = {0.0173f}, pa.zero_point = {sym ? 0 : (is_signed ? -7 : 121)};
            pb.scale = {0.0419f}, pb.zero_point = {sym ? 0 : (is_signed ? 12 : 99)};
            const auto ta = bq::QuantizedTensor::from_data(a, {n}, pa).unwrap();
            const auto tb = bq::QuantizedTensor::from_data(b, {n}, pb).unwrap();
            const int32_t qmin = is_signed ? -128 : 0, qmax = is_signed ? 127 : 255;
            std::vector<uint8_t> want(n);
            float s;
            int32_t z;
            const auto sum = ops.qadd(ta, tb).unwrap();
            CHECK_EQ(tq_backend_qadd_or_qrelu(a.data(), is_signed, pa.scale[0], pa.zero_point[0], b.data(), is_signed,
                                              pb.scale[0], pb.zero_point[0], n, scheme == bq::QuantizationScheme::Symmetric,
                                              qmin, qmax, want.data(), &s, &z), 0);
            CHECK(sum.params.scale[0] == s && sum.params.zero_point[0] == z && sum.params.dtype == dtype);
            check_same(sum.data, want, __LINE__);
            const auto relu = ops.qrelu(ta).unwrap();
            CHECK_EQ(tq_backend_qadd_or_qrelu(a.data(), is_signed, pa.scale[0], pa.zero_point[0], nullptr, 0, 1.0f, 0, n,
                                              scheme == bq::QuantizationScheme::Symmetric, qmin, qmax, want.data(), &s, &z), 0);
            CHECK(relu.params.scale[0] == s && relu.params.zero_point[0] == z);
            check_same(relu.data, want, __LINE__);
            CHECK(relu.params.min_val.value_or(-1.0f) == 0.0f);
        }
    }
    // shape mismatch and unsupported operands
    bq::QuantizationParams p;
    p.dtype = bq::QuantizedDType::Int8;
    p.scale = {0.1f}, p.zero_point = {0};
    const auto t4 = bq::QuantizedTensor::from_data({1, 2, 3, 4}, {4}, p).unwrap();
    const auto t22 = bq::QuantizedTensor::from_data({1, 2, 3, 4}, {2, 2}, p).unwrap();
    CHECK(ops.qadd(t4, t22).is_err() && ops.qadd(t4, t22).unwrap_err().kind == TorshError::InvalidArgument);
    // ReLU of an all-negative tensor: range (0, 0) -> asymmetric degenerate parameters (1.0, qmin)
    const auto neg = bq::QuantizedTensor::from_data({0xF6, 0xEC}, {2}, p).unwrap();  // -10, -20
    const auto r = ops.qrelu(neg).unwrap();
    CHECK(r.params.scale[0] == 1.0f && r.params.zero_point[0] == -128);
    CHECK(r.data[0] == 0x80 && r.data[1] == 0x80);
}


CPU_TEST(test_kernel_plugin_interface) {  // hardware.rs:213-241, 482-555
    const HardwareQuantizer hq = HardwareQuantizer::with_hip();
    CHECK(hq.backend == HardwareBackend::make_custom("rocm-gfx950"));
    CHECK_EQ(hq.kernel_dispatch.size(), size_t(4));
    const QuantizationKernel &k = *hq.kernel_dispatch.at(QScheme::PerTensorAffine);
    CHECK(std::string(k.name()) == "HIP-gfx950");
    CHECK(k.supported_backends().size() == 1 && k.supported_backends()[0].kind == HardwareBackend::Custom);
    CHECK(k.performance_characteristics().throughput > GenericKernel{}.performance_characteristics().throughput);
    CHECK_EQ(hq.get_performance_info().size(), size_t(4));
    // errors surface through the plug-in unchanged
    CHECK(hq.quantize(tensor_1d({}).unwrap(), QuantConfig::int8()).is_err());
    CHECK(hq.dequantize(tensor_1d({1.f}).unwrap(), 0.0f, 0).is_err());
}

GPU_TEST(test_kernel_plugin_dispatch) {
    const HardwareQuantizer hq = HardwareQuantizer::with_hip();
    const std::vector<float> x = normal(5000, 77, 2.0f);
    const Tensor t = tensor_1d(x).unwrap();
    for (const QuantConfig &cfg : {QuantConfig::int8(), QuantConfig::int8().with_scheme(QScheme::PerTensorSymmetric),
                                   QuantConfig::int4() /* no registered kernel: generic fallback */}) {
        const auto [q, s, z] = hq.quantize(t, cfg).unwrap();
        const auto [q2, s2, z2] = quantize_with_config(t, cfg).unwrap();
        CHECK(s == s2 && z == z2);
        check_same(q.as_slice(), q2.as_slice(), __LINE__);
        const Tensor back = hq.dequantize(q, s, z).unwrap();
        check_same(back.as_slice(), dequantize(q2, s2, z2).unwrap().as_slice(), __LINE__);
    }
}

// ---- torsh-core scalar quantized types and torsh-nn's quantizer ---------------------------------
// crates/torsh-core/src/dtype/quantized.rs:126-127 (doc example), 878-892 (test_edge_cases), 865-875.
CPU_TEST(test_scalar_quantized_types) {
    using namespace torsh::dtype::quantized;
    CHECK(QInt8::quantize(2.5f, 0.1f, 5).value == 30);  // round(2.5 / 0.1 + 5)
    CHECK(QInt8::quantize(1000.0f, 1.0f, 0).value == 127);
    CHECK(QInt8::quantize(-1000.0f, 1.0f, 0).value == -128);
    const QInt8 q = QInt8::quantize(3.14159265f, 0.1f, 0);
    CHECK(std::fabs(q.dequantize() - 3.14159265f) < 0.05f);
    // the zero point enters before the rounding: -2.5 + 5 = 2.5 -> 3, not round(-2.5) + 5 = 2
    CHECK(QInt8::quantize(-2.5f, 1.0f, 5).value == 3);
    CHECK(QUInt8::quantize(-2.5f, 1.0f, 5).value == 3);
    CHECK(QUInt8::quantize(-1000.0f, 1.0f, 5).value == 0 && QUInt8::quantize(1000.0f, 1.0f, 5).value == 255);
    CHECK(QInt32::quantize(1e20f, 1.0f, 0).value == 2147483647 && QInt32::quantize(-1e20f, 1.0f, 7).value == INT32_MIN);
    CHECK(QInt32::quantize(2.5f, 1.0f, 1).value == 4);  // f64: round(3.5) = 4
    const QInt32 q32{10, 0.5f, 4};
    const QUInt8 qu8{10, 0.5f, 4};
    CHECK(q32.dequantize() == 3.0f && qu8.dequantize() == 3.0f);
    std::mt19937 rng(7);
    std::uniform_real_distribution<float> dv(-40.0f, 40.0f), ds(0.01f, 0.5f);
    for (int i = 0; i < 2000; ++i) {
        const float v = dv(rng), sc = ds(rng);
        const int zp = static_cast<int>(rng() % 200) - 100;
        CHECK(QInt8::quantize(v, sc, static_cast<int8_t>(zp)).value == tq_qint8_quantize(v, sc, zp));
        if (zp >= 0) CHECK(QUInt8::quantize(v, sc, static_cast<uint8_t>(zp)).value == tq_quint8_quantize(v, sc, zp));
    }
}

// crates/torsh-nn/src/quantization/ops.rs:380-429 (test_symmetric_quantization, test_asymmetric_quantization),
// then every value against the oracle's restatement of quantize_value_* and per_channel_quantize_weights.
GPU_TEST(parity_torsh_nn_quantizer_and_qtype_slices) {
    namespace nq = torsh::nn::quantization;
    {
        const Tensor t = tensor_1d({1.0f, -1.0f, 0.5f, -0.5f, 2.0f, -2.0f}).unwrap();
        const nq::QuantizationParams p = nq::QuantizationParams::symmetric(2.0f / 127.0f, DType::F32, DType::I8).unwrap();
        const Tensor back = p.dequantize(p.quantize(t).unwrap()).unwrap();
        for (size_t i = 0; i < 6; ++i) CHECK(std::fabs(back.as_slice()[i] - t.as_slice()[i]) < 0.1f);
    }
    {
        const Tensor t = tensor_1d({0.0f, 1.0f, 2.0f, 3.0f, 4.0f, 5.0f}).unwrap();
        const nq::QuantizationParams p = nq::QuantizationParams::asymmetric(5.0f / 255.0f, 0, DType::F32, DType::U8).unwrap();
        const Tensor back = p.dequantize(p.quantize(t).unwrap()).unwrap();
        for (size_t i = 0; i < 6; ++i) CHECK(std::fabs(back.as_slice()[i] - t.as_slice()[i]) < 0.1f);
    }
    CHECK(nq::QuantizationParams::symmetric(1.0f, DType::F32, DType::F32).is_err());
    std::mt19937 rng(11);
    std::normal_distribution<float> nd(0.0f, 2.0f);
    std::vector<float> x(3000);
    for (float &v : x) v = nd(rng);
    x[0] = NAN, x[1] = INFINITY, x[2] = -INFINITY, x[3] = 2.5f * 0.05f, x[4] = -2.5f * 0.05f;
    const Tensor t = tensor_1d(x).unwrap();
    {
        const nq::QuantizationParams p = nq::QuantizationParams::symmetric(0.05f, DType::F32, DType::I8).unwrap();
        const Tensor q = p.quantize(t).unwrap();
        for (size_t i = 0; i < x.size(); ++i)
            CHECK(q.as_slice()[i] == static_cast<float>(tq_nn_quantize_value_symmetric(x[i], 0.05f, -128, 127)));
        CHECK(q.as_slice()[0] == 0.0f);  // NaN as i32
    }
    {
        const nq::QuantizationParams p = nq::QuantizationParams::asymmetric(0.05f, 77, DType::F32, DType::U8).unwrap();
        const Tensor q = p.quantize(t).unwrap();
        for (size_t i = 0; i < x.size(); ++i)
            CHECK(q.as_slice()[i] == static_cast<float>(tq_nn_quantize_value_asymmetric(x[i], 0.05f, 77, 0, 255)));
        CHECK(q.as_slice()[0] == 77.0f);  // NaN -> 0, then the zero point
        const Tensor y = p.dequantize(q).unwrap();
        for (size_t i = 0; i < x.size(); ++i)
            CHECK(y.as_slice()[i] == tq_nn_dequantize_value_asymmetric(static_cast<int32_t>(q.as_slice()[i]), 0.05f, 77));
    }
    // per-channel weights: an all-zero channel keeps scale 0 (no guard)
    std::vector<float> w(6 * 100);
    for (float &v : w) v = nd(rng) * 0.01f;
    for (size_t i = 200; i < 300; ++i) w[i] = 0.0f;
    const Tensor wt = Tensor::from_data(w, {6, 100}).unwrap();
    {
        auto r = nq::per_channel_quantize_weights(wt, nq::QuantizationScheme::Symmetric, DType::I8).unwrap();
        std::vector<float> carrier(w.size()), scales(6);
        tq_nn_per_channel_quantize_weights_sym_i8(w.data(), 6, 100, carrier.data(), scales.data());
        check_same(r.first.as_slice(), carrier, __LINE__);
        for (size_t c = 0; c < 6; ++c) CHECK(r.second[c].scale == scales[c] && r.second[c].zero_point == 0);
        CHECK(r.second[2].scale == 0.0f);
    }
    {
        auto r = nq::per_channel_quantize_weights(wt, nq::QuantizationScheme::Asymmetric, DType::U8);
        // (channel 2 has a zero range: scale 0, zero point round(-0/0) = NaN as i32 = 0, codes NaN -> 0 + 0)
        std::vector<float> carrier(w.size()), scales(6);
        std::vector<int32_t> zps(6);
        tq_nn_per_channel_quantize_weights_asym_u8(w.data(), 6, 100, carrier.data(), scales.data(), zps.data());
        check_same(r.unwrap().first.as_slice(), carrier, __LINE__);
        for (size_t c = 0; c < 6; ++c) CHECK(r.unwrap().second[c].scale == scales[c] && r.unwrap().second[c].zero_point == zps[c]);
    }
    CHECK(nq::per_channel_quantize_weights(wt, nq::QuantizationScheme::Dynamic, DType::I8).is_err());
    // slices of the scalar types on the device
    {
        const auto q = torsh::dtype::quantized::quantize_slice_qint8(x, 0.1f, 5).unwrap();
        for (size_t i = 0; i < x.size(); ++i) CHECK(q[i] == tq_qint8_quantize(x[i], 0.1f, 5));
        const auto u = torsh::dtype::quantized::quantize_slice_quint8(x, 0.1f, 130).unwrap();
        for (size_t i = 0; i < x.size(); ++i) CHECK(u[i] == tq_quint8_quantize(x[i], 0.1f, 130));
    }
}

// quantized_matmul_int8 / quantized_conv2d_int8 / quantized_relu_int8 (crates/torsh-nn/src/quantization/ops.rs:175-294)
// with caller-supplied output parameters.  The device result is bit-identical to the exact int32 composition
// (oracle GEMM / conv accumulators, acc * (s_a * s_b) (+ bias), then the reference's own value formulas) and within
// one output code of the oracle's restatement of the reference's f32 path (dequantize, f32 product, quantize),
// whose summation order the reference does not fix.  The ReLU is exact.
GPU_TEST(parity_torsh_nn_quantized_helpers) {
    namespace nq = torsh::nn::quantization;
    std::mt19937 rng(77);
    std::uniform_int_distribution<int> d8(-128, 127), du8(0, 255);
    for (auto [m, k, n] : {std::make_tuple(size_t(5), size_t(7), size_t(3)), std::make_tuple(size_t(33), size_t(256), size_t(70)),
                           std::make_tuple(size_t(64), size_t(512), size_t(48))}) {
        std::vector<float> a(m * k), b(k * n);
        std::vector<int8_t> a8(m * k), bt8(n * k);
        for (size_t i = 0; i < m * k; ++i) a[i] = float(a8[i] = int8_t(d8(rng)));
        for (size_t l = 0; l < k; ++l)
            for (size_t j = 0; j < n; ++j) b[l * n + j] = float(bt8[j * k + l] = int8_t(d8(rng)));
        const Tensor ta = Tensor::from_data(a, {m, k}).unwrap(), tb = Tensor::from_data(b, {k, n}).unwrap();
        const auto pa = nq::QuantizationParams::symmetric(0.031f, DType::F32, DType::I8).unwrap();
        const auto pb = nq::QuantizationParams::symmetric(0.0007f, DType::F32, DType::I8).unwrap();
        std::vector<int32_t> acc(m * n);
        CHECK_EQ(tq_gemm_i8_nk(a8.data(), bt8.data(), m, n, k, acc.data()), 0);
        const float sab = pa.scale * pb.scale;
        for (const auto &po : {nq::QuantizationParams::symmetric(0.05f, DType::F32, DType::I8).unwrap(),
                               nq::QuantizationParams::asymmetric(0.03f, 131, DType::F32, DType::U8).unwrap(),
                               nq::QuantizationParams::symmetric(0.0004f, DType::F32, DType::I16).unwrap()}) {
            const bool o_u8 = po.dst_dtype == DType::U8;
            const Tensor got = nq::quantized_matmul_int8(ta, tb, pa, pb, po).unwrap();
            CHECK(got.shape().dims() == (std::vector<size_t>{m, n}));
            std::vector<float> ref(m * n);
            CHECK_EQ(tq_nn_quantized_matmul_int8(a.data(), b.data(), m, k, n, pa.scale, 0, 0, pb.scale, 0, 0, po.scale,
                                                 po.zero_point, o_u8, po.qmin, po.qmax, ref.data()), 0);
            for (size_t i = 0; i < m * n; ++i) {
                const float v = float(acc[i]) * sab;
                const float want = float(o_u8 ? tq_nn_quantize_value_asymmetric(v, po.scale, po.zero_point, po.qmin, po.qmax)
                                              : tq_nn_quantize_value_symmetric(v, po.scale, po.qmin, po.qmax));
                CHECK(got.as_slice()[i] == want);
                CHECK(std::fabs(got.as_slice()[i] - ref[i]) <= 1.0f);
            }
        }
    }
    {
        const Tensor ta = Tensor::from_data(std::vector<float>(6, 1.0f), {2, 3}).unwrap();
        const Tensor tb = Tensor::from_data(std::vector<float>(8, 1.0f), {4, 2}).unwrap();
        const auto p = nq::QuantizationParams::symmetric(0.1f, DType::F32, DType::I8).unwrap();
        CHECK(nq::quantized_matmul_int8(ta, tb, p, p, p).is_err());  // K mismatch
        const Tensor big = Tensor::from_data(std::vector<float>(6, 300.0f), {3, 2}).unwrap();
        CHECK(nq::quantized_matmul_int8(ta, big, p, p, p).is_err());  // not an int8 carrier
        const auto pu = nq::QuantizationParams::asymmetric(0.1f, 3, DType::F32, DType::U8).unwrap();
        CHECK(nq::quantized_matmul_int8(ta, Tensor::from_data(std::vector<float>(6, 1.0f), {3, 2}).unwrap(), pu, p, p)
                  .unwrap_err().kind == TorshError::NotImplemented);
    }
    struct G { size_t nb, c, h, w, oc, k, stride, pad; bool in_u8, with_bias; };
    for (G g : {G{2, 3, 8, 8, 4, 3, 1, 1, true, true}, G{1, 32, 7, 7, 16, 3, 1, 1, false, true}, G{1, 16, 9, 9, 6, 3, 2, 1, true, false},
                G{2, 64, 6, 6, 32, 3, 1, 1, true, true}}) {
        const size_t nx = g.nb * g.c * g.h * g.w, nw = g.oc * g.c * g.k * g.k;
        std::vector<float> x(nx), w(nw), bias(g.oc);
        std::vector<uint8_t> xq(nx);
        std::vector<int8_t> wq(nw);
        for (size_t i = 0; i < nx; ++i) {
            const int q = g.in_u8 ? du8(rng) : d8(rng);
            x[i] = float(q);
            xq[i] = uint8_t(g.in_u8 ? q : int8_t(q));
        }
        for (size_t i = 0; i < nw; ++i) w[i] = float(wq[i] = int8_t(d8(rng)));
        for (size_t i = 0; i < g.oc; ++i) bias[i] = float(d8(rng));
        const auto px = g.in_u8 ? nq::QuantizationParams::asymmetric(0.02f, 117, DType::F32, DType::U8).unwrap()
                                : nq::QuantizationParams::symmetric(0.02f, DType::F32, DType::I8).unwrap();
        const auto pw = nq::QuantizationParams::symmetric(0.0009f, DType::F32, DType::I8).unwrap();
        const auto pbias = nq::QuantizationParams::symmetric(0.0005f, DType::F32, DType::I8).unwrap();
        const Tensor tx = Tensor::from_data(x, {g.nb, g.c, g.h, g.w}).unwrap();
        const Tensor tw = Tensor::from_data(w, {g.oc, g.c, g.k, g.k}).unwrap();
        const Tensor tbias = Tensor::from_data(bias, {g.oc}).unwrap();
        const size_t ho = (g.h + 2 * g.pad - g.k) / g.stride + 1, wo = (g.w + 2 * g.pad - g.k) / g.stride + 1;
        std::vector<int32_t> acc(g.nb * g.oc * ho * wo);
        CHECK_EQ(tq_backend_conv2d_i32(xq.data(), g.in_u8 ? 0 : 1, g.in_u8 ? px.zero_point : 0, wq.data(), g.nb, g.c, g.h,
                                       g.w, g.oc, g.k, g.k, g.stride, g.stride, g.pad, g.pad, acc.data()), 0);
        for (const auto &po : {nq::QuantizationParams::symmetric(0.04f, DType::F32, DType::I8).unwrap(),
                               nq::QuantizationParams::asymmetric(0.03f, 120, DType::F32, DType::U8).unwrap()}) {
            const bool o_u8 = po.dst_dtype == DType::U8;
            const Tensor got = nq::quantized_conv2d_int8(tx, tw, g.with_bias ? &tbias : nullptr, px, pw,
                                                         g.with_bias ? &pbias : nullptr, po, {g.stride, g.stride},
                                                         {g.pad, g.pad}).unwrap();
            CHECK(got.shape().dims() == (std::vector<size_t>{g.nb, g.oc, ho, wo}));
            std::vector<float> ref(acc.size());
            CHECK_EQ(tq_nn_quantized_conv2d_int8(x.data(), w.data(), g.with_bias ? bias.data() : nullptr, g.nb, g.c, g.h, g.w,
                                                 g.oc, g.k, g.k, g.stride, g.stride, g.pad, g.pad, px.scale, px.zero_point,
                                                 g.in_u8, pw.scale, 0, 0, pbias.scale, 0, 0, po.scale, po.zero_point, o_u8,
                                                 po.qmin, po.qmax, ref.data()), 0);
            for (size_t i = 0; i < acc.size(); ++i) {
                const size_t oc = (i / (ho * wo)) % g.oc;
                float v = float(acc[i]) * (px.scale * pw.scale);
                if (g.with_bias) v = v + bias[oc] * pbias.scale;
                const float want = float(o_u8 ? tq_nn_quantize_value_asymmetric(v, po.scale, po.zero_point, po.qmin, po.qmax)
                                              : tq_nn_quantize_value_symmetric(v, po.scale, po.qmin, po.qmax));
                CHECK(got.as_slice()[i] == want);
                CHECK(std::fabs(got.as_slice()[i] - ref[i]) <= 1.0f);
            }
        }
    }
    for (const auto &p : {nq::QuantizationParams::asymmetric(0.05f, 77, DType::F32, DType::U8).unwrap(),
                          nq::QuantizationParams::symmetric(0.05f, DType::F32, DType::I8).unwrap(),
                          nq::QuantizationParams::asymmetric(0.05f, 300, DType::F32, DType::U8).unwrap()}) {
        std::vector<float> x(5000);
        for (float &v : x) v = float(p.dst_dtype == DType::U8 ? du8(rng) : d8(rng));
        const Tensor t = tensor_1d(x).unwrap();
        const Tensor got = nq::quantized_relu_int8(t, p, p).unwrap();
        std::vector<float> want(x.size());
        CHECK_EQ(tq_nn_quantized_relu_int8(x.data(), x.size(), p.scale, p.zero_point, p.qmin, p.qmax, want.data()), 0);
        check_same(got.as_slice(), want, __LINE__);
    }
}

}  // namespace

int main(int argc, char **argv) {
    const bool cpu_only = argc > 1 && std::strcmp(argv[1], "--cpu-only") == 0;
    int failed = 0;
    for (const Case &c : cases()) {
        if (c.needs_gpu && cpu_only) {
            std::printf("skip %s\n", c.name);
            continue;
        }
        std::printf("run %s\n", c.name);
        std::fflush(stdout);
        try {
            c.fn();
            std::printf("ok %s\n", c.name);
        } catch (const Failure &f) {
            std::printf("FAIL %s: line %s\n", c.name, f.why.c_str());
            ++failed;
        } catch (const std::exception &e) {
            std::printf("FAIL %s: %s\n", c.name, e.what());
            ++failed;
        }
        std::fflush(stdout);
    }
    return failed ? 1 : 0;
}
