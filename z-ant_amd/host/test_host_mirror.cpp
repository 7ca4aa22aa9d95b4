// The reference's own operator tests, restated against the C++ host mirror (runs on the GPU).
// Each block cites the Zig test it mirrors; expected values are the reference's.
#include <cmath>
#include <cstdio>
#include <cstdlib>

#include "zant_tensor_math.hpp"

using namespace zant;
using tensMath::Dims;

static int failures = 0;
#define EXPECT(cond)                                                            \
    do {                                                                        \
        if (!(cond)) { std::printf("FAIL %s:%d %s\n", __FILE__, __LINE__, #cond); ++failures; } \
    } while (0)
template <typename F>
static int error_of(F f) {
    try { f(); } catch (const Error &e) { return e.code(); }
    return ZANT_OK;
}

int main() {
    {   // tests/Core/Tensor/TensorMath/test_op_convolution.zig:654-709  "OnnxConvLean - NOTSET padding"
        std::vector<float> ones(25, 1.0f), k(9, 1.0f);
        auto x = Tensor<float>::fromArray(ones.data(), {1, 1, 5, 5});
        auto w = Tensor<float>::fromArray(k.data(), {1, 1, 3, 3});
        auto y = Tensor<float>::fromShape({1, 1, 3, 3});
        Dims pads{0, 0, 0, 0};
        tensMath::conv_lean(&x, &w, &y, nullptr, {1}, &pads, nullptr, std::nullopt, nullptr);
        for (float v : y.toHost()) EXPECT(v == 9.0f);
    }
    {   // test_op_convolution.zig:931-987  Conv with SAME_UPPER
        std::vector<float> ones(25, 1.0f), k(9, 1.0f);
        auto x = Tensor<float>::fromArray(ones.data(), {1, 1, 5, 5});
        auto w = Tensor<float>::fromArray(k.data(), {1, 1, 3, 3});
        auto y = tensMath::Conv(&x, &w, nullptr, {1}, nullptr, nullptr, std::nullopt, "SAME_UPPER");
        const float expect[25] = {4, 6, 6, 6, 4, 6, 9, 9, 9, 6, 6, 9, 9, 9, 6, 6, 9, 9, 9, 6, 4, 6, 6, 6, 4};
        auto h = y.toHost();
        EXPECT(y.shape == Dims({1, 1, 5, 5}));
        for (int i = 0; i < 25; ++i) EXPECT(h[i] == expect[i]);
    }
    {   // test_op_convolution.zig:989-1042  bias and dilation
        std::vector<float> ones(25, 1.0f), k(4, 1.0f), b{1.0f};
        auto x = Tensor<float>::fromArray(ones.data(), {1, 1, 5, 5});
        auto w = Tensor<float>::fromArray(k.data(), {1, 1, 2, 2});
        auto bias = Tensor<float>::fromArray(b.data(), {1});
        Dims dil{2};
        auto y = tensMath::Conv(&x, &w, &bias, {1}, nullptr, &dil, std::nullopt, nullptr);
        EXPECT(y.shape == Dims({1, 1, 3, 3}));
        for (float v : y.toHost()) EXPECT(v == 5.0f);
    }
    {   // group != 1 is rejected: op_convolution.zig:59-65
        auto x = Tensor<float>::fromShape({1, 2, 4, 4});
        auto w = Tensor<float>::fromShape({2, 1, 3, 3});
        auto y = Tensor<float>::fromShape({1, 2, 2, 2});
        EXPECT(error_of([&] { tensMath::conv_lean(&x, &w, &y, nullptr, {1, 1}, nullptr, nullptr, 2, nullptr); }) == ZANT_InvalidDimensions);
    }
    {   // test_op_gemm.zig:109-144  alpha 2, beta 3, transB
        float a[9] = {1, 2, 3, 4, 5, 6, 7, 8, 9}, b[6] = {1, 4, 7, 2, 5, 8}, c[2] = {1, 2};
        auto A = Tensor<float>::fromArray(a, {1, 1, 3, 3});
        auto B = Tensor<float>::fromArray(b, {1, 1, 2, 3});
        auto C = Tensor<float>::fromArray(c, {1, 1, 1, 2});
        auto Y = tensMath::gemm(&A, &B, &C, 2, 3, false, true);
        auto h = Y.toHost();
        EXPECT(h[0] == 63.0f && h[5] == 258.0f);
    }
    {   // test_op_gemm.zig:280-335 error cases
        auto t3 = Tensor<float>::fromShape({1, 2, 2});
        EXPECT(error_of([&] { tensMath::gemm(&t3, &t3, nullptr, 1, 1, false, false); }) == ZANT_InputTensorsWrongShape);
        auto a = Tensor<float>::fromShape({2, 1, 2, 2});
        auto b = Tensor<float>::fromShape({1, 2, 2, 2});
        EXPECT(error_of([&] { tensMath::gemm(&a, &b, nullptr, 1, 1, false, false); }) == ZANT_InputTensorDifferentShape);
        auto c = Tensor<float>::fromShape({4, 4, 2, 2});
        auto d = Tensor<float>::fromShape({4, 4, 3, 2});
        EXPECT(error_of([&] { tensMath::gemm(&c, &d, nullptr, 1, 1, false, false); }) == ZANT_InputTensorDimensionMismatch);
    }
    {   // test_op_mat_mul.zig:9-64
        float a[4] = {1, 2, 4, 5};
        auto A = Tensor<float>::fromArray(a, {2, 2});
        auto Y = tensMath::mat_mul(&A, &A);
        auto h = Y.toHost();
        EXPECT(h[0] == 9.0f && h[1] == 12.0f);
        auto B = Tensor<float>::fromShape({3, 2});
        EXPECT(error_of([&] { tensMath::mat_mul(&A, &B); }) == ZANT_InputTensorsWrongShape);
    }
    {   // test_op_pooling.zig:353-416 explicit padding
        float v[9] = {1, 2, 3, 4, 5, 6, 7, 8, 9};
        auto x = Tensor<float>::fromArray(v, {1, 1, 3, 3});
        auto y = tensMath::onnx_maxpool<float>(&x, {2, 2}, {1, 1}, {1, 1}, {1, 1, 1, 1}, AutoPadType::NOTSET, false);
        const float expect[16] = {1, 2, 3, 3, 4, 5, 6, 6, 7, 8, 9, 9, 7, 8, 9, 9};
        auto h = y.toHost();
        EXPECT(y.shape == Dims({1, 1, 4, 4}));
        for (int i = 0; i < 16; ++i) EXPECT(h[i] == expect[i]);
    }
    {   // tests/Model/test_activation_function.zig:13-36, 265-287, 153-175
        float v[4] = {1, -2, -4, 5};
        auto x = Tensor<float>::fromArray(v, {2, 2});
        auto r = tensMath::ReLU(&x).toHost();
        EXPECT(r[0] > 0 && r[1] == 0 && r[2] == 0 && r[3] > 0);
        auto l = tensMath::leakyReLU(&x, 0.01f).toHost();
        EXPECT(l[0] == 1.0f && std::fabs(l[1] + 0.02f) < 1e-5f && std::fabs(l[2] + 0.04f) < 1e-5f && l[3] == 5.0f);
        float z[4] = {0, 0, 0, 0};
        auto zt = Tensor<float>::fromArray(z, {2, 2});
        auto s = tensMath::softmax(&zt).toHost();
        EXPECT(s[0] == s[1] && s[2] == s[3]);
    }
    {   // test_lib_elementWise_math.zig:90-115 add_bias; test_lib_shape_math.zig:1808-1836 reshape with -1
        float v[6] = {1, 2, 3, 4, 5, 6}, b[3] = {1, 1, 1};
        auto t = Tensor<float>::fromArray(v, {2, 3});
        auto bias = Tensor<float>::fromArray(b, {3});
        tensMath::add_bias(&t, &bias);
        auto h = t.toHost();
        for (int i = 0; i < 6; ++i) EXPECT(h[i] == v[i] + 1);
        auto out = Tensor<float>::fromShape({6});
        tensMath::reshape_lean<float>(&t, {3, -1}, std::nullopt, &out);
        EXPECT(out.shape == Dims({3, 2}));
        EXPECT(error_of([&] { tensMath::reshape_lean<float>(&t, {-1, -1}, std::nullopt, &out); }) == ZANT_InvalidInput);
    }
    {   // tests/Model/test_activation_function.zig:210-227 sigmoid; test_lib_reduction_math.zig:45-61, 126-155 reduce_mean
        float v[3] = {0, 2, -2};
        auto x = Tensor<float>::fromArray(v, {3});
        auto s = tensMath::sigmoid(&x).toHost();
        EXPECT(std::fabs(s[0] - 0.5f) < 1e-6f && std::fabs(s[1] - 0.880797f) < 1e-6f && std::fabs(s[2] - 0.119203f) < 1e-6f);
        float w[24];
        for (int i = 0; i < 24; ++i) w[i] = float(i + 1);
        auto t = Tensor<float>::fromArray(w, {2, 2, 2});
        Dims axes = {1, 2};
        auto m = tensMath::reduce_mean(&t, &axes, false, false);
        auto h = m.toHost();
        EXPECT(m.shape == Dims({2}) && std::fabs(h[0] - 2.5f) < 1e-4f && std::fabs(h[1] - 6.5f) < 1e-4f);
        auto t3 = Tensor<float>::fromArray(w, {2, 3, 4});
        Dims axes02 = {0, 2};
        auto m3 = tensMath::reduce_mean(&t3, &axes02, true, false);
        auto h3 = m3.toHost();
        EXPECT(m3.shape == Dims({1, 3, 1}) && std::fabs(h3[0] - 8.5f) < 1e-4f && std::fabs(h3[2] - 16.5f) < 1e-4f);
        Dims bad = {3};
        EXPECT(error_of([&] { tensMath::reduce_mean(&t3, &bad, true, false); }) == ZANT_InvalidAxes);
    }
    {   // test_lib_shape_math.zig:139-192 concat along axis 2, :2182-2255 errors; :480-499, 596-627 resize
        float a[8] = {1, 2, 3, 4, 5, 6, 7, 8}, b[12];
        for (int i = 0; i < 12; ++i) b[i] = float(9 + i);
        auto A = Tensor<float>::fromArray(a, {2, 2, 2});
        auto B = Tensor<float>::fromArray(b, {2, 2, 3});
        auto Y = tensMath::concatenate<float>({&A, &B}, 2);
        const float expect[20] = {1, 2, 9, 10, 11, 3, 4, 12, 13, 14, 5, 6, 15, 16, 17, 7, 8, 18, 19, 20};
        auto h = Y.toHost();
        EXPECT(Y.shape == Dims({2, 2, 5}));
        for (int i = 0; i < 20; ++i) EXPECT(h[i] == expect[i]);
        EXPECT(error_of([&] { tensMath::concatenate<float>({&A, &B}, 0); }) == ZANT_MismatchedShape);
        EXPECT(error_of([&] { tensMath::concatenate<float>({&A, &A}, 3); }) == ZANT_AxisOutOfBounds);
        EXPECT(error_of([&] { tensMath::concatenate<float>({}, 0); }) == ZANT_EmptyTensorList);
        uint8_t u[4] = {1, 2, 3, 4};
        auto U = Tensor<uint8_t>::fromArray(u, {4});
        std::vector<float> scales = {2.0f};
        auto R = tensMath::resize<uint8_t>(&U, "nearest", &scales, nullptr, "half_pixel");
        auto r = R.toHost();
        EXPECT(R.size == 8 && r[0] == 1 && r[1] == 1 && r[2] == 2 && r[3] == 2);
        Dims sizes = {8};
        EXPECT(error_of([&] { tensMath::resize<uint8_t>(&U, "invalid_mode", &scales, nullptr, "half_pixel"); }) == ZANT_UnsupportedMode);
        EXPECT(error_of([&] { tensMath::resize<uint8_t>(&U, "nearest", &scales, &sizes, "half_pixel"); }) == ZANT_InvalidInput);
        EXPECT(error_of([&] { tensMath::resize<uint8_t>(&U, "nearest", nullptr, nullptr, "half_pixel"); }) == ZANT_InvalidInput);
    }
    {   // QuantizeLinear / DequantizeLinear (ONNX; the reference holds no test): ties round to even, results saturate
        float v[8] = {0.5f, 1.5f, 2.5f, -0.5f, 300.0f, -300.0f, 3.49f, 126.5f}, one[1] = {1.0f};
        uint8_t zp0[1] = {0}, zp128[1] = {128};
        auto x = Tensor<float>::fromArray(v, {8});
        auto sc = Tensor<float>::fromArray(one, {1});
        auto z0 = Tensor<uint8_t>::fromArray(zp0, {1});
        auto z128 = Tensor<uint8_t>::fromArray(zp128, {1});
        auto q = tensMath::quantize_linear<uint8_t>(&x, &sc, &z0, 0).toHost();
        const uint8_t e0[8] = {0, 2, 2, 0, 255, 0, 3, 126};
        for (int i = 0; i < 8; ++i) EXPECT(q[i] == e0[i]);
        auto q128 = tensMath::quantize_linear<uint8_t>(&x, &sc, &z128, 0).toHost();
        const uint8_t e128[8] = {128, 130, 130, 128, 255, 0, 131, 254};
        for (int i = 0; i < 8; ++i) EXPECT(q128[i] == e128[i]);
        auto qs = tensMath::quantize_linear<int8_t>(&x, &sc, nullptr, 0).toHost();
        const int8_t es[8] = {0, 2, 2, 0, 127, -128, 3, 126};
        for (int i = 0; i < 8; ++i) EXPECT(qs[i] == es[i]);
        // per-axis scales: rows of a [2, 3] tensor quantised with scales {0.5, 2}; then dequantised with the same
        float m[6] = {1, 2, 3, 4, 5, 6}, sc2[2] = {0.5f, 2.0f};
        auto xm = Tensor<float>::fromArray(m, {2, 3});
        auto s2 = Tensor<float>::fromArray(sc2, {2});
        auto qm = tensMath::quantize_linear<uint8_t>(&xm, &s2, nullptr, 0);
        auto hm = qm.toHost();
        const uint8_t em[6] = {2, 4, 6, 2, 2, 3};  // 4/2 = 2, 5/2 = 2.5 -> 2, 6/2 = 3
        for (int i = 0; i < 6; ++i) EXPECT(hm[i] == em[i]);
        auto dm = tensMath::dequantize_linear<uint8_t>(&qm, &s2, nullptr, -2).toHost();  // axis -2 = 0
        const float ed[6] = {1, 2, 3, 4, 4, 6};
        for (int i = 0; i < 6; ++i) EXPECT(dm[i] == ed[i]);
        int32_t acc[3] = {-4, 0, 1000};
        int32_t azp[1] = {-2};
        auto a = Tensor<int32_t>::fromArray(acc, {3});
        auto az = Tensor<int32_t>::fromArray(azp, {1});
        float half[1] = {0.5f};
        auto sh = Tensor<float>::fromArray(half, {1});
        auto da = tensMath::dequantize_linear<int32_t>(&a, &sh, &az, 0).toHost();
        EXPECT(da[0] == -1.0f && da[1] == 1.0f && da[2] == 501.0f);
    }
    {   // QLinearConv (ONNX): with unit scales and zero zero-points it is the integer convolution: ones * ones counts
        // the taps inside the image (the f32 known answer of test_op_convolution.zig:711-812 on integer codes); with
        // x_zero_point 128 a padding pixel holds the zero point and contributes nothing
        std::vector<uint8_t> ones(25, 1), x130(25, 130);
        std::vector<int8_t> k(9, 1);
        float one[1] = {1.0f};
        auto w = Tensor<int8_t>::fromArray(k.data(), {1, 1, 3, 3});
        auto ws = Tensor<float>::fromArray(one, {1});
        Dims pads{1, 1, 1, 1};
        const uint8_t expect[25] = {4, 6, 6, 6, 4, 6, 9, 9, 9, 6, 6, 9, 9, 9, 6, 6, 9, 9, 9, 6, 4, 6, 6, 6, 4};
        auto x = Tensor<uint8_t>::fromArray(ones.data(), {1, 1, 5, 5});
        auto y = tensMath::qlinearconv(&x, 1.0f, 0, &w, &ws, nullptr, 1.0f, 0, nullptr, {1}, &pads, nullptr, std::nullopt);
        EXPECT(y.shape == Dims({1, 1, 5, 5}));
        auto h = y.toHost();
        for (int i = 0; i < 25; ++i) EXPECT(h[i] == expect[i]);
        auto x2 = Tensor<uint8_t>::fromArray(x130.data(), {1, 1, 5, 5});  // every pixel is +2 after the zero point
        int32_t bv[1] = {-3};
        auto b = Tensor<int32_t>::fromArray(bv, {1});
        auto y2 = tensMath::qlinearconv(&x2, 1.0f, 128, &w, &ws, nullptr, 1.0f, 10, &b, {1, 1}, &pads, nullptr, 1).toHost();
        for (int i = 0; i < 25; ++i) EXPECT(y2[i] == 2 * expect[i] - 3 + 10);
        // the same through a plan, twice (the second run reuses what the first packed)
        tensMath::QLinearConvPlan plan({1, 1, 5, 5}, 1.0f, 128, &w, &ws, nullptr, 1.0f, 10, &b, {1, 1, 5, 5}, {1, 1}, &pads, nullptr, 1);
        auto yp = Tensor<uint8_t>::fromShape({1, 1, 5, 5});
        for (int rep = 0; rep < 2; ++rep) {
            plan.run(x2.data, yp.data);
            auto hp = yp.toHost();
            for (int i = 0; i < 25; ++i) EXPECT(hp[i] == 2 * expect[i] - 3 + 10);
        }
        // depthwise: group == channels, each channel with its own filter (1s and 2s)
        std::vector<uint8_t> two_ch(50, 1);
        std::vector<int8_t> kd(18, 1);
        for (int i = 9; i < 18; ++i) kd[size_t(i)] = 2;
        auto xd = Tensor<uint8_t>::fromArray(two_ch.data(), {1, 2, 5, 5});
        auto wd = Tensor<int8_t>::fromArray(kd.data(), {2, 1, 3, 3});
        auto yd = tensMath::qlinearconv(&xd, 1.0f, 0, &wd, &ws, nullptr, 1.0f, 0, nullptr, {1, 1}, &pads, nullptr, 2).toHost();
        for (int i = 0; i < 25; ++i) EXPECT(yd[i] == expect[i] && yd[25 + i] == 2 * expect[i]);
        // errors: a group that does not divide the channels, negative padding through the plan
        EXPECT(error_of([&] { tensMath::qlinearconv(&xd, 1.0f, 0, &wd, &ws, nullptr, 1.0f, 0, nullptr, {1, 1}, &pads, nullptr, 3); }) == ZANT_InvalidDimensions);
        Dims neg{-1, 0, 0, 0};
        EXPECT(error_of([&] { tensMath::QLinearConvPlan bad({1, 1, 5, 5}, 1.0f, 0, &w, &ws, nullptr, 1.0f, 0, nullptr, {1, 1, 5, 5}, {1, 1}, &neg, nullptr, 1); }) == ZANT_InvalidPadding);
        // MaxPool on quantised values (test_op_pooling.zig:156-202 on integer codes)
        uint8_t pv[16];
        for (int i = 0; i < 16; ++i) pv[i] = uint8_t(i + 1);
        auto px = Tensor<uint8_t>::fromArray(pv, {1, 1, 4, 4});
        auto py = tensMath::onnx_maxpool<uint8_t>(&px, {2, 2}, {2, 2}, {1, 1}, {0, 0, 0, 0}, AutoPadType::NOTSET, false).toHost();
        EXPECT(py[0] == 6 && py[1] == 8 && py[2] == 14 && py[3] == 16);
    }
    {   // conv_lean through a plan (test_op_convolution.zig:654-709 twice)
        std::vector<float> ones(25, 1.0f), k(9, 1.0f);
        auto x = Tensor<float>::fromArray(ones.data(), {1, 1, 5, 5});
        auto w = Tensor<float>::fromArray(k.data(), {1, 1, 3, 3});
        auto y = Tensor<float>::fromShape({1, 1, 3, 3});
        Dims pads{0, 0, 0, 0};
        tensMath::ConvPlan plan({1, 1, 5, 5}, &w, nullptr, {1, 1, 3, 3}, {1}, &pads, nullptr, std::nullopt, nullptr);
        for (int rep = 0; rep < 2; ++rep) {
            plan.run(x.data, y.data);
            for (float v : y.toHost()) EXPECT(v == 9.0f);
        }
        EXPECT(error_of([&] { tensMath::ConvPlan bad({1, 1, 5, 5}, &w, nullptr, {1, 1, 4, 4}, {1}, &pads, nullptr, std::nullopt, nullptr); }) == ZANT_InvalidDimensions);
    }
    check(zant_hip_sync(default_ctx()));
    std::printf(failures ? "host mirror: %d FAILED\n" : "host mirror: all passed\n", failures);
    return failures ? 1 : 0;
}
