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
    check(zant_hip_sync(default_ctx()));
    std::printf(failures ? "host mirror: %d FAILED\n" : "host mirror: all passed\n", failures);
    return failures ? 1 : 0;
}
