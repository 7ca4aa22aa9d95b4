"""Pins the int8 family of the oracle.

The reference holds no quantised operators (its quantization.zig is empty), so these functions are
"parity unpinned by the reference"; what fixes them is the ONNX operator definitions, checked here through
exact int64 numpy accumulation, known answers on ties and saturation, scipy's correlate2d, and reductions
of one operator to another.
"""
import numpy as np
import pytest
import scipy.signal

from oracle import oracle as zo


def rng(seed):
    return np.random.default_rng(seed)


def np_qconv_acc(x, x_zp, w, bias, stride, pads, dil, group):
    """Exact int64 accumulation with numpy (ground truth for the accumulator)."""
    N, C, H, W = x.shape
    K, CG, KH, KW = w.shape
    xp = np.full((N, C, H + pads[0] + pads[2], W + pads[1] + pads[3]), x_zp, np.int64)
    xp[:, :, pads[0]:pads[0] + H, pads[1]:pads[1] + W] = x
    xp -= x_zp
    OH = (xp.shape[2] - ((KH - 1) * dil[0] + 1)) // stride[0] + 1
    OW = (xp.shape[3] - ((KW - 1) * dil[1] + 1)) // stride[1] + 1
    acc = np.zeros((N, K, OH, OW), np.int64)
    KG = K // group
    for k in range(K):
        g = k // KG
        for c in range(CG):
            for kh in range(KH):
                for kw in range(KW):
                    patch = xp[:, g * CG + c, kh * dil[0]: kh * dil[0] + (OH - 1) * stride[0] + 1: stride[0],
                               kw * dil[1]: kw * dil[1] + (OW - 1) * stride[1] + 1: stride[1]]
                    acc[:, k] += patch * int(w[k, c, kh, kw])
        if bias is not None:
            acc[:, k] += int(bias[k])
    return acc


QCASES = [
    # N, C, H, W, K, KH, KW, stride, pads, dil, group
    (2, 8, 7, 7, 6, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1),
    (1, 6, 9, 8, 4, 3, 3, (2, 2), (1, 1, 1, 1), (1, 1), 1),
    (2, 6, 8, 8, 6, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 6),   # depthwise
    (1, 8, 6, 6, 4, 3, 3, (2, 1), (0, 1, 2, 0), (1, 1), 2),   # grouped, asymmetric pads
    (1, 16, 5, 5, 8, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), 1),  # pointwise
    (1, 3, 9, 9, 5, 2, 2, (1, 1), (0, 0, 0, 0), (2, 2), 1),   # dilation
]


@pytest.mark.parametrize("case", QCASES)
def test_qconv_accumulator_exact(case):
    N, C, H, W, K, KH, KW, s, p, d, grp = case
    g = rng(abs(hash(case)) % 2**32)
    x = g.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = g.integers(-127, 128, (K, C // grp, KH, KW), dtype=np.int8)
    b = g.integers(-1000, 1001, K, dtype=np.int32)
    acc = zo.qconv_acc(x, 128, w, None, b, list(s), list(p), list(d), grp)
    ref = np_qconv_acc(x, 128, w, b, s, p, d, grp)
    np.testing.assert_array_equal(acc.astype(np.int64), ref)


def test_qconv_with_weight_zero_point():
    g = rng(2)
    x = g.integers(0, 256, (1, 4, 5, 5), dtype=np.uint8)
    w = g.integers(-127, 128, (3, 4, 3, 3), dtype=np.int8)
    wz = np.array([3, -5, 0], np.int8)
    acc = zo.qconv_acc(x, 7, w, wz, None, [1, 1], [1, 1, 1, 1], [1, 1])
    ref = np_qconv_acc(x, 7, w.astype(np.int64) - wz[:, None, None, None], None, (1, 1), (1, 1, 1, 1), (1, 1), 1)
    np.testing.assert_array_equal(acc.astype(np.int64), ref)


def test_depthwise_is_per_channel_correlate2d():
    g = rng(3)
    x = g.integers(0, 256, (1, 5, 9, 9), dtype=np.uint8)
    w = g.integers(-127, 128, (5, 1, 3, 3), dtype=np.int8)
    acc = zo.qconv_acc(x, 100, w, None, None, [1, 1], [1, 1, 1, 1], [1, 1], 5)
    for c in range(5):
        ref = scipy.signal.correlate2d(x[0, c].astype(np.int64) - 100, w[c, 0].astype(np.int64), mode="same",
                                       boundary="fill", fillvalue=0)
        np.testing.assert_array_equal(acc[0, c], ref)


def test_pointwise_is_an_integer_gemm():
    g = rng(4)
    x = g.integers(0, 256, (3, 16, 4, 4), dtype=np.uint8)
    w = g.integers(-127, 128, (8, 16, 1, 1), dtype=np.int8)
    acc = zo.qconv_acc(x, 128, w, None, None, [1, 1], [0, 0, 0, 0], [1, 1])
    xm = (x.astype(np.int64) - 128).transpose(0, 2, 3, 1).reshape(-1, 16)
    ref = (xm @ w[:, :, 0, 0].astype(np.int64).T).reshape(3, 4, 4, 8).transpose(0, 3, 1, 2)
    np.testing.assert_array_equal(acc, ref)


def test_qlinearconv_unit_scales_is_integer_conv_saturated():
    g = rng(5)
    x = g.integers(0, 20, (1, 2, 5, 5), dtype=np.uint8)
    w = g.integers(-3, 4, (2, 2, 3, 3), dtype=np.int8)
    y = zo.qlinearconv(x, 1.0, 0, w, [1.0], None, 1.0, 0, None, [1, 1], [1, 1, 1, 1], [1, 1])
    ref = np.clip(np_qconv_acc(x, 0, w, None, (1, 1), (1, 1, 1, 1), (1, 1), 1), 0, 255)
    np.testing.assert_array_equal(y, ref.astype(np.uint8))


def test_qlinearconv_requantisation_formula():
    g = rng(6)
    x = g.integers(0, 256, (2, 8, 6, 6), dtype=np.uint8)
    w = g.integers(-127, 128, (4, 8, 3, 3), dtype=np.int8)
    ws = g.uniform(0.001, 0.01, 4).astype(np.float32)
    b = g.integers(-1000, 1001, 4, dtype=np.int32)
    xs, ys = np.float32(0.02), np.float32(0.05)
    y = zo.qlinearconv(x, xs, 128, w, ws, None, ys, 128, b, [1, 1], [1, 1, 1, 1], [1, 1])
    acc = np_qconv_acc(x, 128, w, b, (1, 1), (1, 1, 1, 1), (1, 1), 1)
    m = ((xs * ws) / ys).astype(np.float32)  # one f32 multiplier per channel
    v = acc.astype(np.float32) * m[None, :, None, None]
    ref = np.clip(np.rint(v) + np.float32(128), 0, 255).astype(np.uint8)  # np.rint = round half to even
    np.testing.assert_array_equal(y, ref)
    assert ref.min() == 0 and ref.max() == 255  # both saturation ends are exercised


def test_round_half_even_and_saturation_known_answers():
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 3.5, 254.5, 255.5, 1000.0, -1000.0, 0.49999997], np.float32)
    y = zo.quantize_linear(x, 1.0, 0)
    np.testing.assert_array_equal(y, [0, 2, 2, 0, 0, 4, 254, 255, 255, 0, 0])
    y = zo.quantize_linear(np.array([-0.5, -1.5, -2.5], np.float32), 1.0, 10)
    np.testing.assert_array_equal(y, [10, 8, 8])
    # division, not multiplication by a reciprocal: 0.3f / 0.1f rounds to 3.0000002 -> 3; ties come from x/s
    y = zo.quantize_linear(np.array([0.25, 0.75], np.float32), np.float32(0.5), 0)
    np.testing.assert_array_equal(y, [0, 2])  # 0.5 -> 0, 1.5 -> 2


def test_quantize_per_axis_and_dequantize_roundtrip():
    g = rng(7)
    x = g.standard_normal((2, 3, 4, 4)).astype(np.float32)
    s = np.array([0.01, 0.02, 0.05], np.float32); zp = np.array([128, 100, 0], np.uint8)
    q = zo.quantize_linear(x, s, zp, axis=1)
    ref = np.clip(np.rint(x / s[None, :, None, None]) + zp[None, :, None, None].astype(np.float32), 0, 255).astype(np.uint8)
    np.testing.assert_array_equal(q, ref)
    d = zo.dequantize_linear(q, s, zp, axis=1)
    np.testing.assert_array_equal(d, (q.astype(np.int32) - zp[None, :, None, None]).astype(np.float32) * s[None, :, None, None])
    # quantize(dequantize(q)) is the identity on in-range codes
    np.testing.assert_array_equal(zo.quantize_linear(d, s, zp, axis=1), q)


def test_signed_and_int32_codes():
    """int8 QuantizeLinear saturates to [-128, 127] with the same rounding; int8 / int32 DequantizeLinear are (x - zp) * s."""
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 1000.0, -128.5, -129.5, -1000.0], np.float32)
    y = zo.quantize_linear(x, 1.0, None, signed=True)
    assert y.dtype == np.int8
    np.testing.assert_array_equal(y, [0, 2, 2, 0, -2, -2, 126, 127, 127, -128, -128, -128])
    np.testing.assert_array_equal(zo.quantize_linear(x[:4], 1.0, np.array([-3], np.int8)), [-3, -1, -1, -3])
    g = rng(11)
    v = g.standard_normal((2, 3, 5)).astype(np.float32) * 4
    s = np.array([0.02, 0.05, 0.1], np.float32); zp = np.array([-5, 0, 17], np.int8)
    q = zo.quantize_linear(v, s, zp, axis=1)
    ref = np.clip(np.rint(v / s[None, :, None]) + zp[None, :, None].astype(np.float32), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(q, ref)
    d = zo.dequantize_linear(q, s, zp, axis=1)
    np.testing.assert_array_equal(d, (q.astype(np.int32) - zp[None, :, None]).astype(np.float32) * s[None, :, None])
    np.testing.assert_array_equal(zo.quantize_linear(d, s, zp, axis=1), q)  # identity on in-range codes
    acc = np.array([0, 1, -1, 2**31 - 1, -2**31, 123456789], np.int32)
    np.testing.assert_array_equal(zo.dequantize_linear(acc, np.float32(0.5)), acc.astype(np.float64).astype(np.float32) * np.float32(0.5))
    # the difference cannot wrap: (2^31 - 1) - (-2^31) = 2^32 - 1
    z = zo.dequantize_linear(np.array([2**31 - 1], np.int32), np.float32(1.0), np.array([-2**31], np.int32))
    assert z[0] == np.float32(2.0**32)


@pytest.mark.parametrize("act,alpha", [("relu", 0.0), ("leaky", 0.1), ("relu6", 0.0), (None, 0.0)])
def test_qlinear_act_matches_dequant_act_quant(act, alpha):
    q = np.arange(256, dtype=np.uint8)
    xs, xz, ys, yz = np.float32(0.05), 128, np.float32(0.03), 20
    y = zo.qlinear_act(q, xs, xz, act, alpha, ys, yz)
    f = zo.dequantize_linear(q, xs, xz)
    if act == "relu":
        f = np.maximum(f, 0)
    elif act == "leaky":
        f = np.where(f <= 0, np.float32(alpha) * f, f).astype(np.float32)
    elif act == "relu6":
        f = np.clip(f, 0, 6)
    np.testing.assert_array_equal(y, zo.quantize_linear(f, ys, yz))
    assert np.all(np.diff(y.astype(int)) >= 0)  # monotone


def test_fused_conv_act_equals_unfused_sequence():
    g = rng(8)
    x = g.integers(0, 256, (1, 4, 6, 6), dtype=np.uint8)
    w = g.integers(-127, 128, (4, 4, 3, 3), dtype=np.int8)
    ws = g.uniform(0.001, 0.01, 4).astype(np.float32)
    args = (x, 0.02, 128, w, ws, None, 0.05, 128, None, [1, 1], [1, 1, 1, 1], [1, 1])
    fused = zo.qlinearconv(*args, act="leaky", act_alpha=0.1, act_scale=0.04, act_zp=30)
    plain = zo.qlinearconv(*args)
    np.testing.assert_array_equal(fused, zo.qlinear_act(plain, 0.05, 128, "leaky", 0.1, 0.04, 30))


def test_qlinear_add():
    g = rng(9)
    a = g.integers(0, 256, 4096, dtype=np.uint8); b = g.integers(0, 256, 4096, dtype=np.uint8)
    y = zo.qlinear_add(a, 0.02, 128, b, 0.03, 120, 0.04, 125)
    fa = (a.astype(np.int32) - 128).astype(np.float32) * np.float32(0.02)
    fb = (b.astype(np.int32) - 120).astype(np.float32) * np.float32(0.03)
    ref = np.clip(np.rint((fa + fb) / np.float32(0.04)) + np.float32(125), 0, 255).astype(np.uint8)
    np.testing.assert_array_equal(y, ref)
    # same scale and zero point on all three => integer addition around the zero point
    y = zo.qlinear_add(a, 0.5, 128, b, 0.5, 128, 0.5, 128)
    np.testing.assert_array_equal(y, np.clip(a.astype(int) + b.astype(int) - 128, 0, 255))


def test_qlinear_global_avgpool():
    g = rng(10)
    x = g.integers(0, 256, (3, 5, 3, 3), dtype=np.uint8)
    y = zo.qlinear_global_avgpool(x, 0.05, 128, 0.02, 110)
    s = (x.astype(np.int64) - 128).sum(axis=(2, 3))
    mean = (s.astype(np.float32) * np.float32(0.05)) / np.float32(9)
    ref = np.clip(np.rint(mean / np.float32(0.02)) + np.float32(110), 0, 255).astype(np.uint8)
    np.testing.assert_array_equal(y[:, :, 0, 0], ref)
    const = np.full((1, 2, 4, 4), 200, np.uint8)  # mean of a constant is the constant
    np.testing.assert_array_equal(zo.qlinear_global_avgpool(const, 0.1, 128, 0.1, 128).ravel(), [200, 200])
