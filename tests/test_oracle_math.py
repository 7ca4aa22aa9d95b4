"""Pins the f32 oracle where the reference's fixtures leave room: brute force, library routines, closed forms.

Each check is chosen so that a plausible slip (transposed weight matrix, dropped bias, wrong pad side,
swapped stride axes, wrong broadcast axis) fails it.
"""
import numpy as np
import pytest
import scipy.special
import torch
import torch.nn.functional as F

from oracle import oracle as zo

RTOL, ATOL = 1e-4, 1e-5  # the f32 tolerance of the hot path


def rng(seed):
    return np.random.default_rng(seed)


CONV_CASES = [
    # N, C, H, W, K, KH, KW, stride, pads(t,l,b,r), dil
    (2, 3, 7, 9, 4, 3, 3, (1, 1), (0, 0, 0, 0), (1, 1)),
    (1, 5, 8, 8, 6, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1)),
    (2, 4, 9, 7, 3, 3, 2, (2, 1), (1, 0, 2, 1), (1, 1)),   # asymmetric pads, rectangular kernel + stride
    (1, 2, 11, 10, 5, 2, 3, (1, 2), (0, 2, 1, 0), (2, 1)),  # dilation on one axis
    (3, 1, 6, 6, 2, 5, 5, (1, 1), (2, 2, 2, 2), (1, 1)),   # kernel_w >= 4 (im2col vector branch in the reference)
    (1, 8, 5, 5, 8, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1)),   # 1x1
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_vs_brute_force_and_torch(case):
    N, C, H, W, K, KH, KW, s, p, d = case
    g = rng(hash(case) % 2**32)
    x = g.standard_normal((N, C, H, W), dtype=np.float32)
    w = g.standard_normal((K, C, KH, KW), dtype=np.float32)
    b = g.standard_normal(K, dtype=np.float32)
    y = zo.Conv(x, w, b, list(s), list(p), list(d), 1, "NOTSET")
    ref = zo.conv_direct(x, w, b, list(s), list(p), list(d))
    assert y.shape == ref.shape
    np.testing.assert_allclose(y, ref, rtol=RTOL, atol=ATOL)
    # independent library routine (explicit asymmetric pad via F.pad)
    xt = F.pad(torch.from_numpy(x), (p[1], p[3], p[0], p[2]))
    yt = F.conv2d(xt, torch.from_numpy(w), torch.from_numpy(b), stride=s, dilation=d).numpy()
    np.testing.assert_allclose(y, yt, rtol=RTOL, atol=ATOL)


def test_conv_delta_kernel_is_a_shift():
    g = rng(1)
    x = g.standard_normal((1, 1, 6, 6), dtype=np.float32)
    w = np.zeros((1, 1, 3, 3), np.float32)
    w[0, 0, 0, 2] = 1.0  # tap (kh=0, kw=2): y[oh,ow] = x[oh, ow+2]  (correlation, not flipped)
    y = zo.Conv(x, w, None, [1, 1], [0, 0, 0, 0], None, 1, "NOTSET")
    np.testing.assert_array_equal(y[0, 0], x[0, 0, 0:4, 2:6])


@pytest.mark.parametrize("mode", ["SAME_UPPER", "SAME_LOWER"])
def test_conv_same_padding_side(mode):
    # even kernel => total pad 1: UPPER pads the end, LOWER the beginning (op_convolution.zig:100-110)
    x = np.arange(16, dtype=np.float32).reshape(1, 1, 4, 4) + 1
    w = np.ones((1, 1, 2, 2), np.float32)
    y = zo.Conv(x, w, None, [1, 1], None, None, 1, mode)
    pads = [0, 0, 1, 1] if mode == "SAME_UPPER" else [1, 1, 0, 0]
    ref = zo.conv_direct(x, w, None, [1, 1], pads, [1, 1])
    assert y.shape == (1, 1, 4, 4)
    np.testing.assert_array_equal(y, ref)


def test_conv_same_with_stride():
    g = rng(7)
    x = g.standard_normal((1, 2, 7, 7), dtype=np.float32)
    w = g.standard_normal((3, 2, 3, 3), dtype=np.float32)
    y = zo.Conv(x, w, None, [2, 2], None, None, 1, "SAME_UPPER")
    assert y.shape == (1, 3, 4, 4)  # ceil(7/2); total pad = 3*2+3-7 = 2 -> 1,1
    np.testing.assert_allclose(y, zo.conv_direct(x, w, None, [2, 2], [1, 1, 1, 1], [1, 1]), rtol=RTOL, atol=ATOL)


def test_conv_accumulation_order_is_k_ascending_then_bias():
    # 1e8 + 1 - 1e8 depends on the order: k ascending gives (1e8 + 1) - 1e8 = 0 in f32, then + bias
    x = np.array([1e8, 1.0, -1e8], np.float32).reshape(1, 3, 1, 1)
    w = np.ones((1, 3, 1, 1), np.float32)
    y = zo.Conv(x, w, np.array([0.5], np.float32), [1, 1], None, None, 1, None)
    assert y.ravel()[0] == np.float32(0.5)


def test_matmul_vs_numpy_and_identities():
    g = rng(3)
    a = g.standard_normal((37, 53), dtype=np.float32)
    b = g.standard_normal((53, 29), dtype=np.float32)  # 29 = 3*8 + 5: vector body and scalar tail
    y = zo.mat_mul(a, b)
    np.testing.assert_allclose(y, a.astype(np.float64) @ b.astype(np.float64), rtol=RTOL, atol=ATOL)
    np.testing.assert_array_equal(zo.mat_mul(a, np.eye(53, dtype=np.float32)), a)
    # leading dims are ignored: only the first matrix is multiplied (op_mat_mul.zig:93-97)
    a4 = np.stack([a, 2 * a])[None]
    b4 = np.stack([b, 3 * b])[None]
    y4 = np.full((1, 2, 37, 29), -1.0, np.float32)
    zo.mat_mul_lean(a4, b4, y4)
    np.testing.assert_array_equal(y4[0, 0], y)
    assert np.all(y4[0, 1] == -1.0)


def test_matmul_k_ascending_separate_mul_add():
    a = np.array([[1e8, 1.0, -1e8]], np.float32)
    b = np.ones((3, 1), np.float32)
    assert zo.mat_mul(a, b)[0, 0] == np.float32(0.0)
    # a fused multiply-add would keep the low bits of 0.1f*0.1f; separate rounding does not
    p = np.float32(0.1) * np.float32(0.1)
    a = np.array([[0.1, 1.0]], np.float32)
    b = np.array([[0.1], [-float(p)]], np.float32)
    assert zo.mat_mul(a, b)[0, 0] == np.float32(0.0)


@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_gemm_vs_numpy(ta, tb):
    g = rng(10 + 2 * ta + tb)
    M, K, N = 9, 13, 11
    a = g.standard_normal((1, 1, K, M) if ta else (1, 1, M, K), dtype=np.float32)
    b = g.standard_normal((1, 1, N, K) if tb else (1, 1, K, N), dtype=np.float32)
    for cshape in [(1, 1, M, N), (1, 1, 1, N), (1, 1, M, 1), (1, 1, 1, 1)]:
        c = g.standard_normal(cshape, dtype=np.float32)
        y = zo.gemm(a, b, c, 0.75, -1.5, ta, tb)
        A = a[0, 0].T if ta else a[0, 0]
        B = b[0, 0].T if tb else b[0, 0]
        ref = 0.75 * (A.astype(np.float64) @ B.astype(np.float64)) + (-1.5) * c[0, 0].astype(np.float64)
        np.testing.assert_allclose(y[0, 0], ref, rtol=RTOL, atol=ATOL)
    y0 = zo.gemm(a, b, c, 1.0, 0.0, ta, tb)  # beta == 0 skips C (op_gemm.zig:139)
    np.testing.assert_allclose(y0[0, 0], A.astype(np.float64) @ B.astype(np.float64), rtol=RTOL, atol=ATOL)


def test_gemm_bad_c():
    a = np.zeros((1, 1, 2, 3), np.float32); b = np.zeros((1, 1, 3, 4), np.float32)
    with pytest.raises(zo.OracleError) as e:
        zo.gemm(a, b, np.zeros((1, 1, 3, 4), np.float32), 1, 1, 0, 0)
    assert e.value.name == "IncompatibleBroadcastShapes"
    with pytest.raises(zo.OracleError) as e:
        zo.gemm(a, b, np.zeros((2, 4), np.float32), 1, 1, 0, 0)
    assert e.value.name == "InputTensorsWrongShape"


@pytest.mark.parametrize("k,s,d,p", [((2, 2), (2, 2), (1, 1), (0, 0, 0, 0)), ((3, 3), (2, 2), (1, 1), (1, 1, 1, 1)),
                                     ((3, 2), (1, 2), (2, 1), (0, 1, 2, 0)), ((3, 3), (3, 3), (1, 1), (0, 0, 0, 0))])
def test_maxpool_vs_torch(k, s, d, p):
    g = rng(5)
    x = g.standard_normal((2, 3, 13, 11), dtype=np.float32)
    y = zo.onnx_maxpool(x, list(k), list(s), list(d), list(p), "NOTSET", False)
    xt = F.pad(torch.from_numpy(x), (p[1], p[3], p[0], p[2]), value=float("-inf"))
    yt = F.max_pool2d(xt, k, s, 0, d).numpy()
    np.testing.assert_array_equal(y, yt)


def test_maxpool_u8_commutes_with_dequantize():
    g = rng(6)
    q = g.integers(0, 256, (2, 3, 8, 8), dtype=np.uint8)
    a = zo.onnx_maxpool(q, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    b = zo.onnx_maxpool(zo.dequantize_linear(q, 0.05, 128), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    np.testing.assert_array_equal(zo.dequantize_linear(a, 0.05, 128), b)


def test_softmax_vs_scipy_and_shift_invariance():
    g = rng(8)
    x = (g.standard_normal((17, 10)) * 5).astype(np.float32)
    y = zo.softmax(x)
    np.testing.assert_allclose(y, scipy.special.softmax(x.astype(np.float64), axis=1), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(y.sum(axis=1), 1.0, rtol=1e-6)
    np.testing.assert_allclose(zo.softmax(x + np.float32(100.0)), y, rtol=1e-4, atol=1e-6)
    big = np.array([[1000.0, 1000.0, -1000.0]], np.float32)  # max-subtraction keeps it finite
    np.testing.assert_allclose(zo.softmax(big), [[0.5, 0.5, 0.0]])


def test_leaky_relu_closed_form():
    x = np.array([-3.0, -0.0, 0.0, 2.5], np.float32)
    y = zo.leakyReLU(x, 0.1)
    np.testing.assert_array_equal(y, np.where(x <= 0, np.float32(0.1) * x, x))


@pytest.mark.parametrize("sa,sb", [((1, 8, 5, 5), (8, 1, 1)), ((2, 3), (3,)), ((2, 3), (2, 1)), ((4, 1, 3), (1, 5, 1)),
                                   ((2, 3, 4, 5), (1,)), ((3, 1), (1, 4))])
def test_broadcast_add_vs_numpy(sa, sb):
    g = rng(9)
    a = g.standard_normal(sa, dtype=np.float32); b = g.standard_normal(sb, dtype=np.float32)
    np.testing.assert_array_equal(zo.sum_tensors_lean(a, b), a + b)
    np.testing.assert_array_equal(zo.sum_tensors_lean(b, a), a + b)


def test_broadcast_add_incompatible():
    with pytest.raises(zo.OracleError) as e:
        zo.sum_tensors_lean(np.zeros((2, 3), np.float32), np.zeros((4,), np.float32))
    assert e.value.name == "IncompatibleBroadcastShapes"


# ---- Sigmoid / ReduceMean / Concat / Resize(nearest): pinned beyond the reference's vectors by numpy / scipy / closed forms

def test_sigmoid_matches_scipy_expit():
    from scipy.special import expit
    x = np.random.default_rng(0).standard_normal(4096).astype(np.float32) * 8
    np.testing.assert_allclose(zo.sigmoid(x), expit(x.astype(np.float64)), rtol=1e-6, atol=1e-7)
    assert zo.sigmoid(np.array([-200.0, 200.0], np.float32)).tolist() == [0.0, 1.0]  # exp overflow gives 1/inf, not NaN


@pytest.mark.parametrize("shape,axes,keep", [((3, 4, 5), [1], True), ((3, 4, 5), [0, 2], False), ((2, 3, 4, 5), [2, 3], True),
                                             ((2, 3, 4, 5), [-1, 1], False), ((6,), [0], False), ((2, 3, 4, 5), [3, 0], True)])
def test_reduce_mean_matches_numpy(shape, axes, keep):
    x = np.random.default_rng(1).standard_normal(shape).astype(np.float32)
    y = zo.reduce_mean(x, axes, keep, False)
    ref = x.astype(np.float64).mean(axis=tuple(axes), keepdims=keep)
    assert y.shape == ref.shape
    np.testing.assert_allclose(y, ref, rtol=1e-5, atol=1e-6)


def test_reduce_mean_axis_errors():
    x = np.zeros((2, 3), np.float32)
    for axes in ([2], [-3], [0, 0]):
        with pytest.raises(zo.OracleError) as e:
            zo.reduce_mean(x, axes, True, False)
        assert e.value.name == "InvalidAxes"
    assert zo.reduce_mean(x + 2, None, False, False).shape == (1,)


@pytest.mark.parametrize("shapes,axis", [([(2, 3, 4), (2, 5, 4), (2, 1, 4)], 1), ([(2, 3), (4, 3)], 0), ([(1, 2, 3, 4), (1, 2, 3, 1)], -1),
                                         ([(5,), (3,)], 0)])
def test_concatenate_matches_numpy(shapes, axis):
    g = np.random.default_rng(2)
    for dt in (np.float32, np.uint8):
        ts = [(g.standard_normal(s) * 50).astype(dt) for s in shapes]
        np.testing.assert_array_equal(zo.concatenate(ts, axis), np.concatenate(ts, axis))


def test_concatenate_pads_lower_ranks_with_leading_ones():
    a, b = np.arange(6, dtype=np.float32).reshape(1, 2, 3), np.arange(3, dtype=np.float32) + 10  # [1,2,3] and [3] -> [1,1,3]
    np.testing.assert_array_equal(zo.concatenate([a, b], 1), np.concatenate([a, b.reshape(1, 1, 3)], 1))


def test_resize_nearest_closed_forms():
    g = np.random.default_rng(3)
    x = g.integers(0, 255, (2, 3, 4, 5), dtype=np.uint8)
    # half_pixel: an integer upscale repeats every element
    y = zo.resize(x, "nearest", [1.0, 1.0, 2.0, 3.0], None, "half_pixel")
    np.testing.assert_array_equal(y, x.repeat(2, axis=2).repeat(3, axis=3))
    # asymmetric x2 takes round-half-away(o / 2), clamped: 0 1 1 2 2 3 3 3 on an axis of 4
    y = zo.resize(x, "nearest", [1.0, 1.0, 2.0, 1.0], None, "asymmetric")
    np.testing.assert_array_equal(y, x[:, :, [0, 1, 1, 2, 2, 3, 3, 3], :])
    np.testing.assert_array_equal(zo.resize(x, "nearest", None, list(x.shape), "half_pixel"), x)  # identity
    # asymmetric halving keeps round(2 i): every other element
    np.testing.assert_array_equal(zo.resize(x[..., :4], "nearest", [1, 1, 0.5, 0.5], None, "asymmetric"), x[:, :, ::2, 0:4:2])
    # align_corners maps the ends onto the ends
    xf = g.standard_normal((1, 1, 5, 7)).astype(np.float32)
    y = zo.resize(xf, "nearest", None, [1, 1, 9, 13], "align_corners")
    assert y[0, 0, 0, 0] == xf[0, 0, 0, 0] and y[0, 0, -1, -1] == xf[0, 0, -1, -1] and y[0, 0, 4, 6] == xf[0, 0, 2, 3]
    # brute force with the published formula, half_pixel, round half away from zero, clamped
    y = zo.resize(xf, "nearest", None, [1, 1, 8, 4], "half_pixel")
    for oh in range(8):
        for ow in range(4):
            ph = np.float32(np.float32(oh + 0.5) / np.float32(8 / 5)) - np.float32(0.5)
            pw = np.float32(np.float32(ow + 0.5) / np.float32(np.float32(4) / np.float32(7))) - np.float32(0.5)
            ih = int(min(max(np.floor(abs(ph) + 0.5) * np.sign(ph), 0), 4))
            iw = int(min(max(np.floor(abs(pw) + 0.5) * np.sign(pw), 0), 6))
            assert y[0, 0, oh, ow] == xf[0, 0, ih, iw]
