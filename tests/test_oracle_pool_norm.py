"""Pins the oracle's average pooling and inference batch normalisation.  The reference holds no expected values for
either (its pooling tests use PoolingType.Max only; its BatchNormLayer test checks shapes), so they are pinned by a
brute-force restatement of the formula's definition, by torch's CPU routines and by closed forms."""
import numpy as np
import pytest
import torch

from oracle import oracle as zo


def brute_avgpool(x, k, s, pads, ceil_mode, include_pad):
    N, C, H, W = x.shape
    oshape = zo.avgpool_out_shape(x.shape, k, s, pads, ceil_mode)
    y = np.zeros(oshape, np.float64)
    for oh in range(oshape[2]):
        for ow in range(oshape[3]):
            taps, padded = [], 0
            for kr in range(k[0]):
                for kc in range(k[1]):
                    ih, iw = oh * s[0] - pads[0] + kr, ow * s[1] - pads[1] + kc
                    if 0 <= ih < H and 0 <= iw < W:
                        taps.append(x[:, :, ih, iw].astype(np.float64))
                    if -pads[0] <= ih < H + pads[2] and -pads[1] <= iw < W + pads[3]:
                        padded += 1
            div = padded if include_pad else len(taps)
            y[:, :, oh, ow] = sum(taps) / div if div else 0.0
    return y


CASES = [
    ([2, 2], [2, 2], [0, 0, 0, 0], False, False),   # what pool_forward itself covers: no padding, floor
    ([3, 3], [1, 1], [0, 0, 0, 0], False, False),
    ([3, 2], [2, 3], [0, 0, 0, 0], False, False),
    ([3, 3], [2, 2], [1, 1, 1, 1], False, False),   # ONNX: pads, divisor = taps inside the input
    ([3, 3], [2, 2], [1, 1, 1, 1], False, True),    # ONNX: divisor counts the pad cells
    ([3, 3], [2, 2], [1, 1, 1, 1], True, True),     # ceil_mode: cells past the padded input never count
    ([2, 3], [2, 2], [1, 0, 0, 2], True, False),
]


@pytest.mark.parametrize("k,s,pads,ceil_mode,include_pad", CASES)
def test_avgpool_against_brute_force_and_torch(k, s, pads, ceil_mode, include_pad):
    g = np.random.default_rng(sum(k) + sum(s) + sum(pads))
    x = g.standard_normal((2, 3, 9, 11)).astype(np.float32)
    y = zo.avgpool(x, k, s, pads, ceil_mode, include_pad)
    np.testing.assert_allclose(y, brute_avgpool(x, k, s, pads, ceil_mode, include_pad), rtol=1e-6, atol=1e-6)
    if pads[0] == pads[2] and pads[1] == pads[3]:  # torch pads symmetrically
        t = torch.nn.functional.avg_pool2d(torch.from_numpy(x), k, s, (pads[0], pads[1]), ceil_mode=ceil_mode,
                                           count_include_pad=include_pad).numpy()
        assert y.shape == t.shape
        np.testing.assert_allclose(y, t, rtol=1e-6, atol=1e-6)


def test_avgpool_closed_forms_and_errors():
    # a constant image averages to the constant wherever the divisor is the in-bounds count
    x = np.full((1, 2, 7, 7), 3.25, np.float32)
    assert np.all(zo.avgpool(x, [3, 3], [2, 2], [1, 1, 1, 1], False, False) == np.float32(3.25))
    # with the pad cells counted, a corner window of a 3x3 / pad 1 pool holds 4 of 9 taps
    y = zo.avgpool(x, [3, 3], [2, 2], [1, 1, 1, 1], False, True)
    assert y[0, 0, 0, 0] == np.float32(3.25 * 4 / 9) and y[0, 0, 1, 1] == np.float32(3.25)
    # a 1x1 window is the identity; a window of the whole image is the mean
    x = np.random.default_rng(3).standard_normal((2, 2, 4, 6)).astype(np.float32)
    np.testing.assert_array_equal(zo.avgpool(x, [1, 1], [1, 1]), x)
    np.testing.assert_allclose(zo.avgpool(x, [4, 6], [1, 1])[:, :, 0, 0], x.mean(axis=(2, 3)), rtol=1e-6, atol=1e-6)
    # the reference's summation order (row, then column) and single division: 1e8 + 1 - 1e8 + 1 in f32 is 1, not 2
    probe = np.array([[[[1e8, 1.0], [-1e8, 1.0]]]], np.float32)
    assert zo.avgpool(probe, [2, 2], [2, 2])[0, 0, 0, 0] == np.float32(0.25)
    with pytest.raises(zo.OracleError):
        zo.avgpool(x, [5, 2], [1, 1])            # kernel taller than the image (op_pooling.zig:243-245)
    with pytest.raises(zo.OracleError):
        zo.avgpool(x[0], [2, 2], [1, 1])         # not rank 4 (:229-231)


def test_batchnorm_against_the_definition_and_torch():
    g = np.random.default_rng(9)
    for shape in [(3, 4), (2, 5, 7), (2, 3, 6, 5)]:
        F = shape[1]
        x = (g.standard_normal(shape) * 2 + 1).astype(np.float32)
        ga, be = g.uniform(0.5, 2, F).astype(np.float32), g.standard_normal(F).astype(np.float32)
        mu, va = g.standard_normal(F).astype(np.float32), g.uniform(0.1, 3, F).astype(np.float32)
        y = zo.batchnorm(x, ga, be, mu, va, 1e-5)
        bshape = (1, F) + (1,) * (len(shape) - 2)
        x64 = x.astype(np.float64)
        ref = (x64 - mu.reshape(bshape)) / np.sqrt(va.reshape(bshape).astype(np.float64) + 1e-5) * ga.reshape(bshape) + be.reshape(bshape)
        np.testing.assert_allclose(y, ref, rtol=2e-6, atol=2e-6)
        t = torch.nn.functional.batch_norm(torch.from_numpy(x), torch.from_numpy(mu), torch.from_numpy(va), torch.from_numpy(ga),
                                           torch.from_numpy(be), False, 0.1, 1e-5).numpy()
        np.testing.assert_allclose(y, t, rtol=1e-5, atol=1e-5)


def test_batchnorm_closed_forms():
    # the reference's own test input (test_layers.zig:574-582) with identity statistics: zero mean, unit variance,
    # gamma 1, beta 0 and epsilon 0 leave the input unchanged
    x = np.array([[1, 2, 3, 4], [2, 3, 4, 5], [3, 4, 5, 6]], np.float32)
    one, zero = np.ones(4, np.float32), np.zeros(4, np.float32)
    np.testing.assert_array_equal(zo.batchnorm(x, one, zero, zero, one, 0.0), x)
    # gamma scales and beta shifts AFTER the normalisation: (x - 1) / 2 * 3 + 0.5 with var 4, eps 0
    y = zo.batchnorm(x, 3 * one, 0.5 * one, one, 4 * one, 0.0)
    np.testing.assert_array_equal(y, (x - 1) / 2 * 3 + np.float32(0.5))
    # the feature index is axis 1, not the last axis
    x4 = np.zeros((1, 2, 1, 3), np.float32)
    y4 = zo.batchnorm(x4, [1, 1], [10, 20], [0, 0], [1, 1], 0.0)
    assert np.all(y4[0, 0] == 10) and np.all(y4[0, 1] == 20)
    with pytest.raises(zo.OracleError):
        zo.batchnorm(x, one[:3], zero, zero, one)
