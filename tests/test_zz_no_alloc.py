"""The convolution entry point that allocates nothing (zant_hip_conv2d_f32_static) against zant_hip_conv2d_f32.

Both run the same kernels, one with its scratch in a static device array, the other in the context workspace, so
the outputs must be equal bit for bit; the oracle bounds both within the f32 tolerance of the path."""
import ctypes as C

import numpy as np
import pytest
import torch

from gpu_util import ATOL, RTOL, ZantError, dev, host, tm, za
from oracle import oracle as zo

pytestmark = pytest.mark.gpu


def _case(seed, n, c, h, w, k, relu):
    g = np.random.default_rng(seed)
    x = g.standard_normal((n, c, h, w)).astype(np.float32)
    wt = (g.standard_normal((k, c, 3, 3)) * np.sqrt(2.0 / (9 * c))).astype(np.float32)
    b = (g.standard_normal(k) * 0.1).astype(np.float32)
    return x, wt, b, "relu" if relu else None


def _both(x, wt, b, act):
    X, W, B = dev(x), dev(wt), dev(b)
    shape = tm.get_convolution_output_shape(x.shape, wt.shape, [1, 1], [1, 1, 1, 1], [1, 1], "NOTSET")
    # poisoned outputs: every element must be written by the call itself
    y_ws = torch.full(shape, float("nan"), dtype=torch.float32, device="cuda:0")
    y_st = torch.full(shape, float("nan"), dtype=torch.float32, device="cuda:0")
    tm.conv_lean(X, W, y_ws, B, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET", fuse_act=act)
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    tm.conv_lean_static(X, W, y_st, B, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET", fuse_act=act)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "the static entry point changed the device's free memory"
    return host(y_ws), host(y_st)


def _static_on_a_fresh_context(x, wt, b, act):
    """The static entry point as the FIRST operator call of a new context: its workspace is still empty, so a path
    that took its scratch from the workspace (or allocated anything else) would have to call hipMalloc here, and the
    device's free memory would drop."""
    from zant_amd.capi import Context, dims
    X, W, B = dev(x), dev(wt), dev(b)
    shape = tm.get_convolution_output_shape(x.shape, wt.shape, [1, 1], [1, 1, 1, 1], [1, 1], "NOTSET")
    y = torch.full(shape, float("nan"), dtype=torch.float32, device="cuda:0")
    ctx = Context()
    xd, _ = dims(x.shape); wd, _ = dims(wt.shape); yd, _ = dims(shape)
    s, ns = dims([1, 1]); p, npd = dims([1, 1, 1, 1]); d, nd = dims([1, 1])
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    ctx.check(za.lib.zant_hip_conv2d_f32_static(ctx.handle, X.data_ptr(), xd, W.data_ptr(), wd, B.data_ptr(), y.data_ptr(), yd,
                                                s, ns, p, npd, d, nd, 1, b"NOTSET", tm.ACT[act]))
    ctx.sync()
    free1 = torch.cuda.mem_get_info()[0]
    ctx.close()
    assert free1 == free0, "the static entry point allocated device memory on a context that had none"
    return host(y)


def test_static_entry_point_allocates_nothing_on_a_fresh_context():
    # the largest shape of this file first, before any allocating convolution has grown a workspace for it
    x, wt, b, act = _case(1, 16, 64, 28, 28, 64, True)
    y_fresh = _static_on_a_fresh_context(x, wt, b, act)
    y_ws, y_st = _both(x, wt, b, act)
    np.testing.assert_array_equal(y_fresh, y_ws)
    np.testing.assert_array_equal(y_st, y_ws)


def test_static_entry_point_two_calls_in_a_row_second_one_smaller():
    # first a large convolution (tiled kernel, many tiles, packed weights of 64 x 64 x 9), then a smaller one that
    # leaves most of the scratch array holding the first call's contents
    big = _case(1, 16, 64, 28, 28, 64, True)
    small = _case(2, 3, 16, 12, 12, 24, False)
    for x, wt, b, act in (big, small):
        y_ws, y_st = _both(x, wt, b, act)
        np.testing.assert_array_equal(y_st, y_ws)
        ref = zo.Conv(x, wt, b, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
        if act:
            ref = zo.ReLU(ref)
        np.testing.assert_allclose(y_st, ref, rtol=RTOL, atol=ATOL)


def test_static_entry_point_without_scratch_and_error_paths():
    # a first-layer shape goes to the few-channel kernel, which has no scratch at all
    x, wt, b, act = _case(3, 5, 1, 14, 14, 8, True)
    y_ws, y_st = _both(x, wt, b, act)
    np.testing.assert_array_equal(y_st, y_ws)
    # the checks are those of conv_lean
    X, W = dev(x), dev(wt)
    with pytest.raises(ZantError) as e:
        tm.conv_lean_static(X, W, torch.zeros((5, 8, 3, 3), device="cuda:0"), None, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
    assert e.value.name == "InvalidDimensions"
    with pytest.raises(ZantError) as e:
        tm.conv_lean_static(X, W, torch.zeros((5, 8, 14, 14), device="cuda:0"), None, [1, 1], [1, 1, 1, 1], [1, 1], 2, "NOTSET")
    assert e.value.name == "InvalidDimensions"


def test_static_entry_point_rejects_weights_beyond_the_scratch_array():
    # 512 x 512 x 3 x 3 packed weights are 9.4 MB: more than the 8 MiB array; nothing may be launched or written
    g = np.random.default_rng(4)
    x = g.standard_normal((1, 512, 10, 10)).astype(np.float32)
    wt = (g.standard_normal((512, 512, 3, 3)) * 0.02).astype(np.float32)
    X, W = dev(x), dev(wt)
    y = torch.full((1, 512, 10, 10), 7.0, dtype=torch.float32, device="cuda:0")
    with pytest.raises(ZantError) as e:
        tm.conv_lean_static(X, W, y, None, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
    assert e.value.name == "ArenaOverflow"
    ctx = tm.context()
    msg = za.lib.zant_hip_last_error(ctx.handle).decode()
    assert "static scratch too small" in msg and str(8 << 20) in msg
    assert float(host(y).min()) == 7.0 and float(host(y).max()) == 7.0
    # the allocating entry point takes the same call
    y2 = torch.zeros((1, 512, 10, 10), dtype=torch.float32, device="cuda:0")
    tm.conv_lean(X, W, y2, None, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
    ref = zo.Conv(x, wt, None, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
    np.testing.assert_allclose(host(y2), ref, rtol=RTOL, atol=ATOL)
