"""Bit-exact parity of the HIP int8 family (through the C ABI) with the CPU oracle."""
import numpy as np
import pytest

from oracle import oracle as zo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


QCASES = [
    # N, C, H, W, K, KH, KW, stride, pads, dil, group
    (2, 8, 7, 7, 6, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], 1),
    (2, 128, 28, 28, 128, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], 1),   # config-3 shape, small batch
    (3, 3, 96, 96, 16, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], 1),      # tiny-YOLO first layer
    (2, 256, 3, 3, 27, 1, 1, [1, 1], [0, 0, 0, 0], [1, 1], 1),      # tiny-YOLO head
    (2, 3, 96, 96, 16, 3, 3, [2, 2], [1, 1, 1, 1], [1, 1], 1),      # MobileNet stem
    (2, 96, 24, 24, 96, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], 96),    # depthwise
    (2, 48, 25, 25, 48, 3, 3, [2, 2], [1, 1, 1, 1], [1, 1], 48),    # depthwise stride 2, odd size
    (3, 40, 9, 11, 40, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], 40),     # depthwise stride 1, odd output height (row pairs)
    (2, 32, 7, 5, 32, 3, 3, [1, 1], [0, 0, 0, 0], [1, 1], 32),      # depthwise, no padding, 5 x 3 outputs
    (1, 16, 3, 9, 16, 3, 3, [1, 1], [0, 1, 0, 1], [1, 1], 16),      # depthwise, a single output row
    (2, 16, 24, 24, 96, 1, 1, [1, 1], [0, 0, 0, 0], [1, 1], 1),     # pointwise expand
    (1, 8, 6, 6, 4, 3, 3, [2, 1], [0, 1, 2, 0], [1, 1], 2),         # grouped, asymmetric pads
    (1, 3, 9, 9, 5, 2, 2, [1, 1], [0, 0, 0, 0], [2, 2], 1),         # dilation
    (4, 1280, 1, 1, 1000, 1, 1, [1, 1], [0, 0, 0, 0], [1, 1], 1),   # final Gemm as a 1x1 conv
    # the same on the matrix cores (64 images and up), where 16-channel blocks are regrouped 8, 4 or 2 at a time:
    (96, 1280, 1, 1, 1000, 1, 1, [1, 1], [0, 0, 0, 0], [1, 1], 1),  # 80 blocks: groups of 8
    (64, 192, 1, 1, 33, 1, 1, [1, 1], [0, 0, 0, 0], [1, 1], 1),     # 12 blocks: groups of 4
    (65, 90, 1, 1, 70, 1, 1, [1, 1], [0, 0, 0, 0], [1, 1], 1),      # 6 blocks, the last one partly filled: groups of 2
    (128, 64, 1, 1, 64, 1, 1, [2, 2], [0, 0, 0, 0], [1, 1], 1),     # 4 blocks: groups of 2 (a stride changes nothing)
    (70, 200, 1, 1, 40, 1, 1, [1, 1], [0, 0, 0, 0], [1, 1], 1),     # 13 blocks: not regrouped
    # 3x3 stride-1 layers of 32 channels and up whose NCHW output leaves in dwords of four positions (rows of whole
    # quads), with a channel count that ends inside a group of four and inside a block of 32:
    (3, 32, 10, 12, 42, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], 1),     # 12-wide rows, 42 channels
    (2, 48, 14, 18, 75, 3, 3, [1, 1], [0, 0, 0, 0], [1, 1], 1),     # no padding, 16-wide rows, 75 channels
    (5, 64, 37, 8, 66, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], 1),      # 37 rows of 8: a last tile of fewer rows
    (2, 40, 9, 9, 50, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], 1),       # rows that are not whole quads: byte stores
    # NCHW input of whole-dword planes on its way to the 16-channel blocked layout, the last block holding 2 and 13 channels
    (2, 50, 8, 12, 40, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], 1),
    (3, 45, 6, 6, 35, 3, 3, [1, 1], [0, 0, 0, 0], [1, 1], 1),
    (70, 77, 2, 2, 40, 1, 1, [1, 1], [0, 0, 0, 0], [1, 1], 1),      # pointwise layer on 2 x 2 planes: one quad per plane
    # two outputs per image and a last position tile that is mostly past the end of the batch (the lanes there would be
    # images 37 .. 47): first-layer kernel, depthwise kernel
    (37, 3, 3, 4, 16, 3, 3, [1, 1], [0, 0, 0, 0], [1, 1], 1),
    (37, 16, 3, 4, 16, 3, 3, [1, 1], [0, 0, 0, 0], [1, 1], 16),
]


@pytest.mark.parametrize("case", QCASES, ids=[str(i) for i in range(len(QCASES))])
@pytest.mark.parametrize("act", [None, "leaky", "relu6"])
def test_qlinearconv_bit_exact(G, case, act):
    N, C, H, W, K, KH, KW, s, p, d, grp = case
    g = np.random.default_rng(7 * N + C + K)
    x = g.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = g.integers(-127, 128, (K, C // grp, KH, KW), dtype=np.int8)
    fan = (C // grp) * KH * KW
    ws = (g.uniform(0.5, 1.5, K) * 0.08 / np.sqrt(fan)).astype(np.float32)   # spreads outputs over the u8 range
    b = g.integers(-1000, 1001, K, dtype=np.int32)
    kw = dict(act=act, act_alpha=0.1, act_scale=0.04, act_zp=30) if act else {}
    ref = zo.qlinearconv(x, 0.02, 128, w, ws, None, 0.05, 128, b, s, p, d, grp, **kw)
    y = G.tm.qlinearconv(G.dev(x), 0.02, 128, G.dev(w), G.dev(ws), None, 0.05, 128, G.dev(b), s, p, d, grp, **kw)
    np.testing.assert_array_equal(G.host(y), ref)
    assert len(np.unique(ref)) > 8  # the case really exercises requantisation


@pytest.mark.parametrize("shift", [1, 2, 4])
def test_qlinearconv_output_at_an_odd_address(G, shift):
    """An NCHW output that does not start on a 4-byte boundary takes the byte-store epilogue; nothing around it is written."""
    import torch
    N, C, H, W, K = 2, 32, 6, 8, 36
    g = np.random.default_rng(40 + shift)
    x = g.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = g.integers(-127, 128, (K, C, 3, 3), dtype=np.int8)
    ws = (g.uniform(0.5, 1.5, K) * 0.08 / np.sqrt(C * 9)).astype(np.float32)
    b = g.integers(-1000, 1001, K, dtype=np.int32)
    ref = zo.qlinearconv(x, 0.02, 128, w, ws, None, 0.05, 128, b, [1, 1], [1, 1, 1, 1], [1, 1], 1)
    buf = torch.full((ref.size + 64,), 7, dtype=torch.uint8, device="cuda:0")
    y = buf[shift:shift + ref.size].view(N, K, H, W)
    G.tm.qlinearconv_lean(G.dev(x), 0.02, 128, G.dev(w), G.dev(ws), None, 0.05, 128, G.dev(b), y, [1, 1], [1, 1, 1, 1], [1, 1])
    out = buf.cpu().numpy()
    np.testing.assert_array_equal(out[shift:shift + ref.size].reshape(ref.shape), ref)
    assert (out[:shift] == 7).all() and (out[shift + ref.size:] == 7).all()


def test_qlinearconv_per_tensor_scale_weight_zero_point_no_bias(G):
    g = np.random.default_rng(1)
    x = g.integers(0, 256, (2, 8, 9, 9), dtype=np.uint8)
    w = g.integers(-127, 128, (12, 8, 3, 3), dtype=np.int8)
    wz = g.integers(-5, 6, 12, dtype=np.int8)
    ws = np.array([0.004], np.float32)
    ref = zo.qlinearconv(x, 0.03, 7, w, ws, wz, 0.06, 100, None, [1, 1], [1, 1, 1, 1], [1, 1])
    y = G.tm.qlinearconv(G.dev(x), 0.03, 7, G.dev(w), G.dev(ws), G.dev(wz), 0.06, 100, None, [1, 1], [1, 1, 1, 1], [1, 1])
    np.testing.assert_array_equal(G.host(y), ref)


def test_qlinearconv_errors(G):
    import torch
    x = torch.zeros((1, 4, 5, 5), dtype=torch.uint8, device="cuda:0")
    w = torch.zeros((4, 2, 3, 3), dtype=torch.int8, device="cuda:0")
    ws = torch.ones(4, device="cuda:0")
    with pytest.raises(G.ZantError) as e:  # group does not match the weight's channels per group
        G.tm.qlinearconv(x, 1.0, 0, w, ws, None, 1.0, 0, None, [1, 1], [1, 1, 1, 1], [1, 1], 1)
    assert e.value.name == "InvalidDimensions"
    with pytest.raises(G.ZantError) as e:  # wrong number of weight scales
        G.tm.qlinearconv(x, 1.0, 0, w, ws[:3].contiguous(), None, 1.0, 0, None, [1, 1], [1, 1, 1, 1], [1, 1], 2)
    assert e.value.name == "InputTensorDimensionMismatch"


def test_quantize_dequantize_bit_exact(G):
    g = np.random.default_rng(2)
    x = (g.standard_normal((3, 5, 17, 9)) * 3).astype(np.float32)
    x.ravel()[:8] = [0.5, 1.5, 2.5, -0.5, -1.5, 1e9, -1e9, 0.49999997]
    for s, zp, axis in [(np.float32(0.05), 128, 1), (np.array([0.01, 0.02, 0.05, 0.1, 1.0], np.float32), np.array([128, 100, 0, 255, 3], np.uint8), 1),
                        (np.array([0.5, 0.25, 1.0], np.float32), None, 0)]:
        ref = zo.quantize_linear(x, s, zp, axis)
        q = G.tm.quantize_linear(G.dev(x), s, zp, axis)
        np.testing.assert_array_equal(G.host(q), ref)
        np.testing.assert_array_equal(G.host(G.tm.dequantize_linear(q, s, zp, axis)), zo.dequantize_linear(ref, s, zp, axis))
    t = np.array([0.5, 1.5, 2.5, -0.5, 3.5, 254.5, 255.5], np.float32)  # ties and saturation
    np.testing.assert_array_equal(G.host(G.tm.quantize_linear(G.dev(t), 1.0, 0)), [0, 2, 2, 0, 4, 254, 255])


def test_signed_and_int32_codes_bit_exact(G):
    import torch
    g = np.random.default_rng(12)
    x = (g.standard_normal((3, 4, 9, 7)) * 40).astype(np.float32)
    x.ravel()[:8] = [0.5, 1.5, -0.5, -2.5, 127.5, -128.5, 1e9, -1e9]
    for s, zp, axis in [(np.float32(0.7), None, 1), (np.array([0.3, 0.5, 1.0, 2.0], np.float32), np.array([-128, -7, 0, 127], np.int8), 1)]:
        ref = zo.quantize_linear(x, s, zp, axis, signed=True)
        zt = None if zp is None else torch.from_numpy(zp)
        q = G.tm.quantize_linear(G.dev(x), s, zt, axis, signed=True)
        assert q.dtype == torch.int8
        np.testing.assert_array_equal(G.host(q), ref)
        np.testing.assert_array_equal(G.host(G.tm.dequantize_linear(q, s, zt, axis)), zo.dequantize_linear(ref, s, zp, axis))
    acc = g.integers(-2**31, 2**31, (2, 5, 3), dtype=np.int64).astype(np.int32)
    acc.ravel()[:2] = [2**31 - 1, -2**31]
    sc = np.array([1e-3, 0.5, 2.0, 7.0, 1.0], np.float32)
    np.testing.assert_array_equal(G.host(G.tm.dequantize_linear(G.dev(acc), sc, None, 1)), zo.dequantize_linear(acc, sc, None, 1))
    zp32 = np.array([-2**31, 5, 0, -9, 2**31 - 1], np.int32)
    np.testing.assert_array_equal(G.host(G.tm.dequantize_linear(G.dev(acc), sc, torch.from_numpy(zp32), 1)),
                                  zo.dequantize_linear(acc, sc, zp32, 1))


@pytest.mark.parametrize("act,alpha", [("relu", 0.0), ("leaky", 0.1), ("relu6", 0.0), (None, 0.0)])
@pytest.mark.parametrize("n", [256, 100003])
def test_qlinear_act_bit_exact(G, act, alpha, n):
    g = np.random.default_rng(n)
    q = g.integers(0, 256, n, dtype=np.uint8)
    q[:256] = np.arange(256)
    y = G.tm.qlinear_act(G.dev(q), 0.05, 128, act, alpha, 0.03, 20)
    np.testing.assert_array_equal(G.host(y), zo.qlinear_act(q, 0.05, 128, act, alpha, 0.03, 20))


@pytest.mark.parametrize("n", [7, 4096, 1000003])
def test_qlinear_add_bit_exact(G, n):
    g = np.random.default_rng(n)
    a = g.integers(0, 256, n, dtype=np.uint8); b = g.integers(0, 256, n, dtype=np.uint8)
    y = G.tm.qlinear_add(G.dev(a), 0.02, 128, G.dev(b), 0.03, 120, 0.04, 125)
    np.testing.assert_array_equal(G.host(y), zo.qlinear_add(a, 0.02, 128, b, 0.03, 120, 0.04, 125))


def test_qlinear_global_avgpool_bit_exact(G):
    g = np.random.default_rng(4)
    for shape in [(3, 5, 3, 3), (8, 1280, 3, 3), (2, 7, 13, 11)]:
        x = g.integers(0, 256, shape, dtype=np.uint8)
        y = G.tm.qlinear_global_avgpool(G.dev(x), 0.05, 128, 0.02, 110)
        np.testing.assert_array_equal(G.host(y), zo.qlinear_global_avgpool(x, 0.05, 128, 0.02, 110))


def test_full_size_qlinearconv_properties(G):
    """Config 3 at its real shape: a slice against the oracle plus batch-permutation equivariance."""
    import torch
    g = np.random.default_rng(3)
    N, C, H, K = 128, 128, 28, 128
    x = g.integers(0, 256, (N, C, H, H), dtype=np.uint8)
    w = g.integers(-127, 128, (K, C, 3, 3), dtype=np.int8)
    ws = g.uniform(0.001, 0.01, K).astype(np.float32)
    b = g.integers(-1000, 1001, K, dtype=np.int32)
    args = ([1, 1], [1, 1, 1, 1], [1, 1])
    X, Wt, WS, Bt = G.dev(x), G.dev(w), G.dev(ws), G.dev(b)
    y = G.tm.qlinearconv(X, 0.02, 128, Wt, WS, None, 0.05, 128, Bt, *args)
    perm = torch.randperm(N, device="cuda:0")
    yp = G.tm.qlinearconv(X[perm].contiguous(), 0.02, 128, Wt, WS, None, 0.05, 128, Bt, *args)
    torch.cuda.synchronize()
    assert torch.equal(yp, y[perm])
    ref = zo.qlinearconv(x[60:62], 0.02, 128, w, ws, None, 0.05, 128, b, *args)
    np.testing.assert_array_equal(G.host(y[60:62]), ref)
