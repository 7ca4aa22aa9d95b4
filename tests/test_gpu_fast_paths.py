"""Shapes chosen to hit (and to just miss) the specialised kernels behind the operator entry points: every operator keeps
one definition, so each fast path must agree with the oracle exactly like the general kernel it replaces."""
import numpy as np
import pytest

import int8_ref
from oracle import oracle as zo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


# ---- first int8 layers: 1..4 input channels, 3x3 -------------------------------------------------------------------
FIRST = [
    # N, C, H, W, K, stride, pad
    (2, 1, 28, 28, 8, 1, 1),      # one channel, half an output block
    (2, 2, 17, 19, 16, 2, 1),     # two channels, odd sizes, stride 2
    (3, 4, 12, 12, 24, 1, 0),     # four channels, no padding, more than 16 filters
    (2, 3, 11, 5, 40, 2, 0),      # narrow rows, two blocks of output channels
    (1, 3, 4, 4, 16, 1, 1),       # the narrowest row the dword loads take
    (2, 3, 9, 3, 8, 1, 1),        # narrower than that: the dot-product kernel
]


@pytest.mark.parametrize("case", FIRST, ids=[str(i) for i in range(len(FIRST))])
@pytest.mark.parametrize("act", [None, "leaky"])
def test_first_layer_kernels(G, case, act):
    N, C, H, W, K, s, p = case
    g = np.random.default_rng(100 + C * 7 + K)
    x = g.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = g.integers(-127, 128, (K, C, 3, 3), dtype=np.int8)
    ws = (g.uniform(0.5, 1.5, K) * 0.08 / np.sqrt(C * 9)).astype(np.float32)
    ws[::3] *= -1.0  # negative multipliers reverse the order the pooled maximum is taken in
    b = g.integers(-500, 501, K, dtype=np.int32)
    kw = dict(act=act, act_alpha=0.1, act_scale=0.04, act_zp=30) if act else {}
    for x_zp in (128, 3):
        ref = zo.qlinearconv(x, 0.02, x_zp, w, ws, None, 0.05, 120, b, [s, s], [p] * 4, [1, 1], 1, **kw)
        y = G.tm.qlinearconv(G.dev(x), 0.02, x_zp, G.dev(w), G.dev(ws), None, 0.05, 120, G.dev(b), [s, s], [p] * 4, [1, 1], 1, **kw)
        np.testing.assert_array_equal(G.host(y), ref)


def _pool_net(cin, hw, convs, batch_c=3):
    """3x3 stem on `cin` channels followed by conv(+act)+pool stages; a 1x1 tail keeps the last pool blocked."""
    layers = [dict(op="conv", k=3, stride=1, pad=1, cin=cin, cout=convs[0][0], group=1, act="leaky", alpha=0.1),
              dict(op="pool")]
    c = convs[0][0]
    for cout, k, act in convs[1:]:
        d = dict(op="conv", k=k, stride=1, pad=k // 2, cin=c, cout=cout, group=1, act=act)
        if act == "leaky":
            d["alpha"] = 0.1
        layers += [d, dict(op="pool")]
        c = cout
    layers.append(dict(op="conv", k=1, stride=1, pad=0, cin=c, cout=5, group=1, act=None))
    return dict(name="pools", input=(cin,) + tuple(hw), layers=layers)


@pytest.mark.parametrize("cin,hw,convs,launches", [
    (3, (26, 26), [(16, 3, "leaky"), (24, 3, "leaky"), (40, 1, "relu6")], 4),   # odd pooled sizes, narrow and wide tiles
    (1, (20, 28), [(8, 3, "leaky"), (64, 3, None)], 3),                          # pool straight after the convolution
])
def test_conv_act_pool_chains_run_as_one_kernel_each(G, cin, hw, convs, launches):
    from zant_amd import networks as nets
    arch = _pool_net(cin, hw, convs)
    params = nets.int8_params(arch, seed=9)
    rng = np.random.default_rng(3)
    quant = int8_ref.calibrate(arch, params, rng.integers(0, 256, (2,) + arch["input"], dtype=np.uint8))
    x = rng.integers(0, 256, (5,) + arch["input"], dtype=np.uint8)
    m = nets.build_int8_model(G.tm.context(), arch, params, quant, 5)
    assert m.num_launches == launches
    np.testing.assert_array_equal(m.predict_host(x), int8_ref.forward(arch, params, quant, x))
    m.close()


# ---- memory-bound operators ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(2, 3, 32, 48), (3, 5, 16, 16), (2, 2, 18, 32), (1, 4, 6, 20)])
def test_maxpool_u8_row_vector_path_and_its_neighbours(G, shape):
    x = np.random.default_rng(sum(shape)).integers(0, 256, shape, dtype=np.uint8)
    ref = zo.onnx_maxpool(x, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    y = G.tm.onnx_maxpool(G.dev(x), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    np.testing.assert_array_equal(G.host(y), ref)


@pytest.mark.parametrize("shape", [(3, 4, 26, 26), (2, 3, 7, 10), (5, 1, 4, 2), (2, 2, 9, 9)])
def test_maxpool_f32_row_vector_path_and_its_neighbours(G, shape):
    x = np.random.default_rng(sum(shape)).standard_normal(shape).astype(np.float32)
    ref = zo.onnx_maxpool(x, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    y = G.tm.onnx_maxpool(G.dev(x), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    np.testing.assert_array_equal(G.host(y), ref)


@pytest.mark.parametrize("ashape,bshape", [
    ((4, 6, 10, 10), (6, 1, 1)),        # per-channel, inner a multiple of 4
    ((6, 1, 1), (4, 6, 10, 10)),        # the same with the operands swapped
    ((3, 5, 8, 4), (1, 5, 1, 1)),
    ((2, 7, 16), (7, 1)),
    ((4, 6, 5, 5), (6, 1, 1)),          # inner not a multiple of 4: the general kernel
    ((2, 3, 4, 8), (3, 1, 8)),          # two broadcast-free axes: the general kernel
])
def test_broadcast_add_per_channel_path_and_its_neighbours(G, ashape, bshape):
    g = np.random.default_rng(len(ashape) * 10 + len(bshape))
    a = g.standard_normal(ashape).astype(np.float32)
    b = g.standard_normal(bshape).astype(np.float32)
    y = G.tm.sum_tensors_lean(G.dev(a), G.dev(b))
    np.testing.assert_array_equal(G.host(y), a + b)  # one f32 addition per element: exact


@pytest.mark.parametrize("rows,cols", [(1, 1), (5, 10), (256, 16), (257, 7), (1000, 3), (700, 17), (3, 64)])
def test_softmax_small_row_path_and_its_neighbours(G, rows, cols):
    x = (np.random.default_rng(rows + cols).standard_normal((rows, cols)) * 4).astype(np.float32)
    y = G.host(G.tm.softmax(G.dev(x)))
    np.testing.assert_allclose(y, zo.softmax(x), rtol=G.RTOL, atol=G.ATOL)
    np.testing.assert_allclose(y.sum(axis=1), 1.0, rtol=1e-5)


@pytest.mark.parametrize("scales", [(0.02, 0.03, 0.04), (1e-12, 2e-12, 1.5e-12), (3.0e5, 1.0e4, 2.0e5)])
@pytest.mark.parametrize("n", [16, 4099])
def test_qlinear_add_division_variants(G, scales, n):
    """Ordinary scales take the short division sequence, extreme ones the general division: same bytes either way."""
    g = np.random.default_rng(n)
    a = g.integers(0, 256, n, dtype=np.uint8)
    b = g.integers(0, 256, n, dtype=np.uint8)
    sa, sb, sy = scales
    y = G.tm.qlinear_add(G.dev(a), sa, 128, G.dev(b), sb, 120, sy, 125)
    np.testing.assert_array_equal(G.host(y), zo.qlinear_add(a, sa, 128, b, sb, 120, sy, 125))


def test_qlinear_add_covers_every_byte_pair(G):
    a, b = np.meshgrid(np.arange(256, dtype=np.uint8), np.arange(256, dtype=np.uint8))
    a, b = a.ravel().copy(), b.ravel().copy()
    for sa, sb, sy, zy in ((0.0235, 0.0171, 0.0302, 128), (0.05, 0.05, 0.05, 0), (0.011, 0.093, 0.041, 255)):
        y = G.tm.qlinear_add(G.dev(a), sa, 131, G.dev(b), sb, 7, sy, zy)
        np.testing.assert_array_equal(G.host(y), zo.qlinear_add(a, sa, 131, b, sb, 7, sy, zy))


@pytest.mark.parametrize("shape", [(4, 6, 8, 8), (2, 3, 48, 48), (3, 5, 4, 4), (2, 2, 5, 16)])
def test_global_avgpool_vector_path_and_its_neighbours(G, shape):
    x = np.random.default_rng(sum(shape)).integers(0, 256, shape, dtype=np.uint8)
    y = G.tm.qlinear_global_avgpool(G.dev(x), 0.05, 117, 0.02, 110)
    np.testing.assert_array_equal(G.host(y), zo.qlinear_global_avgpool(x, 0.05, 117, 0.02, 110))
