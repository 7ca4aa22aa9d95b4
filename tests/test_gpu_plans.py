"""Prepared-weights handles (zant_hip_qlinearconv_prepack / zant_hip_conv2d_f32_prepack) through the C ABI: the same
results as the plain lean entry points and the oracle on every call, with NCHW and with channel-blocked activations."""
import numpy as np
import pytest

from oracle import oracle as zo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def _q_operands(seed, N, C, H, W, K, cg=None, k=3):
    g = np.random.default_rng(seed)
    cg = C if cg is None else cg
    x = g.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = g.integers(-127, 128, (K, cg, k, k), dtype=np.int8)
    ws = (g.uniform(0.5, 1.5, K) * 0.08 / np.sqrt(k * k * cg)).astype(np.float32)
    b = g.integers(-1000, 1001, K, dtype=np.int32)
    return x, w, ws, b


Q_CASES = [
    # N, C, H, W, K, group, kernel, stride, pads        which kernel serves it
    (3, 64, 12, 12, 96, 1, 3, 1, [1, 1, 1, 1]),          # patch-stationary matrix-core kernel
    (2, 3, 20, 20, 16, 1, 3, 2, [1, 1, 1, 1]),           # first-layer kernel
    (2, 48, 14, 14, 48, 48, 3, 1, [1, 1, 1, 1]),         # depthwise
    (4, 24, 10, 10, 40, 1, 1, 1, [0, 0, 0, 0]),          # pointwise through the tiled matrix-core kernel
    (2, 8, 9, 9, 12, 2, 3, 1, [1, 1, 1, 1]),             # grouped: direct kernel (nothing to pack)
]


@pytest.mark.parametrize("case", Q_CASES, ids=[str(i) for i in range(len(Q_CASES))])
@pytest.mark.parametrize("act", [None, "leaky"])
def test_qlinearconv_plan_matches_oracle_on_every_call(G, case, act):
    N, C, H, W, K, group, k, st, pads = case
    x, w, ws, b = _q_operands(5 * N + C + K, N, C, H, W, K, C // group, k)
    x2 = np.random.default_rng(1).integers(0, 256, x.shape, dtype=np.uint8)
    kw = dict(act=act, act_alpha=0.1, act_scale=0.04, act_zp=30) if act else {}
    W_, S_, B_ = G.dev(w), G.dev(ws), G.dev(b)
    plan = G.tm.QConvPlan(x.shape, 0.02, 128, W_, S_, None, 0.05, 128, B_, [st, st], pads, [1, 1], group, **kw)
    for xi in (x, x2, x):  # the first call packs, the later ones reuse what it packed
        ref = zo.qlinearconv(xi, 0.02, 128, w, ws, None, 0.05, 128, b, [st, st], pads, [1, 1], group, **kw)
        np.testing.assert_array_equal(G.host(plan(G.dev(xi))), ref)
    plan.close()


def test_blocked_activations_between_prepared_convolutions(G):
    """NCHW -> blocked once, two prepared convolutions on blocked tensors, blocked -> NCHW once."""
    N, C, H, K1, K2 = 6, 64, 14, 128, 64
    x, w1, s1, b1 = _q_operands(3, N, C, H, H, K1)
    _, w2, s2, b2 = _q_operands(4, N, K1, H, H, K2)
    tm = G.tm
    keep = [G.dev(a) for a in (w1, s1, b1, w2, s2, b2)]
    p1 = tm.QConvPlan(x.shape, 0.02, 128, keep[0], keep[1], None, 0.05, 120, keep[2], [1, 1], [1, 1, 1, 1], [1, 1], 1,
                      act="relu6", act_alpha=0.0, act_scale=0.03, act_zp=0, x_layout=tm.BLOCKED16, y_layout=tm.BLOCKED16)
    p2 = tm.QConvPlan((N, K1, H, H), 0.03, 0, keep[3], keep[4], None, 0.06, 110, keep[5], [1, 1], [1, 1, 1, 1], [1, 1], 1,
                      x_layout=tm.BLOCKED16, y_layout=tm.BLOCKED16)
    r1 = zo.qlinearconv(x, 0.02, 128, w1, s1, None, 0.05, 120, b1, [1, 1], [1, 1, 1, 1], [1, 1], 1, act="relu6",
                        act_alpha=0.0, act_scale=0.03, act_zp=0)
    r2 = zo.qlinearconv(r1, 0.03, 0, w2, s2, None, 0.06, 110, b2, [1, 1], [1, 1, 1, 1], [1, 1], 1)
    xb = tm.to_blocked16(G.dev(x))
    assert xb.numel() == tm.blocked16_bytes(x.shape) == N * 4 * H * H * 16
    np.testing.assert_array_equal(G.host(tm.from_blocked16(xb, x.shape)), x)  # the conversions are inverses
    for _ in range(2):
        y2 = tm.from_blocked16(p2(p1(xb)), (N, K2, H, H))
        np.testing.assert_array_equal(G.host(y2), r2)
    p1.close(); p2.close()


def test_prepack_makes_the_checks_of_the_plain_entry_point(G):
    x, w, ws, b = _q_operands(9, 2, 32, 8, 8, 48)
    tm = G.tm
    W_, S_, B_ = G.dev(w), G.dev(ws), G.dev(b)
    with pytest.raises(G.ZantError) as e:  # group does not divide the channels
        tm.QConvPlan(x.shape, 0.02, 128, W_, S_, None, 0.05, 128, B_, [1, 1], [1, 1, 1, 1], [1, 1], 5)
    assert e.value.name == "InvalidDimensions"
    with pytest.raises(G.ZantError) as e:  # negative padding
        tm.QConvPlan(x.shape, 0.02, 128, W_, S_, None, 0.05, 128, B_, [1, 1], [-1, 1, 1, 1], [1, 1], 1)
    assert e.value.name == "InvalidPadding"
    with pytest.raises(G.ZantError) as e:  # a layout that does not exist
        tm.QConvPlan(x.shape, 0.02, 128, W_, S_, None, 0.05, 128, B_, [1, 1], [1, 1, 1, 1], [1, 1], 1, x_layout=7)
    assert e.value.name == "InvalidInput"


F_CASES = [
    # N, C, H, W, K, k, stride, pads, auto_pad
    (5, 32, 13, 13, 64, 3, [1, 1], None, None),            # the README CNN's second convolution: matrix-core kernel
    (3, 1, 28, 28, 32, 3, [1, 1], None, None),             # its first: few-channel kernel
    (2, 8, 12, 12, 16, 5, [1, 1], None, "SAME_UPPER"),     # mnist-8 style
    (2, 6, 9, 11, 10, 3, [2, 2], [1, 1, 1, 1], "NOTSET"),  # strided
]


@pytest.mark.parametrize("case", F_CASES, ids=[str(i) for i in range(len(F_CASES))])
@pytest.mark.parametrize("relu", [False, True])
def test_conv_plan_matches_oracle_on_every_call(G, case, relu):
    N, C, H, W, K, k, stride, pads, auto_pad = case
    g = np.random.default_rng(N + C + K)
    w = (g.standard_normal((K, C, k, k)) * np.sqrt(2 / (C * k * k))).astype(np.float32)
    b = (g.standard_normal(K) * 0.1).astype(np.float32)
    xs = [g.standard_normal((N, C, H, W)).astype(np.float32) for _ in range(2)]
    tm = G.tm
    W_, B_ = G.dev(w), G.dev(b)
    yshape = tm.get_convolution_output_shape((N, C, H, W), w.shape, stride, pads, None, auto_pad, 1)
    plan = tm.ConvPlan((N, C, H, W), W_, B_, yshape, stride, pads, None, 1, auto_pad, "relu" if relu else None)
    for xi in (xs[0], xs[1], xs[0]):
        ref = zo.Conv(xi, w, b, stride, pads, None, 1, auto_pad)
        ref = zo.ReLU(ref) if relu else ref
        y = G.dev(np.zeros(yshape, np.float32))
        np.testing.assert_allclose(G.host(plan(G.dev(xi), y)), ref, rtol=G.RTOL, atol=G.ATOL)
    plan.close()
    with pytest.raises(G.ZantError) as e:  # the output shape is checked when the plan is made
        tm.ConvPlan((N, C, H, W), W_, B_, (N, K, 1, 1), stride, pads, None, 1, auto_pad)
    assert e.value.name == "InvalidDimensions"


@pytest.mark.parametrize("N,C,H,K,k", [(6, 1, 28, 32, 3), (5, 32, 13, 64, 3), (3, 3, 20, 16, 3), (4, 16, 12, 24, 3)])
def test_conv_plan_with_the_pool_fused_matches_conv_relu_maxpool(G, N, C, H, K, k):
    """Conv -> ReLU -> MaxPool 2x2/2 as ONE prepared call against the three oracle operators."""
    g = np.random.default_rng(N + C + K)
    w = (g.standard_normal((K, C, k, k)) * np.sqrt(2 / (C * k * k))).astype(np.float32)
    b = (g.standard_normal(K) * 0.1).astype(np.float32)
    x = g.standard_normal((N, C, H, H)).astype(np.float32)
    tm = G.tm
    W_, B_ = G.dev(w), G.dev(b)
    ref = zo.onnx_maxpool(zo.ReLU(zo.Conv(x, w, b, [1, 1], None, None, 1, None)), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    plan = tm.ConvPlan(x.shape, W_, B_, ref.shape, [1, 1], None, None, 1, None, "relu", True)
    for _ in range(2):
        y = G.dev(np.full(ref.shape, np.nan, np.float32))
        np.testing.assert_allclose(G.host(plan(G.dev(x), y)), ref, rtol=G.RTOL, atol=G.ATOL)
    plan.close()


def test_conv_plan_refuses_a_fused_pool_its_kernels_do_not_have(G):
    tm = G.tm
    w = G.dev(np.zeros((8, 16, 3, 3), np.float32))
    with pytest.raises(G.ZantError) as e:  # a strided convolution has no pooled epilogue
        tm.ConvPlan((2, 16, 20, 20), w, None, (2, 8, 4, 4), [2, 2], None, None, 1, None, "relu", True)
    assert e.value.name == "InvalidInput"
    with pytest.raises(G.ZantError) as e:  # the pooled shape is checked
        tm.ConvPlan((2, 16, 20, 20), w, None, (2, 8, 18, 18), [1, 1], None, None, 1, None, "relu", True)
    assert e.value.name == "InvalidDimensions"
