"""GPU parity for AveragePool, BatchNormalization, the ONNX Gemm mapping (the reference's debug_model.onnx) and the
executor's fusion corner cases, against the CPU oracle."""
import os

import numpy as np
import pytest

from oracle import oracle as zo

import onnx_writer as ow

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


AVG_CASES = [
    ((2, 3, 9, 11), [2, 2], [2, 2], None, False, False),
    ((4, 8, 26, 28), [2, 2], [2, 2], None, False, False),           # the vector kernel
    ((2, 3, 9, 11), [3, 3], [1, 1], [0, 0, 0, 0], False, False),
    ((2, 3, 9, 11), [3, 2], [2, 3], None, False, False),
    ((2, 3, 9, 11), [3, 3], [2, 2], [1, 1, 1, 1], False, False),
    ((2, 3, 9, 11), [3, 3], [2, 2], [1, 1, 1, 1], True, True),
    ((1, 5, 7, 7), [2, 3], [2, 2], [1, 0, 0, 2], True, False),
    ((3, 4, 6, 6), [6, 6], [1, 1], None, False, False),             # one window: the mean of the plane
    ((5, 3, 26, 26), [2, 2], [2, 2], None, False, False),           # the plane-staged kernel, a partial last group
    ((3, 7, 13, 26), [2, 2], [2, 2], None, False, False),           # planes that are not a whole number of vectors
    ((3, 1, 10, 14), [2, 2], [2, 2], None, False, False),
]


@pytest.mark.parametrize("shape,k,s,pads,ceil_mode,include_pad", AVG_CASES)
def test_avgpool_vs_oracle(G, shape, k, s, pads, ceil_mode, include_pad):
    x = np.random.default_rng(sum(shape)).standard_normal(shape).astype(np.float32)
    ref = zo.avgpool(x, k, s, pads or [0, 0, 0, 0], ceil_mode, include_pad)
    y = G.host(G.tm.avgpool(G.dev(x), k, s, pads, ceil_mode, include_pad))
    assert y.shape == ref.shape
    np.testing.assert_allclose(y, ref, rtol=G.RTOL, atol=G.ATOL)
    if k == [2, 2] and s == [2, 2] and pads is None:  # these kernels add the four taps in the reference's order
        np.testing.assert_array_equal(y, ref)


def test_avgpool_errors(G):
    import torch
    x = torch.zeros((1, 2, 4, 6), device="cuda:0")
    for k, s, p, name in [([5, 2], [1, 1], None, "InvalidDimensions"), ([0, 2], [1, 1], None, "InvalidDimensions"),
                          ([2, 2], [0, 1], None, "InvalidDimensions"), ([2, 2], [1, 1], [2, 0, 0, 0], "InvalidPadding")]:
        with pytest.raises(G.ZantError) as e:
            G.tm.avgpool(x, k, s, p)
        assert e.value.name == name
    with pytest.raises(G.ZantError) as e:
        G.tm.avgpool(x[0], [2, 2], [1, 1])
    assert e.value.name == "InputTensorDimensionMismatch"


@pytest.mark.parametrize("shape", [(3, 4), (2, 5, 7), (2, 3, 6, 5), (4, 16, 8, 8)])
def test_batchnorm_vs_oracle(G, shape):
    g = np.random.default_rng(len(shape) + shape[1])
    F = shape[1]
    x = (g.standard_normal(shape) * 2 + 1).astype(np.float32)
    ga, be = g.uniform(0.5, 2, F).astype(np.float32), g.standard_normal(F).astype(np.float32)
    mu, va = g.standard_normal(F).astype(np.float32), g.uniform(0.1, 3, F).astype(np.float32)
    ref = zo.batchnorm(x, ga, be, mu, va, 1e-5)
    y = G.host(G.tm.batchnorm(G.dev(x), G.dev(ga), G.dev(be), G.dev(mu), G.dev(va), 1e-5))
    np.testing.assert_allclose(y, ref, rtol=G.RTOL, atol=G.ATOL)


def _bn_params(g, F):
    return (g.uniform(0.5, 2, F).astype(np.float32), g.standard_normal(F).astype(np.float32),
            g.standard_normal(F).astype(np.float32), g.uniform(0.1, 3, F).astype(np.float32))


def test_conv_batchnorm_relu_avgpool_through_the_onnx_front_end(G, tmp_path):
    """Conv -> BatchNormalization -> Relu -> AveragePool -> BatchNormalization: the first normalisation is folded into
    the convolution (one launch for Conv+BN+Relu), the second one runs as its own kernel."""
    from zant_amd import onnx_front
    g = np.random.default_rng(21)
    N, C, H, K = 3, 8, 12, 16
    w = (g.standard_normal((K, C, 3, 3)) * 0.2).astype(np.float32)
    b = g.standard_normal(K).astype(np.float32)
    bn1, bn2 = _bn_params(g, K), _bn_params(g, K)
    inits = [ow.tensor("w", w), ow.tensor("b", b)]
    for tag, p in (("1", bn1), ("2", bn2)):
        inits += [ow.tensor(n + tag, a) for n, a in zip(("ga", "be", "mu", "va"), p)]
    nodes = [ow.node("Conv", ["x", "w", "b"], ["c"], kernel_shape=[3, 3], pads=[1, 1, 1, 1]),
             ow.node("BatchNormalization", ["c", "ga1", "be1", "mu1", "va1"], ["n1"], epsilon=1e-3),
             ow.node("Relu", ["n1"], ["r"]),
             ow.node("AveragePool", ["r"], ["p"], kernel_shape=[2, 2], strides=[2, 2]),
             ow.node("BatchNormalization", ["p", "ga2", "be2", "mu2", "va2"], ["y"])]
    path = tmp_path / "bn.onnx"
    path.write_bytes(ow.model(nodes, inits, [ow.value_info("x", (N, C, H, H), np.float32)],
                              [ow.value_info("y", (N, K, H // 2, H // 2), np.float32)]))
    graph = onnx_front.read_graph(str(path))
    m = onnx_front.build_model(G.tm.context(), graph)
    assert m.num_launches == 3
    x = g.standard_normal((N, C, H, H)).astype(np.float32)
    ref = onnx_front.run_graph(graph, zo, x)
    np.testing.assert_allclose(m.predict_host(x), ref, rtol=G.RTOL, atol=1e-4)
    m.close()


def test_debug_model_onnx_against_the_oracle(G):
    """The reference's datasets/models/debug_model/debug_model.onnx (kept as a data fixture): Gemm(transB, alpha, beta
    from the file, 2-D operands, 1-D bias) -> Relu -> Gemm -> Relu -> Softmax, node by node against the oracle."""
    from zant_amd import onnx_front
    graph = onnx_front.read_graph(os.path.join(GOLDEN, "debug_model.onnx"))
    assert [n["op"] for n in graph["nodes"]] == ["Gemm", "Relu", "Gemm", "Relu", "Softmax"]
    assert all(n["attrs"].get("transB") == 1 for n in graph["nodes"] if n["op"] == "Gemm")
    m = onnx_front.build_model(G.tm.context(), graph)
    assert m.num_launches == 3  # Gemm+Relu, Gemm+Relu, Softmax (the second ReLU sits between the Gemm and the Softmax)
    g = np.random.default_rng(4)
    for k in range(4):
        x = (g.standard_normal((1, 5)) * (3.0 if k else 1.0)).astype(np.float32)
        ref = onnx_front.run_graph(graph, zo, x)
        y = m.predict_host(x)
        assert y.shape == (1, 5)
        np.testing.assert_allclose(y, ref, rtol=G.RTOL, atol=G.ATOL)
        np.testing.assert_allclose(y.sum(), 1.0, rtol=1e-5)
    # the intermediate tensors, one by one: what each node of the file produces
    x = g.standard_normal((1, 5)).astype(np.float32)
    init = graph["initializers"]
    h1 = zo.ReLU(zo.gemm(x.reshape(1, 1, 1, 5), init["layer1.weight"].reshape(1, 1, 5, 5), init["layer1.bias"].reshape(1, 1, 1, 5),
                         1.0, 1.0, False, True))
    np.testing.assert_allclose(h1.reshape(1, 5), np.maximum(x @ init["layer1.weight"].T + init["layer1.bias"], 0), rtol=1e-5, atol=1e-6)
    m.close()


def test_gemm_rejects_batched_operands_in_a_model(G):
    from zant_amd.model import Model
    m = Model(G.tm.context())
    t = m.input((2, 1, 3, 4))
    with pytest.raises(G.ZantError) as e:
        m.gemm(t, np.zeros((2, 1, 4, 5), np.float32))
    assert e.value.name == "InvalidInput"
    m.close()


def test_plain_requantisation_node_is_not_fused_into_the_convolution(G):
    """QLinearConv -> QLinearAct('none'): the second node requantises the rounded, saturated u8 of the first; fused,
    that intermediate rounding would be skipped."""
    from zant_amd.model import Model, U8
    g = np.random.default_rng(13)
    x = g.integers(0, 256, (2, 16, 9, 9), dtype=np.uint8)
    w = g.integers(-127, 128, (24, 16, 3, 3), dtype=np.int8)
    ws = (g.uniform(0.5, 1.5, 24) * 0.02).astype(np.float32)   # wide outputs: many values saturate at the first stage
    b = g.integers(-1000, 1001, 24, dtype=np.int32)
    m = Model(G.tm.context())
    t = m.input(x.shape, U8, 0.02, 128)
    t = m.qlinearconv(t, w, ws, b, 0.05, 128, [1, 1], [1, 1, 1, 1])
    t = m.qlinear_act(t, "none", 0.0, 0.013, 7)
    m.finalize()
    assert m.num_launches == 2
    ref = zo.qlinearconv(x, 0.02, 128, w, ws, None, 0.05, 128, b, [1, 1], [1, 1, 1, 1], [1, 1], 1)
    assert (ref == 0).any() and (ref == 255).any()
    ref = zo.qlinear_act(ref, 0.05, 128, "none", 0.0, 0.013, 7)
    np.testing.assert_array_equal(m.predict_host(x), ref)
    m.close()


def test_rank1_constant_after_a_1x1_output_is_a_bias_only_for_one_image(G):
    """Conv with a [N, M, 1, 1] result followed by Add({M}): NumPy broadcasting adds along the LAST axis, so for N > 1
    the Add produces [N, M, 1, M] and must not be folded into the convolution as a per-channel bias."""
    from zant_amd.model import Model
    g = np.random.default_rng(17)
    M = 6
    w = g.standard_normal((M, 3, 4, 4)).astype(np.float32)
    c = g.standard_normal(M).astype(np.float32)
    for N, launches in ((1, 1), (3, 2)):
        x = g.standard_normal((N, 3, 4, 4)).astype(np.float32)
        m = Model(G.tm.context())
        t = m.input(x.shape)
        t = m.conv(t, w, None, [1, 1], [0, 0, 0, 0], [1, 1], 1, "NOTSET")
        t = m.add_const(t, c)
        m.finalize()
        assert m.num_launches == launches
        ref = zo.sum_tensors_lean(zo.Conv(x, w, None, [1, 1], [0, 0, 0, 0], [1, 1], 1, "NOTSET"), c)
        y = m.predict_host(x)
        assert y.shape == ref.shape
        np.testing.assert_allclose(y, ref, rtol=G.RTOL, atol=G.ATOL)
        m.close()


def test_input_survives_repeated_passes(G):
    """The input uploaded once to the model's input slot serves every later pass: no node output may be planned over it."""
    import torch
    from zant_amd import networks
    from test_gpu_model import readme_cnn, oracle_readme_cnn
    params = networks.readme_cnn_params(seed=0)
    N = 64
    m = readme_cnn(G, N, params)
    x = np.random.default_rng(23).random((N, 1, 28, 28), dtype=np.float32)
    X = G.dev(x)
    G.za.lib.zant_hip_upload(G.tm.context().handle, m.input_ptr, x.ctypes.data, x.nbytes)
    outs = []
    for _ in range(3):
        m.run()
        torch.cuda.synchronize()
        out = np.empty((N, 10), np.float32)
        G.za.lib.zant_hip_download(G.tm.context().handle, out.ctypes.data, m.output_ptr, out.nbytes)
        outs.append(out)
    np.testing.assert_array_equal(outs[0], outs[1])
    np.testing.assert_array_equal(outs[0], outs[2])
    for n in (0, 31, 63):
        np.testing.assert_allclose(outs[2][n], oracle_readme_cnn(x[n:n + 1], params).ravel(), rtol=G.RTOL, atol=G.ATOL)
    m.close()


def _conv_bn_model(G, N, C, K, H, gamma, beta, mean, var, eps, seed=0):
    from zant_amd.model import Model
    g = np.random.default_rng(seed)
    x = g.standard_normal((N, C, H, H)).astype(np.float32)
    w = (g.standard_normal((K, C, 3, 3)) * np.sqrt(2 / (9 * C))).astype(np.float32)
    b = (g.standard_normal(K) * 0.1).astype(np.float32)
    m = Model(G.tm.context())
    t = m.conv(m.input((N, C, H, H)), w, b, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
    m.batchnorm(t, gamma, beta, mean, var, eps)
    m.finalize()
    ref = zo.batchnorm(zo.Conv(x, w, b, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET"), gamma, beta, mean, var, eps)
    return m, x, ref


def test_conv_batchnorm_fold_is_bounded_against_the_oracle(G):
    """Moderate scales are folded into the convolution (one launch); the folded result stays inside the tolerance of the
    path against the oracle's order of operations, also with a small variance and a large gamma."""
    K = 16
    g = np.random.default_rng(1)
    gamma = g.uniform(0.5, 40.0, K).astype(np.float32)
    var = g.uniform(2e-3, 1.0, K).astype(np.float32)       # s up to 40 / sqrt(2e-3) ~ 900
    beta, mean = g.standard_normal(K).astype(np.float32), g.standard_normal(K).astype(np.float32)
    m, x, ref = _conv_bn_model(G, 3, 8, K, 10, gamma, beta, mean, var, 1e-5)
    assert m.num_launches == 1
    np.testing.assert_allclose(m.predict_host(x), ref, rtol=G.RTOL, atol=G.ATOL * float(np.abs(ref).max()))
    m.close()


def test_conv_batchnorm_is_not_folded_for_extreme_or_non_finite_scales(G):
    K = 8
    ones, zeros = np.ones(K, np.float32), np.zeros(K, np.float32)
    # gamma / sqrt(var + eps) = 1e6: beyond the bound, the normalisation stays its own kernel and matches the oracle
    var = np.full(K, 1e-12, np.float32)
    m, x, ref = _conv_bn_model(G, 2, 4, K, 8, ones, zeros, zeros, var, 0.0)
    assert m.num_launches == 2
    np.testing.assert_allclose(m.predict_host(x), ref, rtol=G.RTOL, atol=G.ATOL * float(np.abs(ref).max()))
    m.close()
    # var + eps < 0 in one channel: sqrt gives NaN there -- in that channel's outputs only, as the operator defines it
    var = np.ones(K, np.float32)
    var[3] = -1.0
    m, x, ref = _conv_bn_model(G, 2, 4, K, 8, ones, zeros, zeros, var, 1e-5)
    assert m.num_launches == 2
    y = m.predict_host(x)
    assert np.isnan(y[:, 3]).all() and np.isnan(ref[:, 3]).all()
    keep = [k for k in range(K) if k != 3]
    np.testing.assert_allclose(y[:, keep], ref[:, keep], rtol=G.RTOL, atol=G.ATOL)
    m.close()
