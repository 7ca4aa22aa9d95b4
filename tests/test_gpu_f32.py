"""Parity of the HIP f32 operators (through the C ABI) with the CPU oracle and the reference's own vectors."""
import numpy as np
import pytest

from conftest import cases_for
from oracle import oracle as zo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


# ---------------------------------------------------------------- the reference's known answers, on the GPU

@pytest.mark.parametrize("c", cases_for("conv_lean", "Conv"))
def test_conv_known_answers(G, c):
    x, w, b = G.dev(G.T(c["x"])), G.dev(G.T(c["w"])), G.dev(G.T(c["bias"]))
    if c["op"] == "conv_lean":
        import torch
        y = torch.zeros(c["expect"]["shape"], device="cuda:0")
        G.tm.conv_lean(x, w, y, b, c["stride"], c["pads"], c["dilations"], c["group"], c["auto_pad"])
    else:
        y = G.tm.Conv(x, w, b, c["stride"], c["pads"], c["dilations"], c["group"], c["auto_pad"])
    assert list(y.shape) == c["expect"]["shape"]
    np.testing.assert_array_equal(G.host(y), G.T(c["expect"]))  # small integers: exact in any order


@pytest.mark.parametrize("c", cases_for("convolve_tensor_with_bias"))
def test_convolve_with_bias_known_answer(G, c):
    y = G.tm.Conv(G.dev(G.T(c["x"])), G.dev(G.T(c["w"])), G.dev(G.T(c["bias"])), c["stride"], None, None, None, None)
    np.testing.assert_array_equal(G.host(y), G.T(c["expect"]))


@pytest.mark.parametrize("c", cases_for("gemm"))
def test_gemm_known_answers(G, c):
    y = G.tm.gemm(G.dev(G.T(c["a"])), G.dev(G.T(c["b"])), G.dev(G.T(c["c"])), c["alpha"], c["beta"], c["transA"], c["transB"])
    assert list(y.shape) == c["expect_shape"]
    yh = G.host(y).ravel()
    for i, v in c["expect_at"].items():
        assert yh[int(i)] == v


@pytest.mark.parametrize("c", cases_for("gemm_error"))
def test_gemm_errors(G, c):
    import torch
    a = torch.zeros(c["a_shape"], device="cuda:0"); b = torch.zeros(c["b_shape"], device="cuda:0")
    with pytest.raises(G.ZantError) as e:
        G.tm.gemm(a, b, None, 1, 1, c["transA"], c["transB"])
    assert e.value.name == c["error"]


@pytest.mark.parametrize("c", cases_for("mat_mul"))
def test_matmul_known_answers(G, c):
    y = G.tm.mat_mul(G.dev(G.T(c["a"])), G.dev(G.T(c["b"])))
    yh = G.host(y).ravel()
    for i, v in c["expect_at"].items():
        assert yh[int(i)] == v


@pytest.mark.parametrize("c", cases_for("mat_mul_error"))
def test_matmul_errors(G, c):
    import torch
    with pytest.raises(G.ZantError) as e:
        G.tm.mat_mul(torch.zeros(c["a_shape"], device="cuda:0"), torch.zeros(c["b_shape"], device="cuda:0"))
    assert e.value.name == c["error"]


@pytest.mark.parametrize("c", cases_for("onnx_maxpool"))
def test_maxpool_known_answers(G, c):
    y = G.tm.onnx_maxpool(G.dev(G.T(c["x"])), c["kernel"], c["strides"], c["dilations"], c["pads"], c["auto_pad"], c["ceil_mode"])
    assert list(y.shape) == c["expect"]["shape"]
    np.testing.assert_array_equal(G.host(y), G.T(c["expect"]))
    yq = G.tm.onnx_maxpool(G.dev(G.T(c["x"], np.uint8)), c["kernel"], c["strides"], c["dilations"], c["pads"], c["auto_pad"], c["ceil_mode"])
    np.testing.assert_array_equal(G.host(yq), G.T(c["expect"], np.uint8))


@pytest.mark.parametrize("c", cases_for("ReLU"))
def test_relu_known_answers(G, c):
    np.testing.assert_array_equal(G.host(G.tm.ReLU(G.dev(G.T(c["x"])))), G.T(c["expect"]))


@pytest.mark.parametrize("c", cases_for("leakyReLU"))
def test_leaky_known_answers(G, c):
    y = G.host(G.tm.leakyReLU(G.dev(G.T(c["x"])), c["slope"]))
    assert np.all(np.abs(y - G.T(c["expect"])) <= c["atol"])
    np.testing.assert_array_equal(y, zo.leakyReLU(G.T(c["x"]), c["slope"]))


@pytest.mark.parametrize("c", cases_for("softmax"))
def test_softmax_known_answers(G, c):
    y = G.host(G.tm.softmax(G.dev(G.T(c["x"]))))
    if c["property"] == "rows_sum_to_1_within_0.1":
        assert np.all(np.abs(y.sum(axis=1) - 1) < 0.1)
    else:
        assert y[0, 0] == y[0, 1] and y[1, 0] == y[1, 1]


@pytest.mark.parametrize("c", cases_for("sum_tensors"))
def test_sum_tensors_known_answers(G, c):
    np.testing.assert_array_equal(G.host(G.tm.sum_tensors(G.dev(G.T(c["a"])), G.dev(G.T(c["b"])))), G.T(c["expect"]))


@pytest.mark.parametrize("c", cases_for("add_bias"))
def test_add_bias_known_answers(G, c):
    np.testing.assert_array_equal(G.host(G.tm.add_bias(G.dev(G.T(c["t"])), G.dev(G.T(c["bias"])))), G.T(c["expect"]))


@pytest.mark.parametrize("c", cases_for("reshape"))
def test_reshape_known_answers(G, c):
    import torch
    x = G.dev(G.T(c["x"], np.uint8))
    if "error" in c:
        with pytest.raises(G.ZantError) as e:
            G.tm.reshape_lean(x, c["new_shape"])
        assert e.value.name == c["error"]
    else:
        y = G.tm.reshape_lean(x, c["new_shape"], torch.zeros_like(x).view(-1))
        assert list(y.shape) == c["expect_shape"]
        np.testing.assert_array_equal(G.host(y).ravel(), G.T(c["x"], np.uint8).ravel())


def test_conv_error_paths(G):
    import torch
    x = torch.zeros((1, 2, 4, 4), device="cuda:0"); w = torch.zeros((2, 2, 3, 3), device="cuda:0")
    y = torch.zeros((1, 2, 2, 2), device="cuda:0")
    for args, name in [((x, torch.zeros((2, 1, 3, 3), device="cuda:0"), y, None, [1, 1], None, None, 2, None), "InvalidDimensions"),
                       ((x, w, y, None, [1, 1], None, None, 1, "NOTSET"), "InvalidPadding"),
                       ((x, w, torch.zeros((1, 2, 3, 3), device="cuda:0"), None, [1, 1], None, None, 1, None), "InvalidDimensions"),
                       ((x[0], w, y, None, [1, 1]), "InvalidDimensions")]:
        with pytest.raises(G.ZantError) as e:
            G.tm.conv_lean(*args)
        assert e.value.name == name
    with pytest.raises(G.ZantError) as e:  # pads ignored without "NOTSET" -> wrapper/lean shape mismatch
        G.tm.Conv(x, w, None, [1, 1], [1, 1, 1, 1], None, 1, None)
    assert e.value.name == "InvalidDimensions"


# ---------------------------------------------------------------- seeded parity with the oracle

CONV_CASES = [
    # N, C, H, W, K, KH, KW, stride, pads, dil, auto_pad        (direct kernel and MFMA kernel shapes)
    (2, 3, 7, 9, 4, 3, 3, [1, 1], [0, 0, 0, 0], [1, 1], "NOTSET"),
    (1, 1, 28, 28, 32, 3, 3, [1, 1], None, None, None),               # config-1 conv1 (C=1: direct kernel)
    (3, 32, 13, 13, 64, 3, 3, [1, 1], None, None, None),              # config-1 conv2 (several images per tile)
    (70, 32, 13, 13, 64, 3, 3, [1, 1], None, None, None),             # ... with a ragged last image group
    (2, 64, 56, 56, 64, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], "NOTSET"),  # config-2a shape, small batch
    (2, 16, 20, 20, 48, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], "NOTSET"),  # K not a multiple of 32
    (1, 12, 17, 19, 40, 3, 3, [1, 1], None, None, "SAME_UPPER"),      # C not a multiple of 8, odd sizes
    (2, 8, 15, 15, 16, 3, 3, [2, 2], [1, 1, 1, 1], [1, 1], "NOTSET"),   # stride 2
    (1, 8, 16, 16, 24, 3, 3, [1, 1], [2, 2, 2, 2], [2, 2], "NOTSET"),   # dilation 2
    (2, 16, 9, 11, 32, 1, 1, [1, 1], None, None, None),               # 1x1
    (1, 8, 12, 12, 8, 5, 5, [1, 1], None, None, "SAME_LOWER"),        # 5x5 (mnist-8 style)
    (1, 8, 10, 14, 20, 3, 2, [2, 1], [1, 0, 2, 1], [1, 1], "NOTSET"),   # rectangular everything
    (2, 3, 20, 20, 16, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], "NOTSET"),   # 3 input channels (few-channel kernel)
    (2, 3, 17, 17, 16, 3, 3, [2, 2], [1, 1, 1, 1], [1, 1], "NOTSET"),   # ... stride 2 stem
    (2, 1, 12, 12, 8, 5, 5, [1, 1], None, None, "SAME_UPPER"),        # 1 channel, 5x5 (mnist-8 first layer)
    (600, 16, 3, 3, 32, 3, 3, [1, 1], None, None, None),              # one output per image: hundreds of images per tile
    (300, 8, 4, 4, 64, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], "NOTSET"),   # ... padded, ragged last group, a single chunk per tile
    (5, 8, 6, 300, 32, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], "NOTSET"),   # wide rows
    (20000, 8, 4, 4, 32, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], "NOTSET"),  # single-chunk tiles, more tiles than workgroup slots
    (1, 8, 3, 4200, 32, 3, 3, [1, 1], [1, 1, 1, 1], [1, 1], "NOTSET"),   # rows wider than the tiled kernel's patch table takes
]


@pytest.mark.parametrize("case", CONV_CASES, ids=[str(i) for i in range(len(CONV_CASES))])
@pytest.mark.parametrize("relu", [False, True])
def test_conv_vs_oracle(G, case, relu):
    N, C, H, W, K, KH, KW, s, p, d, ap = case
    g = np.random.default_rng(100 + N * 7 + C)
    x = g.standard_normal((N, C, H, W), dtype=np.float32)
    w = (g.standard_normal((K, C, KH, KW)) * np.sqrt(2.0 / (C * KH * KW))).astype(np.float32)
    b = (g.standard_normal(K) * 0.1).astype(np.float32)
    ref = zo.Conv(x, w, b, s, p, d, 1, ap)
    if relu:
        ref = zo.ReLU(ref)
    import torch
    y = torch.full(ref.shape, -7.0, device="cuda:0")  # every element must be overwritten
    G.tm.conv_lean(G.dev(x), G.dev(w), y, G.dev(b), s, p, d, 1, ap, "relu" if relu else None)
    np.testing.assert_allclose(G.host(y), ref, rtol=G.RTOL, atol=G.ATOL)


GEMM_CASES = [(64, 96, 48), (130, 70, 33), (1, 256, 10), (257, 1600, 512), (33, 5, 7), (128, 512, 10), (67, 1100, 16),
              (19, 513, 1), (200, 64, 17),
              # B stored [K][N] with N a multiple of 4 above 32 (copied in 16-byte pieces of four columns): column tiles that
              # end inside the matrix, a K tail
              (130, 70, 36), (96, 45, 100), (40, 160, 68)]


@pytest.mark.parametrize("M,K,N", GEMM_CASES)
@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_gemm_vs_oracle(G, M, K, N, ta, tb):
    g = np.random.default_rng(M + K + N + 2 * ta + tb)
    a = g.standard_normal((1, 1, K, M) if ta else (1, 1, M, K), dtype=np.float32)
    b = (g.standard_normal((1, 1, N, K) if tb else (1, 1, K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
    for cshape, alpha, beta, act in [((1, 1, 1, N), 1.0, 1.0, None), ((1, 1, M, N), 0.75, -1.5, None),
                                     ((1, 1, M, 1), 2.0, 3.0, "relu"), (None, 1.0, 1.0, None)]:
        c = None if cshape is None else (g.standard_normal(cshape) * 0.1).astype(np.float32)
        ref = zo.gemm(a, b, c, alpha, beta, ta, tb)
        if act:
            ref = zo.ReLU(ref)
        import torch
        y = torch.full(ref.shape, -7.0, device="cuda:0")
        G.tm.gemm_lean(G.dev(a), G.dev(b), G.dev(c), alpha, beta, ta, tb, y, act)
        np.testing.assert_allclose(G.host(y), ref, rtol=G.RTOL, atol=G.ATOL)


@pytest.mark.parametrize("M,K,N,tb", [(4096, 512, 10, 0), (37, 700, 16, 1), (5, 3, 2, 0), (64, 1024, 7, 0)])
def test_gemm_with_fused_row_softmax(G, M, K, N, tb):
    """The classifier head in one kernel: Gemm, then lean_softmax over each row of the [M, N] result."""
    import torch
    g = np.random.default_rng(M + K + N)
    a = g.standard_normal((1, 1, M, K), dtype=np.float32)
    b = (g.standard_normal((1, 1, N, K) if tb else (1, 1, K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
    c = (g.standard_normal((1, 1, 1, N)) * 0.1).astype(np.float32)
    ref = zo.softmax(zo.gemm(a, b, c, 1.0, 1.0, False, bool(tb)).reshape(M, N))
    y = torch.full((1, 1, M, N), -7.0, device="cuda:0")
    G.tm.gemm_lean(G.dev(a), G.dev(b), G.dev(c), 1.0, 1.0, False, bool(tb), y, "softmax")
    np.testing.assert_allclose(G.host(y).reshape(M, N), ref, rtol=G.RTOL, atol=G.ATOL)
    np.testing.assert_allclose(G.host(y).reshape(M, N).sum(axis=1), 1.0, rtol=1e-5)
    # not available for wide or transposed-A products
    with pytest.raises(G.ZantError) as e:
        G.tm.gemm_lean(torch.zeros(1, 1, 8, 4, device="cuda:0"), torch.zeros(1, 1, 4, 32, device="cuda:0"), None, 1.0, 1.0,
                       False, False, torch.zeros(1, 1, 8, 32, device="cuda:0"), "softmax")
    assert e.value.name == "InvalidInput"


def test_matmul_vs_oracle_and_ignored_batch_dims(G):
    g = np.random.default_rng(5)
    a = g.standard_normal((37, 53), dtype=np.float32); b = g.standard_normal((53, 29), dtype=np.float32)
    np.testing.assert_allclose(G.host(G.tm.mat_mul(G.dev(a), G.dev(b))), zo.mat_mul(a, b), rtol=G.RTOL, atol=G.ATOL)
    import torch
    a4 = np.stack([a, 2 * a])[None]; b4 = np.stack([b, 3 * b])[None]
    y4 = torch.full((1, 2, 37, 29), -1.0, device="cuda:0")
    G.tm.mat_mul_lean(G.dev(a4), G.dev(b4), y4)  # only the first matrix is multiplied (op_mat_mul.zig:93-97)
    yh = G.host(y4)
    np.testing.assert_allclose(yh[0, 0], zo.mat_mul(a, b), rtol=G.RTOL, atol=G.ATOL)
    assert np.all(yh[0, 1] == -1.0)


POOL_CASES = [((4, 32, 26, 26), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET"),
              ((3, 64, 11, 11), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET"),
              ((2, 5, 13, 11), [3, 3], [2, 2], [1, 1], [1, 1, 1, 1], "NOTSET"),
              ((2, 5, 13, 11), [3, 2], [1, 2], [2, 1], [0, 1, 2, 0], "NOTSET"),
              ((2, 3, 9, 9), [3, 3], [3, 3], [1, 1], [0, 0, 0, 0], "NOTSET"),
              ((1, 3, 9, 10), [2, 2], [1, 1], [1, 1], [0, 0, 0, 0], "SAME_UPPER"),
              ((1, 3, 9, 10), [2, 2], [1, 1], [1, 1], [0, 0, 0, 0], "SAME_LOWER"),
              # the plane-staged 2x2/2 kernels: a partial last group of planes, planes that are not a whole number of
              # vectors (13 x 26), fewer planes than a group, result rows of 24 bytes (u8)
              ((5, 3, 26, 26), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET"),
              ((3, 7, 13, 26), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET"),
              ((3, 1, 10, 14), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET"),
              ((7, 5, 6, 6), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET"),
              ((3, 5, 48, 48), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET"),
              ((2, 3, 16, 48), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET"),
              ((9, 11, 4, 16), [2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET")]


@pytest.mark.parametrize("xs,k,s,d,p,ap", POOL_CASES)
def test_maxpool_vs_oracle(G, xs, k, s, d, p, ap):
    g = np.random.default_rng(11)
    x = g.standard_normal(xs, dtype=np.float32)
    np.testing.assert_array_equal(G.host(G.tm.onnx_maxpool(G.dev(x), k, s, d, p, ap)), zo.onnx_maxpool(x, k, s, d, p, ap))
    q = g.integers(0, 256, xs, dtype=np.uint8)
    np.testing.assert_array_equal(G.host(G.tm.onnx_maxpool(G.dev(q), k, s, d, p, ap)), zo.onnx_maxpool(q, k, s, d, p, ap))


@pytest.mark.parametrize("n", [1, 5, 1024, 4099, 1 << 20])
def test_relu_leaky_vs_oracle(G, n):
    g = np.random.default_rng(n)
    x = g.standard_normal(n, dtype=np.float32)
    x[::7] = 0.0
    np.testing.assert_array_equal(G.host(G.tm.ReLU(G.dev(x))), zo.ReLU(x))
    np.testing.assert_array_equal(G.host(G.tm.leakyReLU(G.dev(x), 0.1)), zo.leakyReLU(x, 0.1))
    if n > 8:  # an unaligned view takes the scalar path
        np.testing.assert_array_equal(G.host(G.tm.ReLU(G.dev(x)[1:].contiguous()[1:])), zo.ReLU(x[2:]))


@pytest.mark.parametrize("rows,cols", [(1, 10), (4096, 10), (33, 1000), (5, 1)])
def test_softmax_vs_oracle(G, rows, cols):
    g = np.random.default_rng(rows + cols)
    x = (g.standard_normal((rows, cols)) * 4).astype(np.float32)
    y = G.host(G.tm.softmax(G.dev(x)))
    np.testing.assert_allclose(y, zo.softmax(x), rtol=G.RTOL, atol=G.ATOL)
    np.testing.assert_allclose(y.sum(axis=1), 1.0, rtol=1e-5)


@pytest.mark.parametrize("sa,sb", [((1, 8, 28, 28), (8, 1, 1)), ((2, 3), (3,)), ((2, 3), (2, 1)), ((4, 1, 3), (1, 5, 1)),
                                   ((2, 3, 4, 5), (1,)), ((64, 512), (64, 512)), ((3, 1), (1, 4))])
def test_add_vs_oracle(G, sa, sb):
    g = np.random.default_rng(3)
    a = g.standard_normal(sa, dtype=np.float32); b = g.standard_normal(sb, dtype=np.float32)
    np.testing.assert_array_equal(G.host(G.tm.sum_tensors_lean(G.dev(a), G.dev(b))), zo.sum_tensors_lean(a, b))
    np.testing.assert_array_equal(G.host(G.tm.sum_tensors_lean(G.dev(b), G.dev(a))), zo.sum_tensors_lean(b, a))


def test_add_incompatible(G):
    import torch
    with pytest.raises(G.ZantError) as e:
        G.tm.sum_tensors_lean(torch.zeros((2, 3), device="cuda:0"), torch.zeros((4,), device="cuda:0"))
    assert e.value.name == "IncompatibleBroadcastShapes"


def test_full_size_conv_properties(G):
    """Config 2a at its real shape: linearity in the weights and a ones-kernel closed form (no CPU run needed)."""
    import torch
    torch.manual_seed(0)
    N, C, H, K = 256, 64, 56, 64
    x = torch.randn((N, C, H, H), device="cuda:0")
    w1 = torch.randn((K, C, 3, 3), device="cuda:0") * 0.05
    w2 = torch.randn((K, C, 3, 3), device="cuda:0") * 0.05
    args = ([1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
    y1 = G.tm.Conv(x, w1, None, *args); y2 = G.tm.Conv(x, w2, None, *args); y12 = G.tm.Conv(x, w1 + w2, None, *args)
    torch.cuda.synchronize()
    assert torch.allclose(y12, y1 + y2, rtol=1e-4, atol=1e-4)
    ones = torch.ones((N, C, H, H), device="cuda:0")
    wk = torch.ones((K, C, 3, 3), device="cuda:0")
    y = G.tm.Conv(ones, wk, None, *args)
    torch.cuda.synchronize()
    assert float(y[0, 0, 0, 0]) == 4 * C and float(y[3, 5, 0, 7]) == 6 * C and float(y[255, 63, 30, 30]) == 9 * C
    assert float(y[255, 63, 55, 55]) == 4 * C
    # a slice of the big run against the oracle
    xs = x[100:102].contiguous()
    ref = zo.Conv(G.host(xs), G.host(w1), None, *args)
    np.testing.assert_allclose(G.host(y1[100:102]), ref, rtol=G.RTOL, atol=G.ATOL)


# The staged Gemm kernel has one instantiation per (A copy mode, B copy mode); which one runs follows from the
# transposition flags, the row lengths and the alignment of the operands.  Modes: 0 = k-contiguous 16-byte copies,
# 1 = k-contiguous 4-byte copies, 2 = 4-byte copies of the other orientation, 3 (B only) = B stored [K][N] with N a multiple
# of 4 copied as it lies, the lane gathering its four k with two hand-issued LDS reads.  Every instantiation that takes that
# last mode is run here with K tails (K not a multiple of the 32-k chunk, K below one chunk), ragged M and N tiles, and
# the fall-back to 4-byte copies when B is not 16-byte aligned.
GEMM_MODE_CASES = [
    # M, K, N, transA, misalign A, misalign B -> expected (A mode, B mode)
    (300, 100, 64, 0, 0, 0, (0, 3)),     # aligned row-major A, K tail of 4
    (300, 37, 36, 0, 0, 0, (1, 3)),      # K = 37: A rows are not whole 16-byte units; ragged N tile
    (129, 1600, 512, 0, 0, 0, (0, 3)),   # the README CNN's first Gemm with a ragged M tile
    (64, 24, 40, 0, 0, 0, (0, 3)),       # K below one chunk
    (200, 96, 48, 1, 0, 0, (2, 3)),      # transposed A
    (70, 33, 68, 1, 0, 0, (2, 3)),       # transposed A, K tail of 1
    (300, 100, 64, 0, 0, 1, (0, 2)),     # B off the 16-byte grid: falls back to 4-byte copies
    (300, 100, 64, 0, 1, 0, (1, 3)),     # A off the grid
    (90, 64, 50, 0, 0, 0, (0, 2)),       # N not a multiple of 4
]


# ... and each of them exists for both tile shapes: 64 x 64 (four waves) while 128 x 64 tiles would leave more than half of
# the CUs without one, 128 x 64 (eight waves) from there on.  `many_rows` grows M until the second shape is taken.
@pytest.mark.parametrize("many_rows", [False, True], ids=["tile64x64", "tile128x64"])
@pytest.mark.parametrize("M,K,N,ta,mis_a,mis_b,modes", GEMM_MODE_CASES)
def test_gemm_copy_modes_vs_oracle(G, M, K, N, ta, mis_a, mis_b, modes, many_rows):
    import torch
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    n_tiles = -(-N // 64)
    if many_rows:
        M += 128 * (cus // 2 // n_tiles + 1)
    assert (2 * -(-M // 128) * n_tiles > cus) == many_rows
    g = np.random.default_rng(M + 3 * K + 5 * N + ta)
    a = g.standard_normal((1, 1, K, M) if ta else (1, 1, M, K), dtype=np.float32)
    b = (g.standard_normal((1, 1, K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
    c = (g.standard_normal((1, 1, 1, N)) * 0.1).astype(np.float32)

    def place(arr, misalign):  # a device copy that starts 4 bytes past a 16-byte boundary when asked
        flat = torch.zeros(arr.size + 4, dtype=torch.float32, device="cuda:0")
        view = flat[1:1 + arr.size] if misalign else flat[:arr.size]
        view.copy_(torch.from_numpy(arr.ravel()))
        return view.view(arr.shape)

    A, B = place(a, mis_a), place(b, mis_b)
    assert (A.data_ptr() % 16 != 0) == bool(mis_a) and (B.data_ptr() % 16 != 0) == bool(mis_b)
    y = torch.full((1, 1, M, N), -7.0, device="cuda:0")
    G.tm.gemm_lean(A, B, G.dev(c), 1.0, 1.0, bool(ta), False, y, "relu")
    assert G.tm.context().kernel_name() == "gemm_f32_dma_kernel<1,%d,2,%d,%d,5>" % ((4 if many_rows else 2,) + modes)
    ref = zo.ReLU(zo.gemm(a, b, c, 1.0, 1.0, bool(ta), False))
    np.testing.assert_allclose(G.host(y), ref, rtol=G.RTOL, atol=G.ATOL)
