"""The generated-library level (zant_model): whole networks in one arena, against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as zo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def readme_cnn(G, batch, params):
    from zant_amd.model import Model
    m = Model(G.tm.context())
    x = m.input((batch, 1, 28, 28))
    t = m.conv(x, params["w1"], params["b1"], [1, 1], None, None, 1, None)
    t = m.relu(t)
    t = m.maxpool(t, [2, 2], [2, 2])
    t = m.conv(t, params["w2"], params["b2"], [1, 1], None, None, 1, None)
    t = m.relu(t)
    t = m.maxpool(t, [2, 2], [2, 2])
    t = m.reshape(t, [1, 1, batch, 1600])
    t = m.gemm(t, params["g1"], params["c1"])
    t = m.relu(t)
    t = m.gemm(t, params["g2"], params["c2"])
    t = m.reshape(t, [batch, 10])
    t = m.softmax(t)
    return m.finalize()


def oracle_readme_cnn(img, p):
    y = zo.ReLU(zo.Conv(img, p["w1"], p["b1"], [1, 1], None, None, 1, None))
    y = zo.onnx_maxpool(y, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    y = zo.ReLU(zo.Conv(y, p["w2"], p["b2"], [1, 1], None, None, 1, None))
    y = zo.onnx_maxpool(y, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    y = zo.ReLU(zo.gemm(y.reshape(1, 1, 1, 1600), p["g1"], p["c1"], 1.0, 1.0, False, False))
    y = zo.gemm(y, p["g2"], p["c2"], 1.0, 1.0, False, False)
    return zo.softmax(y.reshape(1, 10))


def test_readme_cnn_matches_oracle_and_plans_one_arena(G):
    from zant_amd import networks
    params = networks.readme_cnn_params(seed=3)
    params["b1"] = (np.random.default_rng(0).standard_normal(32) * 0.1).astype(np.float32)  # exercise the bias path
    batch = 37
    m = readme_cnn(G, batch, params)
    x = np.random.default_rng(1).random((batch, 1, 28, 28), dtype=np.float32)
    y = m.predict_host(x)
    ref = np.concatenate([oracle_readme_cnn(x[i:i + 1], params) for i in range(batch)])
    np.testing.assert_allclose(y, ref, rtol=G.RTOL, atol=G.ATOL)
    # 12 nodes: 3 ReLUs ride in their producers, 2 Reshapes are views, both MaxPools are computed inside their
    # convolutions, the Softmax inside the last Gemm -> 4 kernel-launching nodes
    assert m.num_launches == 4  # conv+relu+pool, conv+relu+pool, gemm+relu, gemm+softmax
    # liveness planning: the arena is much smaller than one static array per node output
    assert m.arena_bytes < 0.6 * m.unfused_bytes


def test_run_on_device_pointers_allocates_nothing(G):
    import torch
    from zant_amd import networks
    params = networks.readme_cnn_params(seed=0)
    batch = 64
    m = readme_cnn(G, batch, params)
    x = torch.rand((batch, 1, 28, 28), device="cuda:0")
    out = torch.zeros((batch, 10), device="cuda:0")
    m.run(x.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    first = out.clone()
    free0, _ = torch.cuda.mem_get_info()
    arena0 = G.za.lib.zant_hip_arena_size(G.tm.context().handle)
    for _ in range(5):
        m.run(x.data_ptr(), out.data_ptr())
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0 and G.za.lib.zant_hip_arena_size(G.tm.context().handle) == arena0
    assert torch.equal(out, first)  # same input, same arena: bit-identical reruns
    ref = np.concatenate([oracle_readme_cnn(G.host(x)[i:i + 1], params) for i in (0, batch - 1)])
    np.testing.assert_allclose(G.host(out)[[0, batch - 1]], ref, rtol=G.RTOL, atol=G.ATOL)


def test_mnist8_style_graph_folds_add_into_conv_bias(G):
    """Conv(SAME_UPPER, no bias) -> Add({M,1,1}) -> Relu -> MaxPool -> Reshape -> MatMul -> Add, as the reference's
    hardcoded_mnist8.zig:186-283 emits it."""
    from zant_amd.model import Model
    g = np.random.default_rng(5)
    w1 = (g.standard_normal((8, 1, 5, 5)) * 0.2).astype(np.float32); b1 = g.standard_normal((8, 1, 1)).astype(np.float32)
    w2 = (g.standard_normal((16, 8, 5, 5)) * 0.07).astype(np.float32); b2 = g.standard_normal((16, 1, 1)).astype(np.float32)
    fc = (g.standard_normal((256, 10)) * 0.06).astype(np.float32); fb = g.standard_normal((1, 10)).astype(np.float32)
    m = Model(G.tm.context())
    x = m.input((1, 1, 28, 28))
    t = m.conv(x, w1, None, [1, 1], None, [1, 1], 1, "SAME_UPPER")
    t = m.add_const(t, b1)
    t = m.relu(t)
    t = m.maxpool(t, [2, 2], [2, 2])
    t = m.conv(t, w2, None, [1, 1], None, [1, 1], 1, "SAME_UPPER")
    t = m.add_const(t, b2)
    t = m.relu(t)
    t = m.maxpool(t, [3, 3], [3, 3])
    t = m.reshape(t, [1, 256])
    t = m.matmul(t, fc)
    t = m.add_const(t, fb)
    m.finalize()
    assert m.num_launches == 5  # conv(+add+relu+pool), conv(+add+relu), pool, matmul, add
    img = g.random((1, 1, 28, 28), dtype=np.float32)
    y = m.predict_host(img)
    r = zo.Conv(img, w1, None, [1, 1], None, [1, 1], 1, "SAME_UPPER")
    r = zo.ReLU(zo.sum_tensors_lean(r, b1))
    r = zo.onnx_maxpool(r, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    r = zo.Conv(r, w2, None, [1, 1], None, [1, 1], 1, "SAME_UPPER")
    r = zo.ReLU(zo.sum_tensors_lean(r, b2))
    r = zo.onnx_maxpool(r, [3, 3], [3, 3], [1, 1], [0, 0, 0, 0])
    r = zo.sum_tensors_lean(zo.mat_mul(r.reshape(1, 256), fc), fb)
    np.testing.assert_allclose(y, r, rtol=G.RTOL, atol=1e-4)


def test_real_mnist8_onnx_weights_against_the_oracle(G):
    """The bundled mnist-8.onnx (the reference's datasets/models/mnist-8, kept as a data fixture) read by the package's
    ONNX reader and run by the executor, against the oracle executing the same graph node by node.  Covers SAME_UPPER
    5x5 convolutions, broadcast-Add biases {C,1,1}, a 3x3/3 MaxPool, a folded constant Reshape and MatMul + Add."""
    import os
    from zant_amd import onnx_front
    graph = onnx_front.read_graph(os.path.join(os.path.dirname(__file__), "golden", "mnist-8.onnx"))
    assert [n["op"] for n in graph["nodes"]].count("Conv") == 2 and graph["inputs"][0][1] == [1, 1, 28, 28]
    m = onnx_front.build_model(G.tm.context(), graph)
    assert m.num_launches == 5  # conv(+add+relu+pool), conv(+add+relu), pool 3x3, matmul, add
    g = np.random.default_rng(8)
    for k in range(4):
        img = g.random((1, 1, 28, 28), dtype=np.float32) * (255.0 if k % 2 else 1.0)  # raw 0..255 pixels and 0..1
        ref = onnx_front.run_graph(graph, zo, img)
        y = m.predict_host(img)
        np.testing.assert_allclose(y, ref, rtol=G.RTOL, atol=1e-4 * max(1.0, float(np.abs(ref).max())))
    m.close()


def test_predict_entry_point_follows_the_reference_abi(G):
    from zant_amd import networks
    params = networks.readme_cnn_params(seed=0)
    m = readme_cnn(G, 1, params)
    m.bind_predict()
    lib = G.za.lib
    img = np.random.default_rng(2).random((1, 1, 28, 28), dtype=np.float32)
    result = C.c_void_p(0)

    def call(shape):
        arr = (C.c_uint32 * max(len(shape), 1))(*shape)
        lib.predict(img.ctypes.data_as(C.c_void_p), arr, len(shape), C.byref(result))

    # wrong rank, empty shape, wrong dimension: silent return, result untouched (predict.zig:317-335)
    for bad in ([1, 28, 28], [], [1, 1, 28, 27], [2, 1, 28, 28]):
        call(bad)
        assert result.value is None
    call([1, 1, 28, 28])
    assert result.value is not None
    out = np.ctypeslib.as_array(C.cast(result, C.POINTER(C.c_float)), shape=(10,)).copy()
    np.testing.assert_allclose(out, oracle_readme_cnn(img, params).ravel(), rtol=G.RTOL, atol=G.ATOL)
    first_ptr = result.value
    call([1, 1, 28, 28])
    assert result.value == first_ptr  # library-owned storage, reused by the next call
    # the batched form: only the batch is passed and must be the compiled-in one
    rb = C.c_void_p(0)
    lib.predict_batched(img.ctypes.data_as(C.c_void_p), 2, C.byref(rb))
    assert rb.value is None
    lib.predict_batched(img.ctypes.data_as(C.c_void_p), 1, C.byref(rb))
    assert rb.value == first_ptr
    lib.zant_model_bind_predict(None)
    result2 = C.c_void_p(0)
    arr = (C.c_uint32 * 4)(1, 1, 28, 28)
    lib.predict(img.ctypes.data_as(C.c_void_p), arr, 4, C.byref(result2))
    assert result2.value is None  # no model bound: nothing happens


@pytest.mark.parametrize("N,C,H,W,K,k,pad,relu", [
    (9, 32, 12, 12, 64, 3, 0, True),     # the README CNN's second layer: several images per tile
    (3, 16, 41, 37, 40, 3, 1, True),     # odd conv rows and columns (the pool drops the last), K not a multiple of 32
    (2, 8, 70, 66, 96, 3, 1, False),     # several row tiles per image, three output-channel blocks, no ReLU
    (5, 12, 20, 20, 32, (2, 3), 1, True),  # 2x3 filter (generic tap loop), 32-channel workgroups
])
def test_conv_with_fused_pool_on_the_matrix_cores(G, N, C, H, W, K, k, pad, relu):
    _fused_pool_case(G, N, C, H, W, K, k, pad, relu, None)


@pytest.mark.parametrize("N,C,H,W,K,k,pad,relu", [
    (9, 32, 12, 12, 64, 3, 0, True),      # 25 windows per image: tiles start anywhere inside an image; the last is part empty
    (7, 16, 12, 12, 64, 3, 0, True),      # the last tile touches fewer images than its patch holds
    (23, 16, 12, 12, 64, 3, 0, False),
    (11, 8, 12, 12, 96, 3, 0, True),      # a single channel chunk, two blocks of output channels (the second half empty)
    (7, 24, 13, 9, 72, 3, 1, True),       # odd conv rows (the pool drops the last), padding, K not a multiple of 32
    (13, 12, 11, 12, 64, (2, 3), 1, True),  # generic tap loop
    (700, 8, 12, 12, 256, 3, 0, True),    # 1096 tiles on 512 workgroups: the last, partial round is dealt out by number
])
def test_conv_with_fused_pool_on_window_packed_tiles(G, N, C, H, W, K, k, pad, relu):
    _fused_pool_case(G, N, C, H, W, K, k, pad, relu, ",true,true>")


def _fused_pool_case(G, N, C, H, W, K, k, pad, relu, kernel_suffix):
    from zant_amd.model import Model
    g = np.random.default_rng(N * 1000 + C)
    x = g.standard_normal((N, C, H, W), dtype=np.float32)
    kh, kw = k if isinstance(k, tuple) else (k, k)
    w = (g.standard_normal((K, C, kh, kw)) * np.sqrt(2.0 / (C * kh * kw))).astype(np.float32)
    b = (g.standard_normal(K) * 0.1).astype(np.float32)
    m = Model(G.tm.context())
    t = m.conv(m.input((N, C, H, W)), w, b, [1, 1], [pad] * 4, [1, 1], 1, "NOTSET")
    if relu:
        t = m.relu(t)
    t = m.maxpool(t, [2, 2], [2, 2])
    m.finalize()
    assert m.num_launches == 1
    ref = zo.Conv(x, w, b, [1, 1], [pad] * 4, [1, 1], 1, "NOTSET")
    if relu:
        ref = zo.ReLU(ref)
    ref = zo.onnx_maxpool(ref, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    for _ in range(2):  # (the second pass draws its tiles from the counter the first one re-armed)
        np.testing.assert_allclose(m.predict_host(x), ref, rtol=G.RTOL, atol=G.ATOL)
    if kernel_suffix is not None:
        m.profile()
        assert m.launch_kernels()[0].endswith(kernel_suffix), m.launch_kernels()
    m.close()


@pytest.mark.parametrize("N,C,H,W,K,k,pad,relu", [
    (19, 1, 28, 28, 32, 3, 0, True),    # single-channel 3x3 on the matrix cores; the last workgroup holds 3 of 8 images
    (5, 1, 31, 27, 40, 3, 0, False),    # odd sizes (scalar image copy, dropped last row / column), two channel blocks, no ReLU
    (4, 1, 64, 64, 8, 3, 0, True),      # two images per workgroup, fewer channels than a block
    (9, 1, 12, 14, 32, 3, 0, True),     # 30 pooled positions per image: several image wraps per 128-position step
    (6, 1, 20, 34, 32, 3, 0, True),     # 16 pooled columns: a step of 128 positions is a whole number of rows
    (3, 1, 120, 90, 16, 3, 0, True),    # an image too large for the LDS copy: the direct kernel
    (6, 1, 28, 28, 32, 3, 1, True),     # padded: the direct kernel
    (7, 1, 28, 28, 20, 5, 0, True),     # 5x5
    (4, 3, 30, 30, 24, 3, 0, True),     # three channels
])
def test_first_layer_conv_with_fused_pool(G, N, C, H, W, K, k, pad, relu):
    from zant_amd.model import Model
    g = np.random.default_rng(N * 100 + K)
    x = g.standard_normal((N, C, H, W), dtype=np.float32)
    w = (g.standard_normal((K, C, k, k)) * np.sqrt(2.0 / (C * k * k))).astype(np.float32)
    b = (g.standard_normal(K) * 0.1).astype(np.float32)
    m = Model(G.tm.context())
    t = m.conv(m.input((N, C, H, W)), w, b, [1, 1], [pad] * 4, [1, 1], 1, "NOTSET")
    if relu:
        t = m.relu(t)
    t = m.maxpool(t, [2, 2], [2, 2])
    m.finalize()
    assert m.num_launches == 1
    ref = zo.Conv(x, w, b, [1, 1], [pad] * 4, [1, 1], 1, "NOTSET")
    if relu:
        ref = zo.ReLU(ref)
    ref = zo.onnx_maxpool(ref, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    np.testing.assert_allclose(m.predict_host(x), ref, rtol=G.RTOL, atol=G.ATOL)
    m.close()


def test_int8_network_fuses_activation_and_is_bit_exact(G):
    """QLinearConv -> Dequant/LeakyReLU/Quant -> MaxPool -> QLinearConv -> ReLU6 -> residual add -> global average pool."""
    from zant_amd.model import Model, U8
    g = np.random.default_rng(7)
    N = 5
    x = g.integers(0, 256, (N, 3, 24, 24), dtype=np.uint8)
    w1 = g.integers(-127, 128, (16, 3, 3, 3), dtype=np.int8); s1 = g.uniform(0.002, 0.004, 16).astype(np.float32)
    b1 = g.integers(-500, 500, 16, dtype=np.int32)
    w2 = g.integers(-127, 128, (16, 16, 3, 3), dtype=np.int8); s2 = g.uniform(0.0005, 0.001, 16).astype(np.float32)
    wd = g.integers(-127, 128, (16, 1, 3, 3), dtype=np.int8); sd = g.uniform(0.002, 0.004, 16).astype(np.float32)
    m = Model(G.tm.context())
    t0 = m.input((N, 3, 24, 24), U8, 0.02, 128)
    t1 = m.qlinearconv(t0, w1, s1, b1, 0.05, 128, [1, 1], [1, 1, 1, 1])
    t2 = m.qlinear_act(t1, "leaky", 0.1, 0.04, 30)
    t3 = m.maxpool(t2, [2, 2], [2, 2])
    t4 = m.qlinearconv(t3, w2, s2, None, 0.05, 120, [1, 1], [1, 1, 1, 1])
    t5 = m.qlinear_act(t4, "relu6", 0.0, 0.03, 0)
    t6 = m.qlinearconv(t5, wd, sd, None, 0.06, 110, [1, 1], [1, 1, 1, 1], group=16)   # depthwise
    t7 = m.qlinear_add(t6, t3, 0.07, 100)                                             # residual
    t8 = m.qlinear_global_avgpool(t7, 0.05, 90)
    m.finalize()
    assert m.num_launches == 5  # both activations ride in their convolutions, the MaxPool in the first one
    y = m.predict_host(x)
    r1 = zo.qlinearconv(x, 0.02, 128, w1, s1, None, 0.05, 128, b1, [1, 1], [1, 1, 1, 1], [1, 1])
    r2 = zo.qlinear_act(r1, 0.05, 128, "leaky", 0.1, 0.04, 30)
    r3 = zo.onnx_maxpool(r2, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    r4 = zo.qlinearconv(r3, 0.04, 30, w2, s2, None, 0.05, 120, None, [1, 1], [1, 1, 1, 1], [1, 1])
    r5 = zo.qlinear_act(r4, 0.05, 120, "relu6", 0.0, 0.03, 0)
    r6 = zo.qlinearconv(r5, 0.03, 0, wd, sd, None, 0.06, 110, None, [1, 1], [1, 1, 1, 1], [1, 1], 16)
    r7 = zo.qlinear_add(r6, 0.06, 110, r3, 0.04, 30, 0.07, 100)
    r8 = zo.qlinear_global_avgpool(r7, 0.07, 100, 0.05, 90)
    np.testing.assert_array_equal(y, r8)
    np.testing.assert_array_equal(m.read_tensor(t3, r3.shape, np.uint8), r3)
    assert len(np.unique(r8)) > 4


@pytest.mark.parametrize("H,W", [(5, 5), (7, 3), (1, 1), (6, 11)])
def test_global_average_pool_of_a_blocked_tensor_whose_plane_is_not_a_multiple_of_eight_positions(G, H, W):
    from zant_amd.model import Model, U8
    g = np.random.default_rng(H * 16 + W)
    N, C, K = 3, 16, 20
    x = g.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = g.integers(-127, 128, (K, C, 3, 3), dtype=np.int8); ws = g.uniform(0.0005, 0.001, K).astype(np.float32)
    m = Model(G.tm.context())
    t0 = m.input((N, C, H, W), U8, 0.02, 128)
    t1 = m.qlinearconv(t0, w, ws, None, 0.05, 120, [1, 1], [1, 1, 1, 1])
    t2 = m.qlinear_global_avgpool(t1, 0.04, 100)
    m.finalize()
    y = m.predict_host(x)
    r1 = zo.qlinearconv(x, 0.02, 128, w, ws, None, 0.05, 120, None, [1, 1], [1, 1, 1, 1], [1, 1])
    np.testing.assert_array_equal(y, zo.qlinear_global_avgpool(r1, 0.05, 120, 0.04, 100))


def test_cpp_host_mirror_runs_the_reference_tests():
    """z-ant_amd/host/test_host_mirror.cpp restates the reference's operator tests against the C++ mirror of its
    interface; the binary is built by z-ant_amd/build.py (g++ over the C ABI)."""
    import os
    import subprocess
    from conftest import ROOT
    exe = os.path.join(ROOT, "z-ant_amd", "host", "test_host_mirror")
    assert os.path.exists(exe), "run `python z-ant_amd/build.py` first"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all passed" in r.stdout


def _neck_graph(tmp_path, N, coord, sizes=False):
    """A detector-neck shaped f32 graph: two convolutions, Sigmoid, a x2 nearest Resize of the coarse map, Concat with the
    fine map along the channels, ReduceMean / GlobalAveragePool heads."""
    import onnx_writer as ow
    g = np.random.default_rng(4)
    w1 = (g.standard_normal((8, 3, 3, 3)) * 0.3).astype(np.float32)
    b1 = g.standard_normal(8).astype(np.float32)
    w2 = (g.standard_normal((16, 8, 3, 3)) * 0.2).astype(np.float32)
    b2 = g.standard_normal(16).astype(np.float32)
    inits = [ow.tensor("w1", w1), ow.tensor("b1", b1), ow.tensor("w2", w2), ow.tensor("b2", b2),
             ow.tensor("scales", np.array([] if sizes else [1, 1, 2, 2], np.float32)),
             ow.tensor("sizes", np.array([N, 16, 12, 12] if sizes else [], np.int64)), ow.tensor("axes", np.array([2, 3], np.int64))]
    nodes = [ow.node("Conv", ["x", "w1", "b1"], ["c1"], pads=[1, 1, 1, 1], kernel_shape=[3, 3]),
             ow.node("MaxPool", ["c1"], ["p1"], kernel_shape=[2, 2], strides=[2, 2]),
             ow.node("Conv", ["p1", "w2", "b2"], ["c2"], pads=[1, 1, 1, 1], kernel_shape=[3, 3]),
             ow.node("Sigmoid", ["c2"], ["s2"]),
             ow.node("Resize", ["s2", "", "scales", "sizes"], ["r2"], mode="nearest", coordinate_transformation_mode=coord,
                     nearest_mode="round_prefer_ceil"),
             ow.node("Concat", ["c1", "r2"], ["cat"], axis=1),
             ow.node("LeakyRelu", ["cat"], ["act"], alpha=0.1),
             ow.node("ReduceMean", ["act", "axes"], ["gm"], keepdims=1),
             ow.node("GlobalAveragePool", ["cat"], ["ga"]),
             ow.node("Add", ["gm", "ga"], ["y"])]
    path = tmp_path / "neck.onnx"
    path.write_bytes(ow.model(nodes, inits, [ow.value_info("x", (N, 3, 12, 12), np.float32)], [ow.value_info("y", (N, 24, 1, 1), np.float32)]))
    return str(path)


@pytest.mark.parametrize("coord,sizes", [("half_pixel", False), ("asymmetric", False), ("align_corners", True)])
def test_neck_graph_with_sigmoid_resize_concat_reduce_mean_through_the_onnx_front_end(G, tmp_path, coord, sizes):
    from zant_amd import onnx_front
    N = 5
    graph = onnx_front.read_graph(_neck_graph(tmp_path, N, coord, sizes))
    m = onnx_front.build_model(G.tm.context(), graph)
    x = np.random.default_rng(8).standard_normal((N, 3, 12, 12)).astype(np.float32)
    ref = onnx_front.run_graph(graph, zo, x)
    y = m.predict_host(x)
    assert y.shape == ref.shape == (N, 24, 1, 1)
    np.testing.assert_allclose(y, ref, rtol=G.RTOL, atol=G.ATOL)
    m.close()


def test_resize_rounding_convention_is_checked_by_the_front_end(G, tmp_path):
    """ONNX's default nearest_mode (round_prefer_floor) and the reference's round-half-away differ only on exact ties:
    half_pixel x2 has none and is accepted, asymmetric x2 has them and is refused rather than silently changed."""
    import onnx_writer as ow
    from zant_amd import onnx_front

    def graph(coord):
        nodes = [ow.node("Resize", ["x", "", "scales"], ["y"], mode="nearest", coordinate_transformation_mode=coord)]
        p = tmp_path / "r.onnx"
        p.write_bytes(ow.model(nodes, [ow.tensor("scales", np.array([1, 1, 2, 2], np.float32))], [ow.value_info("x", (1, 2, 4, 4), np.float32)],
                               [ow.value_info("y", (1, 2, 8, 8), np.float32)]))
        return onnx_front.read_graph(str(p))

    m = onnx_front.build_model(G.tm.context(), graph("half_pixel"))
    x = np.arange(32, dtype=np.float32).reshape(1, 2, 4, 4)
    np.testing.assert_array_equal(m.predict_host(x), x.repeat(2, axis=2).repeat(2, axis=3))
    m.close()
    with pytest.raises(NotImplementedError):
        onnx_front.build_model(G.tm.context(), graph("asymmetric"))


def test_quantised_concat_and_resize_nodes_keep_codes_and_parameters(G):
    """u8 tensors through MaxPool, Resize and Concat: codes move unchanged, scale / zero point ride along; inputs with
    different parameters are refused."""
    from zant_amd.model import Model, U8
    g = np.random.default_rng(6)
    N = 3
    x = g.integers(0, 256, (N, 16, 8, 8), dtype=np.uint8)
    m = Model(G.tm.context())
    t = m.input(x.shape, U8, 0.05, 120)
    p = m.maxpool(t, [2, 2], [2, 2])
    r = m.resize_nearest(p, [1.0, 1.0, 2.0, 2.0], None, "half_pixel")
    c = m.concat([t, r, t], 1)
    o = m.qlinear_act(c, "relu", 0.0, 0.04, 3)  # a reader that needs the propagated parameters
    other = m.qlinear_act(t, "relu", 0.0, 0.07, 0)
    with pytest.raises(G.ZantError) as e:
        m.concat([t, other], 1)
    assert e.value.name == "InvalidInput"
    m2 = Model(G.tm.context())  # the rejected call must not have left a node behind: build the graph again without it
    t = m2.input(x.shape, U8, 0.05, 120)
    c = m2.concat([t, m2.resize_nearest(m2.maxpool(t, [2, 2], [2, 2]), [1.0, 1.0, 2.0, 2.0], None, "half_pixel"), t], 1)
    m2.qlinear_act(c, "relu", 0.0, 0.04, 3)
    m2.finalize()
    pooled = zo.onnx_maxpool(x, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    cat = np.concatenate([x, pooled.repeat(2, axis=2).repeat(2, axis=3), x], axis=1)
    ref = zo.qlinear_act(cat, 0.05, 120, "relu", 0.0, 0.04, 3)
    np.testing.assert_array_equal(m2.predict_host(x), ref)
    m2.close(); m.close()


@pytest.mark.parametrize("N,H,W,K1,K2,pool2,relu", [
    (6, 28, 28, 32, 64, True, True),    # the README CNN's head: first-layer kernel -> pooled matrix-core convolution
    (5, 30, 26, 20, 40, True, False),   # 20 channels: five quads, channel blocks and chunk halves partly filled; no ReLU
    (4, 28, 28, 32, 48, False, True),   # the second convolution without a pool
    (3, 28, 28, 30, 32, True, True),    # 30 channels are not whole quads: the tensor stays NCHW
])
def test_f32_activation_between_two_convolutions(G, N, H, W, K1, K2, pool2, relu):
    """Conv(1 -> K1, 3x3)+[ReLU]+MaxPool -> Conv(K1 -> K2, 3x3)+[ReLU][+MaxPool]: the tensor between the two nodes is kept
    in the 16-byte channel-quad layout when K1 is a multiple of 4; results and the read-back of that tensor (handed out
    as NCHW) must not depend on it."""
    from zant_amd.model import Model
    g = np.random.default_rng(N * 1000 + K1)
    x = g.standard_normal((N, 1, H, W), dtype=np.float32)
    w1 = (g.standard_normal((K1, 1, 3, 3)) * np.sqrt(2.0 / 9)).astype(np.float32)
    b1 = (g.standard_normal(K1) * 0.1).astype(np.float32)
    w2 = (g.standard_normal((K2, K1, 3, 3)) * np.sqrt(2.0 / (K1 * 9))).astype(np.float32)
    b2 = (g.standard_normal(K2) * 0.1).astype(np.float32)
    m = Model(G.tm.context())
    t = m.conv(m.input((N, 1, H, W)), w1, b1, [1, 1], [0, 0, 0, 0], [1, 1], 1, "NOTSET")
    if relu:
        t = m.relu(t)
    mid = m.maxpool(t, [2, 2], [2, 2])
    t = m.conv(mid, w2, b2, [1, 1], [0, 0, 0, 0], [1, 1], 1, "NOTSET")
    if relu:
        t = m.relu(t)
    if pool2:
        t = m.maxpool(t, [2, 2], [2, 2])
    m.finalize()
    assert m.num_launches == 2
    r1 = zo.Conv(x, w1, b1, [1, 1], [0, 0, 0, 0], [1, 1], 1, "NOTSET")
    if relu:
        r1 = zo.ReLU(r1)
    r1 = zo.onnx_maxpool(r1, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    r2 = zo.Conv(r1, w2, b2, [1, 1], [0, 0, 0, 0], [1, 1], 1, "NOTSET")
    if relu:
        r2 = zo.ReLU(r2)
    if pool2:
        r2 = zo.onnx_maxpool(r2, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    y = m.predict_host(x)
    np.testing.assert_allclose(y, r2, rtol=G.RTOL, atol=G.ATOL)
    np.testing.assert_allclose(m.read_tensor(mid, r1.shape, np.float32), r1, rtol=G.RTOL, atol=G.ATOL)
    # reading an intermediate tensor replays the pass around the copy: the output in the arena is the pass's result again
    host_out = np.zeros_like(y)
    G.tm.context().check(G.za.lib.zant_hip_download(G.tm.context().handle, host_out.ctypes.data, m.output_ptr, host_out.nbytes))
    np.testing.assert_array_equal(host_out, y)
    m.close()
