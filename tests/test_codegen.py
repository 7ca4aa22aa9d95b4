"""The code generator: ONNX graph -> C source of a stand-alone library over the C ABI (the counterpart of the reference's
lib_<model>.zig emitter).  Generation and compilation need no GPU; running the generated predict() does."""
import ctypes as C
import json
import os

import numpy as np
import pytest

import __graft_entry__ as ge
import onnx_writer

HERE = os.path.dirname(os.path.abspath(__file__))
MNIST = os.path.join(HERE, "golden", "mnist-8.onnx")
DEBUG_MODEL = os.path.join(HERE, "golden", "debug_model.onnx")


@pytest.fixture(scope="module")
def codegen():
    ge.load_package()
    from zant_amd import codegen
    return codegen


def _load(so):
    lib = C.CDLL(so)
    lib.predict.restype = None
    lib.predict.argtypes = [C.c_void_p, C.POINTER(C.c_uint32), C.c_uint32, C.POINTER(C.c_void_p)]
    return lib


def _predict(lib, x, shape=None):
    shape = x.shape if shape is None else shape
    arr = (C.c_uint32 * max(len(shape), 1))(*shape)
    res = C.c_void_p()
    lib.predict(x.ctypes.data_as(C.c_void_p), arr, len(shape), C.byref(res))
    return res.value


def test_generated_source_replays_the_graph_and_compiles_without_a_gpu(codegen, tmp_path):
    info = codegen.generate(MNIST, str(tmp_path), "mnist8")
    text = open(info["c"]).read()
    # mnist-8: 12 ONNX nodes, one of them a Reshape of an initialiser that is folded at generation time
    assert info["nodes"] == 11 and info["in_shape"] == (1, 1, 28, 28) and info["out_shape"] == (1, 10)
    for call in ("zant_model_input(m, 0,", "zant_model_conv(m, 0,", '"SAME_UPPER"', "zant_model_add_const(m, 1,", "zant_model_relu(m, 2)",
                 "zant_model_maxpool(m, 3,", "zant_model_reshape(m, 8,", "zant_model_matmul(m, 9,", "static float g_result[10];"):
        assert call in text, call
    assert os.path.getsize(info["params"]) == info["param_bytes"] >= 4 * (8 * 25 + 8 + 16 * 8 * 25 + 16 + 2560 + 10)
    so = codegen.compile_library(info)
    lib = _load(so)
    for sym in ("predict", "setLogFunction", "mnist8_init", "mnist8_model", "mnist8_shutdown"):
        assert hasattr(lib, sym)
    # the reference's predict() returns silently, result untouched, on a wrong rank / shape / empty shape
    # (tests/CodeGen/test_model.template.zig:60-160); these paths end before any GPU call
    x = np.zeros((1, 1, 28, 28), np.float32)
    assert _predict(lib, x, (1, 1, 28)) is None
    assert _predict(lib, x, (1, 1, 28, 27)) is None
    assert _predict(lib, x, ()) is None


def test_generator_rejects_a_graph_the_executor_would_reject(codegen, tmp_path):
    nodes = [onnx_writer.node("Conv", ["x", "w"], ["y"], kernel_shape=[3, 3])]
    p = tmp_path / "bad.onnx"   # 4 input channels against a filter with 3: the dry-run model refuses the node
    p.write_bytes(onnx_writer.model(nodes, [onnx_writer.tensor("w", np.zeros((2, 3, 3, 3), np.float32))],
                                    [onnx_writer.value_info("x", (1, 4, 8, 8), np.float32)], [onnx_writer.value_info("y", (1, 2, 6, 6), np.float32)]))
    from zant_amd import ZantError
    with pytest.raises(ZantError):
        codegen.generate(str(p), str(tmp_path), "bad")


@pytest.mark.gpu
def test_generated_mnist8_library_matches_the_oracle(codegen, tmp_path):
    from oracle import oracle as zo
    from zant_amd import onnx_front
    info = codegen.generate(MNIST, str(tmp_path), "mnist8")
    lib = _load(codegen.compile_library(info))
    graph = onnx_front.read_graph(MNIST)
    g = np.random.default_rng(0)
    logged = []
    cb = C.CFUNCTYPE(None, C.c_char_p)(lambda s: logged.append(s))
    lib.setLogFunction(cb)
    for _ in range(3):
        x = g.random((1, 1, 28, 28), dtype=np.float32)
        ptr = _predict(lib, x)
        assert ptr is not None
        y = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_float)), (1, 10)).copy()
        np.testing.assert_allclose(y, onnx_front.run_graph(graph, zo, x), rtol=1e-4, atol=1e-5)
    assert b"Starting prediction...\n" in logged and b"Prediction completed.\n" in logged
    lib.setLogFunction(None)
    lib.mnist8_shutdown()


def test_generator_lifts_onnx_gemm_operands_to_the_lean_form(codegen, tmp_path):
    """debug_model.onnx (Gemm, Relu, Gemm, Relu, Softmax on a [1, 5] input): each Gemm has a 2-D A and B and a 1-D C in
    the file and reaches the executor as [1,1,M,K] x [1,1,N,K] + [1,1,1,N] between two reshape views."""
    info = codegen.generate(DEBUG_MODEL, str(tmp_path), "dbg")
    text = open(info["c"]).read()
    assert info["in_shape"] == (1, 5) and info["out_shape"] == (1, 5) and info["nodes"] == 9
    assert text.count("zant_model_gemm(m,") == 2 and text.count("zant_model_reshape(m,") == 4
    assert "(const int64_t[]){1, 1, 5, 5}" in text and "(const int64_t[]){1, 1, 1, 5}, 4," in text
    assert text.count(", 0, 1) != ") == 2          # transA = 0, transB = 1 as the file says
    assert "zant_model_softmax(m, 8)" in text
    so = codegen.compile_library(info)
    assert hasattr(_load(so), "dbg_init")


def test_generator_records_pooling_and_normalisation_nodes(codegen, tmp_path):
    g = np.random.default_rng(0)
    vec = lambda n: onnx_writer.tensor(n, (g.random(4, dtype=np.float32) + 0.5))
    nodes = [onnx_writer.node("BatchNormalization", ["x", "gamma", "beta", "mean", "var"], ["b"], epsilon=1e-3),
             onnx_writer.node("AveragePool", ["b"], ["y"], kernel_shape=[2, 2], strides=[2, 2], count_include_pad=1)]
    p = tmp_path / "pn.onnx"
    p.write_bytes(onnx_writer.model(nodes, [vec("gamma"), vec("beta"), vec("mean"), vec("var")],
                                    [onnx_writer.value_info("x", (2, 4, 8, 8), np.float32)], [onnx_writer.value_info("y", (2, 4, 4, 4), np.float32)]))
    info = codegen.generate(str(p), str(tmp_path), "pn")
    text = open(info["c"]).read()
    assert "zant_model_batchnorm(m, 0," in text and "zant_model_avgpool(m, 1," in text and info["out_shape"] == (2, 4, 4, 4)


@pytest.mark.gpu
def test_generated_debug_model_library_matches_the_oracle(codegen, tmp_path):
    from oracle import oracle as zo
    from zant_amd import onnx_front
    info = codegen.generate(DEBUG_MODEL, str(tmp_path), "dbg")
    lib = _load(codegen.compile_library(info))
    graph = onnx_front.read_graph(DEBUG_MODEL)
    g = np.random.default_rng(3)
    for _ in range(3):
        x = (g.random((1, 5), dtype=np.float32) * 4 - 2).astype(np.float32)
        ptr = _predict(lib, x)
        assert ptr is not None
        y = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_float)), (1, 5)).copy()
        np.testing.assert_allclose(y, onnx_front.run_graph(graph, zo, x), rtol=1e-4, atol=1e-5)
    lib.dbg_shutdown()


@pytest.mark.gpu
@pytest.mark.parametrize("net", ["tiny_yolo_int8", "mobilenet_v2_035_int8"])
def test_generated_int8_network_library_reproduces_the_golden_bytes(codegen, tmp_path, net):
    from zant_amd import networks as nets
    gold = json.load(open(os.path.join(HERE, "golden", "int8_networks.json")))[net]
    arch = nets.tiny_yolo_arch() if net == "tiny_yolo_int8" else nets.mobilenet_v2_035_arch()
    params = nets.int8_params(arch, seed=gold["param_seed"])
    data, out_shape = onnx_writer.int8_network(arch, params, gold["quant"], 2)
    p = tmp_path / "yolo.onnx"
    p.write_bytes(data)
    info = codegen.generate(str(p), str(tmp_path), net)
    assert info["in_dtype"] == 1 and info["out_dtype"] == 1 and tuple(info["out_shape"]) == tuple(out_shape)
    lib = _load(codegen.compile_library(info))
    x = np.random.default_rng(gold["input_seed"]).integers(0, 256, (2,) + tuple(arch["input"]), dtype=np.uint8)
    ptr = _predict(lib, x)
    assert ptr is not None
    y = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_uint8)), (int(np.prod(out_shape)),)).copy()
    np.testing.assert_array_equal(y, np.array(gold["expected_u8"], np.uint8))
    getattr(lib, net + "_shutdown")()


def test_dry_run_model_validates_and_answers_shapes_without_a_gpu(codegen):
    """A model built without a context: nodes are checked, shapes are available, nothing can run."""
    from zant_amd import ZantError
    from zant_amd.model import Model
    m = Model(None)
    x = m.input((2, 3, 16, 16))
    c = m.conv(x, np.zeros((8, 3, 3, 3), np.float32), np.zeros(8, np.float32), [1, 1], [1, 1, 1, 1], None, 1, "NOTSET")
    p = m.maxpool(m.relu(c), [2, 2], [2, 2])
    r = m.resize_nearest(p, [1.0, 1.0, 2.0, 2.0], None, "half_pixel")
    k = m.concat([c, r], 1)
    g = m.reduce_mean(m.sigmoid(k), [2, 3], False)
    assert m.tensor_shape(c) == (2, 8, 16, 16) and m.tensor_shape(p) == (2, 8, 8, 8) and m.tensor_shape(r) == (2, 8, 16, 16)
    assert m.tensor_shape(k) == (2, 16, 16, 16) and m.tensor_shape(g) == (2, 16)
    with pytest.raises(ZantError) as e:
        m.conv(x, np.zeros((8, 4, 3, 3), np.float32), None, [1, 1], None, None, 1, None)  # channel mismatch
    assert e.value.code < 0
    with pytest.raises(ZantError) as e:
        m.concat([c, p], 1)
    assert e.value.name == "MismatchedShape"
    with pytest.raises(ZantError) as e:
        m.finalize()
    assert e.value.name == "NullPointer"
    assert m.input_ptr is None
    m.close()
