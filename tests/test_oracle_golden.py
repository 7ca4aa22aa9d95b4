"""The CPU oracle against every known-answer vector the reference's own tests hold for the hot path."""
import numpy as np
import pytest

from conftest import cases_for
from oracle import oracle as zo


def T(d, dtype=np.float32):
    return None if d is None else np.array(d["data"], dtype=dtype).reshape(d["shape"])


@pytest.mark.parametrize("c", cases_for("convolve_tensor_with_bias"))
def test_convolve_tensor_with_bias(c):
    y = zo.convolve_tensor_with_bias(T(c["x"]), T(c["w"]), T(c["bias"]), c["stride"], c["dilations"])
    assert list(y.shape) == c["expect"]["shape"]
    np.testing.assert_array_equal(y, T(c["expect"]))


@pytest.mark.parametrize("c", cases_for("conv_lean", "Conv"))
def test_conv(c):
    x, w, b = T(c["x"]), T(c["w"]), T(c["bias"])
    if c["op"] == "conv_lean":
        y = np.zeros(c["expect"]["shape"], np.float32)
        zo.conv_lean(x, w, y, b, c["stride"], c["pads"], c["dilations"], c["group"], c["auto_pad"])
    else:
        y = zo.Conv(x, w, b, c["stride"], c["pads"], c["dilations"], c["group"], c["auto_pad"])
    assert list(y.shape) == c["expect"]["shape"]
    np.testing.assert_array_equal(y, T(c["expect"]))


@pytest.mark.parametrize("c", cases_for("gemm"))
def test_gemm(c):
    y = zo.gemm(T(c["a"]), T(c["b"]), T(c["c"]), c["alpha"], c["beta"], c["transA"], c["transB"])
    assert list(y.shape) == c["expect_shape"]
    for i, v in c["expect_at"].items():
        assert y.ravel()[int(i)] == v


@pytest.mark.parametrize("c", cases_for("gemm_error"))
def test_gemm_errors(c):
    a, b = np.zeros(c["a_shape"], np.float32), np.zeros(c["b_shape"], np.float32)
    with pytest.raises(zo.OracleError) as e:
        zo.gemm(a, b, None, 1, 1, c["transA"], c["transB"])
    assert e.value.name == c["error"]


@pytest.mark.parametrize("c", cases_for("mat_mul"))
def test_mat_mul(c):
    y = zo.mat_mul(T(c["a"]), T(c["b"]))
    assert list(y.shape) == c["expect_shape"]
    for i, v in c["expect_at"].items():
        assert y.ravel()[int(i)] == v


@pytest.mark.parametrize("c", cases_for("mat_mul_error"))
def test_mat_mul_errors(c):
    with pytest.raises(zo.OracleError) as e:
        zo.mat_mul(np.zeros(c["a_shape"], np.float32), np.zeros(c["b_shape"], np.float32))
    assert e.value.name == c["error"]


@pytest.mark.parametrize("c", cases_for("onnx_maxpool"))
def test_maxpool(c):
    y = zo.onnx_maxpool(T(c["x"]), c["kernel"], c["strides"], c["dilations"], c["pads"], c["auto_pad"], c["ceil_mode"])
    assert list(y.shape) == c["expect"]["shape"]
    np.testing.assert_array_equal(y, T(c["expect"]))
    # the u8 variant is order preserving: identical on the same integers
    yq = zo.onnx_maxpool(T(c["x"], np.uint8), c["kernel"], c["strides"], c["dilations"], c["pads"], c["auto_pad"], c["ceil_mode"])
    np.testing.assert_array_equal(yq, T(c["expect"], np.uint8))


@pytest.mark.parametrize("c", cases_for("ReLU"))
def test_relu(c):
    np.testing.assert_array_equal(zo.ReLU(T(c["x"])), T(c["expect"]))


def test_relu_lean_keeps_previous_content():
    # lib_activation_function_math.zig:25-27 has no else branch
    y = np.full(4, 7.0, np.float32)
    zo.ReLU_lean(np.array([1, -2, -4, 5], np.float32), y)
    np.testing.assert_array_equal(y, [1, 7, 7, 5])


@pytest.mark.parametrize("c", cases_for("leakyReLU"))
def test_leaky(c):
    y = zo.leakyReLU(T(c["x"]), c["slope"])
    assert np.all(np.abs(y - T(c["expect"])) <= c["atol"])


@pytest.mark.parametrize("c", cases_for("softmax"))
def test_softmax(c):
    y = zo.softmax(T(c["x"]))
    if c["property"] == "rows_sum_to_1_within_0.1":
        assert np.all(np.abs(y.sum(axis=1) - 1) < 0.1)
    else:
        assert y[0, 0] == y[0, 1] and y[1, 0] == y[1, 1]


@pytest.mark.parametrize("c", cases_for("sum_tensors"))
def test_sum_tensors(c):
    np.testing.assert_array_equal(zo.sum_tensors_lean(T(c["a"]), T(c["b"])), T(c["expect"]))


@pytest.mark.parametrize("c", cases_for("add_bias"))
def test_add_bias(c):
    t = T(c["t"]).copy()
    np.testing.assert_array_equal(zo.add_bias(t, T(c["bias"])), T(c["expect"]))


@pytest.mark.parametrize("c", cases_for("reshape"))
def test_reshape(c):
    x = T(c["x"], np.uint8)
    if "error" in c:
        with pytest.raises(zo.OracleError) as e:
            zo.reshape_lean(x, c["new_shape"])
        assert e.value.name == c["error"]
    else:
        y = zo.reshape_lean(x, c["new_shape"])
        assert list(y.shape) == c["expect_shape"]
        np.testing.assert_array_equal(y.ravel(), x.ravel())


@pytest.mark.parametrize("c", cases_for("sigmoid"))
def test_sigmoid(c):
    assert np.all(np.abs(zo.sigmoid(T(c["x"])) - T(c["expect"])) < c["atol"])


@pytest.mark.parametrize("c", cases_for("reduce_mean"))
def test_reduce_mean(c):
    y = zo.reduce_mean(T(c["x"]), c["axes"], c["keepdims"], c["noop"])
    if "expect" in c:
        assert list(y.shape) == c["expect"]["shape"]
        assert np.all(np.abs(y - T(c["expect"])) <= c["atol"])
    else:
        assert list(y.shape) == c["expect_shape"]
        assert np.all(np.abs(y.ravel()[:len(c["expect_first"])] - np.array(c["expect_first"], np.float32)) <= c["atol"])


@pytest.mark.parametrize("c", cases_for("concatenate"))
def test_concatenate(c):
    ts = [T(t) for t in c["tensors"]]
    if "error" in c:
        with pytest.raises(zo.OracleError) as e:
            zo.concatenate(ts, c["axis"])
        assert e.value.name == c["error"]
        return
    y = zo.concatenate(ts, c["axis"])
    if "expect" in c:
        assert list(y.shape) == c["expect"]["shape"]
        np.testing.assert_array_equal(y, T(c["expect"]))
    else:
        assert list(y.shape) == c["expect_shape"]


@pytest.mark.parametrize("c", cases_for("concatenate_shape"))
def test_concatenate_shape(c):
    ts = [np.zeros(s, np.float32) for s in c["shapes"]]
    if "error" in c:
        with pytest.raises(zo.OracleError) as e:
            zo.concatenate(ts, c["axis"])
        assert e.value.name == c["error"]
    else:
        assert list(zo.concatenate(ts, c["axis"]).shape) == c["expect_shape"]


@pytest.mark.parametrize("c", cases_for("resize", "resize_shape"))
def test_resize(c):
    x = T(c["x"], np.uint8) if "x" in c else np.zeros(c["shape"], np.uint8)
    args = (x, c.get("mode", "nearest"), c["scales"], c["sizes"], c.get("coord", "half_pixel"))
    if "error" in c:
        with pytest.raises(zo.OracleError) as e:
            zo.resize(*args)
        assert e.value.name == c["error"]
        return
    y = zo.resize(*args)
    assert list(y.shape) == c["expect_shape"]
    if "expect_first" in c:
        assert list(y.ravel()[:len(c["expect_first"])]) == c["expect_first"]


def test_conv_error_paths():
    # group != 1 -> InvalidDimensions (op_convolution.zig:59-65)
    x, w = np.zeros((1, 2, 4, 4), np.float32), np.zeros((2, 1, 3, 3), np.float32)
    with pytest.raises(zo.OracleError) as e:
        zo.conv_lean(x, w, np.zeros((1, 2, 2, 2), np.float32), None, [1, 1], None, None, 2, None)
    assert e.value.name == "InvalidDimensions"
    # auto_pad NOTSET without pads -> InvalidPadding (:120-125)
    w = np.zeros((2, 2, 3, 3), np.float32)
    with pytest.raises(zo.OracleError) as e:
        zo.conv_lean(x, w, np.zeros((1, 2, 2, 2), np.float32), None, [1, 1], None, None, 1, "NOTSET")
    assert e.value.name == "InvalidPadding"
    # output shape mismatch -> InvalidDimensions (:212-217)
    with pytest.raises(zo.OracleError) as e:
        zo.conv_lean(x, w, np.zeros((1, 2, 3, 3), np.float32), None, [1, 1], None, None, 1, None)
    assert e.value.name == "InvalidDimensions"
    # rank != 4 -> InvalidDimensions (:44-46)
    with pytest.raises(zo.OracleError) as e:
        zo.conv_lean(x[0], w, np.zeros((1, 2, 2, 2), np.float32), None, [1, 1])
    assert e.value.name == "InvalidDimensions"
    # pads are ignored unless auto_pad == "NOTSET": the allocating wrapper then
    # expects the padded shape and the lean call reports the mismatch (:725-728 vs :86)
    with pytest.raises(zo.OracleError) as e:
        zo.Conv(x, w, None, [1, 1], [1, 1, 1, 1], None, 1, None)
    assert e.value.name == "InvalidDimensions"


def test_onnx_reader_decodes_the_bundled_mnist8_graph():
    """The reader needs no GPU: node list, attributes and initialiser shapes of mnist-8.onnx are what the reference's
    hand-written translation of the same file lists (src/codeGen/hardcoded/hardcoded_mnist8.zig:140-288)."""
    import importlib.util
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("onnx_front", os.path.join(root, "z-ant_amd", "onnx_front.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    g = mod.read_graph(os.path.join(root, "tests", "golden", "mnist-8.onnx"))
    assert [n["op"] for n in g["nodes"]] == ["Reshape", "Conv", "Add", "Relu", "MaxPool", "Conv", "Add", "Relu", "MaxPool",
                                             "Reshape", "MatMul", "Add"]
    assert g["nodes"][1]["attrs"]["auto_pad"] == "SAME_UPPER" and g["nodes"][1]["attrs"]["kernel_shape"] == [5, 5]
    assert g["nodes"][8]["attrs"]["kernel_shape"] == [3, 3] and g["nodes"][8]["attrs"]["strides"] == [3, 3]
    shapes = {k: v.shape for k, v in g["initializers"].items()}
    assert shapes["Parameter5"] == (8, 1, 5, 5) and shapes["Parameter87"] == (16, 8, 5, 5)
    assert shapes["Parameter6"] == (8, 1, 1) and shapes["Parameter193"] == (16, 4, 4, 10) and shapes["Parameter194"] == (1, 10)
    assert g["inputs"] == [("Input3", [1, 1, 28, 28])] and g["outputs"] == [("Plus214_Output_0", [1, 10])]


def test_onnx_reader_decodes_a_quantised_graph_written_by_the_test_writer(tmp_path):
    """Round trip through the wire format without a GPU: node list, attributes, typed initialisers, element types."""
    import importlib.util
    import os
    import sys
    import onnx_writer
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("zant_onnx_front", os.path.join(root, "z-ant_amd", "onnx_front.py"))
    front = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(front)
    arch = dict(name="t", input=(3, 8, 8), layers=[
        dict(op="conv", k=3, stride=2, pad=1, cin=3, cout=8, group=1, act="leaky", alpha=0.1),
        dict(op="pool"),
        dict(op="conv", k=1, stride=1, pad=0, cin=8, cout=8, group=1, act="relu6"),
        dict(op="add", res=1),
        dict(op="gap")])
    g = np.random.default_rng(0)
    params = [dict(w=g.integers(-127, 128, (8, 3, 3, 3), dtype=np.int8), w_scale=g.random(8, dtype=np.float32), bias=g.integers(-9, 9, 8, dtype=np.int32)),
              None, dict(w=g.integers(-127, 128, (8, 8, 1, 1), dtype=np.int8), w_scale=g.random(8, dtype=np.float32), bias=g.integers(-9, 9, 8, dtype=np.int32)),
              None, None]
    quant = {"input": [0.02, 128], "layers": [[0.05, 128, 0.04, 30], None, [0.06, 120, 0.03, 0], [0.07, 100], [0.07, 100]]}
    data, shape = onnx_writer.int8_network(arch, params, quant, 2)
    path = tmp_path / "q.onnx"
    path.write_bytes(data)
    graph = front.read_graph(str(path))
    ops = [n["op"] for n in graph["nodes"]]
    assert ops == ["QLinearConv", "DequantizeLinear", "LeakyRelu", "QuantizeLinear", "MaxPool", "QLinearConv", "DequantizeLinear",
                   "Clip", "QuantizeLinear", "QLinearAdd", "QLinearGlobalAveragePool"]
    assert graph["elem_types"]["input"] == 2 and graph["inputs"][0][1] == [2, 3, 8, 8] and tuple(graph["outputs"][0][1]) == shape
    conv = graph["nodes"][0]
    assert conv["attrs"]["strides"] == [2, 2] and conv["attrs"]["pads"] == [1, 1, 1, 1] and conv["attrs"]["group"] == 1
    np.testing.assert_array_equal(graph["initializers"][conv["inputs"][3]], params[0]["w"])
    np.testing.assert_array_equal(graph["initializers"][conv["inputs"][8]], params[0]["bias"])
    assert graph["initializers"][conv["inputs"][1]].dtype == np.float32 and graph["initializers"][conv["inputs"][2]].dtype == np.uint8
    assert abs(graph["nodes"][2]["attrs"]["alpha"] - 0.1) < 1e-7
