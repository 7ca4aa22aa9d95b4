"""The two int8 benchmark networks (tiny-YOLO style detector; MobileNetV2-0.35 @ 96) through the model executor,
bit-exact against the oracle's golden vectors and, at the full benchmark batch, through batch-independence."""
import json
import os

import numpy as np
import pytest

import int8_ref

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "int8_networks.json")))


def _arch(nets, name):
    return nets.tiny_yolo_arch() if name == "tiny_yolo_int8" else nets.mobilenet_v2_035_arch()


@pytest.mark.parametrize("name", ["tiny_yolo_int8", "mobilenet_v2_035_int8"])
def test_network_matches_the_golden_vectors(G, name):
    from zant_amd import networks as nets
    gold = GOLD[name]
    arch = _arch(nets, name)
    assert nets.int8_macs_per_inference(arch) == gold["macs_per_inference"]
    params = nets.int8_params(arch, seed=gold["param_seed"])
    x = np.random.default_rng(gold["input_seed"]).integers(0, 256, (2,) + tuple(arch["input"]), dtype=np.uint8)
    m = nets.build_int8_model(G.tm.context(), arch, params, gold["quant"], 2)
    y = m.predict_host(x)
    np.testing.assert_array_equal(y.ravel(), np.array(gold["expected_u8"], np.uint8))
    m.close()


@pytest.mark.parametrize("name,batch", [("tiny_yolo_int8", 5), ("mobilenet_v2_035_int8", 3)])
def test_network_matches_the_oracle_on_fresh_inputs_layer_by_layer(G, name, batch):
    from zant_amd import networks as nets
    arch = _arch(nets, name)
    params = nets.int8_params(arch, seed=7)  # other weights than the golden file: scales are then off-calibration,
    quant = GOLD[name]["quant"]              # which exercises saturation at both ends
    x = np.random.default_rng(5).integers(0, 256, (batch,) + tuple(arch["input"]), dtype=np.uint8)
    ref = int8_ref.forward(arch, params, quant, x)
    m = nets.build_int8_model(G.tm.context(), arch, params, quant, batch)
    np.testing.assert_array_equal(m.predict_host(x), ref)
    m.close()


@pytest.mark.parametrize("name,batch", [("tiny_yolo_int8", 512), ("mobilenet_v2_035_int8", 1024)])
def test_full_batch_is_batch_independent_and_matches_golden_rows(G, name, batch):
    """At the benchmark batch the oracle is too slow; every image must give the result it gives alone: the two golden
    images placed at both ends of the batch reproduce the golden rows, and a permuted batch permutes the output."""
    from zant_amd import networks as nets
    gold = GOLD[name]
    arch = _arch(nets, name)
    params = nets.int8_params(arch, seed=gold["param_seed"])
    g = np.random.default_rng(11)
    x = g.integers(0, 256, (batch,) + tuple(arch["input"]), dtype=np.uint8)
    xg = np.random.default_rng(gold["input_seed"]).integers(0, 256, (2,) + tuple(arch["input"]), dtype=np.uint8)
    x[0], x[-1] = xg[0], xg[1]
    m = nets.build_int8_model(G.tm.context(), arch, params, gold["quant"], batch)
    y = m.predict_host(x).reshape(batch, -1)
    exp = np.array(gold["expected_u8"], np.uint8).reshape(2, -1)
    np.testing.assert_array_equal(y[0], exp[0])
    np.testing.assert_array_equal(y[-1], exp[1])
    perm = g.permutation(batch)
    y2 = m.predict_host(np.ascontiguousarray(x[perm])).reshape(batch, -1)
    np.testing.assert_array_equal(y2, y[perm])
    m.close()


@pytest.mark.parametrize("name", ["tiny_yolo_int8", "mobilenet_v2_035_int8"])
def test_network_through_the_onnx_front_end(G, name, tmp_path):
    """The same networks written as ONNX files in operator form, read back by the protobuf reader and turned into an
    executor model node by node: same golden bytes, same number of launches as the direct construction."""
    import onnx_writer
    from zant_amd import networks as nets
    from zant_amd import onnx_front
    gold = GOLD[name]
    arch = _arch(nets, name)
    params = nets.int8_params(arch, seed=gold["param_seed"])
    data, out_shape = onnx_writer.int8_network(arch, params, gold["quant"], 2)
    path = tmp_path / (name + ".onnx")
    path.write_bytes(data)
    graph = onnx_front.read_graph(str(path))
    assert graph["elem_types"]["input"] == 2 and tuple(graph["outputs"][0][1]) == tuple(out_shape)
    m = onnx_front.build_model(G.tm.context(), graph)
    direct = nets.build_int8_model(G.tm.context(), arch, params, gold["quant"], 2)
    assert m.num_launches == direct.num_launches
    x = np.random.default_rng(gold["input_seed"]).integers(0, 256, (2,) + tuple(arch["input"]), dtype=np.uint8)
    np.testing.assert_array_equal(m.predict_host(x).ravel(), np.array(gold["expected_u8"], np.uint8))
    m.close(); direct.close()


def test_float_graph_with_a_quantised_island_through_the_onnx_front_end(G, tmp_path):
    """f32 input -> QuantizeLinear -> QLinearConv -> DequantizeLinear -> Relu: the Q / DQ nodes stay executor nodes of
    their own (nothing to fold them into) and the f32 result equals the oracle's bit for bit (both sides compute
    (q - zp) * scale in f32)."""
    import onnx_writer as ow
    from oracle import oracle as zo
    from zant_amd import onnx_front
    g = np.random.default_rng(3)
    N, C, H, W, K = 3, 8, 12, 12, 16
    x = g.standard_normal((N, C, H, W)).astype(np.float32) * 2
    w = g.integers(-127, 128, (K, C, 3, 3), dtype=np.int8)
    ws = g.uniform(0.001, 0.003, K).astype(np.float32)
    b = g.integers(-50, 50, K, dtype=np.int32)
    xs, xz, ys, yz = np.float32(0.03), 120, np.float32(0.05), 131
    inits = [ow.tensor("xs", xs), ow.tensor("xz", np.uint8(xz)), ow.tensor("w", w), ow.tensor("ws", ws),
             ow.tensor("wz", np.zeros(K, np.int8)), ow.tensor("ys", ys), ow.tensor("yz", np.uint8(yz)), ow.tensor("b", b)]
    nodes = [ow.node("QuantizeLinear", ["x", "xs", "xz"], ["xq"]),
             ow.node("QLinearConv", ["xq", "xs", "xz", "w", "ws", "wz", "ys", "yz", "b"], ["yq"], strides=[1, 1], pads=[1, 1, 1, 1],
                     kernel_shape=[3, 3]),
             ow.node("DequantizeLinear", ["yq", "ys", "yz"], ["yf"]),
             ow.node("Relu", ["yf"], ["y"])]
    path = tmp_path / "island.onnx"
    path.write_bytes(ow.model(nodes, inits, [ow.value_info("x", x.shape, np.float32)], [ow.value_info("y", (N, K, H, W), np.float32)]))
    m = onnx_front.build_model(G.tm.context(), onnx_front.read_graph(str(path)))
    xq = zo.quantize_linear(x, xs, xz)
    yq = zo.qlinearconv(xq, xs, xz, w, ws, None, ys, yz, b, [1, 1], [1, 1, 1, 1], [1, 1], 1)
    ref = np.maximum(zo.dequantize_linear(yq, ys, yz), 0)
    np.testing.assert_array_equal(m.predict_host(x).reshape(ref.shape), ref)
    m.close()


def test_onnx_front_end_rejects_what_the_executor_does_not_cover(G, tmp_path):
    import onnx_writer as ow
    from zant_amd import onnx_front
    K = 4
    base = [ow.tensor("xs", np.float32(0.1)), ow.tensor("xz", np.uint8(3)), ow.tensor("w", np.ones((K, 2, 1, 1), np.int8)),
            ow.tensor("ws", np.ones(K, np.float32)), ow.tensor("ys", np.float32(0.2)), ow.tensor("yz", np.uint8(0))]

    def graph(wz, xz_name="xz", extra=()):
        nodes = [ow.node("QLinearConv", ["x", "xs", xz_name, "w", "ws", "wz", "ys", "yz"], ["y"], kernel_shape=[1, 1])]
        p = tmp_path / "g.onnx"
        p.write_bytes(ow.model(nodes, base + [ow.tensor("wz", wz)] + list(extra), [ow.value_info("x", (1, 2, 4, 4), np.uint8)],
                               [ow.value_info("y", (1, K, 4, 4), np.uint8)]))
        return onnx_front.read_graph(str(p))

    with pytest.raises(NotImplementedError):  # weight zero points other than 0
        onnx_front.build_model(G.tm.context(), graph(np.array([0, 1, 0, 0], np.int8)))
    m = onnx_front.build_model(G.tm.context(), graph(np.zeros(K, np.int8)))
    m.close()
    # a second reader naming other parameters for the same tensor than its producer
    nodes = [ow.node("QLinearConv", ["x", "xs", "xz", "w", "ws", "wz", "ys", "yz"], ["t"], kernel_shape=[1, 1]),
             ow.node("QLinearGlobalAveragePool", ["t", "xs", "yz", "ys", "yz"], ["y"], domain="com.microsoft")]
    p = tmp_path / "h.onnx"
    p.write_bytes(ow.model(nodes, base + [ow.tensor("wz", np.zeros(K, np.int8))], [ow.value_info("x", (1, 2, 4, 4), np.uint8)],
                           [ow.value_info("y", (1, K, 1, 1), np.uint8)]))
    with pytest.raises(ValueError):
        onnx_front.build_model(G.tm.context(), onnx_front.read_graph(str(p)))
