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
