"""The fused inverted-residual block kernel (1x1 expansion -> depthwise 3x3 -> 1x1 projection [-> Add]) against the
oracle run layer by layer, bit-exact, over shapes that exercise every tiling branch of the kernel."""
import numpy as np
import pytest

import int8_ref

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def _conv(k, stride, pad, cin, cout, group, act, alpha=0.0):
    d = dict(op="conv", k=k, stride=stride, pad=pad, cin=cin, cout=cout, group=group, act=act)
    if act == "leaky":
        d["alpha"] = alpha
    return d


def _arch(hw, c0, blocks, tail=8):
    """3x3 stem (so that the first block reads a blocked tensor), the blocks, a 1x1 tail (so that the last block writes
    one).  blocks: (hidden, cout, stride, act_expand, act_dw, dw_pad)."""
    layers = [_conv(3, 1, 1, 3, c0, 1, "relu6")]
    cin = c0
    for hidden, cout, stride, act_e, act_d, dw_pad in blocks:
        block_in = len(layers) - 1
        layers.append(_conv(1, 1, 0, cin, hidden, 1, act_e, 0.1))
        layers.append(_conv(3, stride, dw_pad, hidden, hidden, hidden, act_d, 0.1))
        layers.append(_conv(1, 1, 0, hidden, cout, 1, None))
        if stride == 1 and cin == cout and dw_pad == 1:
            layers.append(dict(op="add", res=block_in))
        cin = cout
    layers.append(_conv(1, 1, 0, cin, tail, 1, None))
    return dict(name="blocks", input=(3,) + tuple(hw), layers=layers)


CASES = [
    # (H, W), stem channels, blocks, batch, expected launches
    ((13, 13), 8, [(48, 8, 1, "relu6", "relu6", 1)], 5, 3),                      # residual, odd size, Ce padded 48 -> 64
    ((14, 14), 16, [(96, 24, 2, "relu6", "relu6", 1)], 3, 3),                    # stride 2
    ((7, 9), 24, [(40, 56, 1, "relu6", "relu6", 1)], 7, 3),                      # ragged channels, two output chunks
    ((6, 6), 16, [(64, 16, 1, "leaky", None, 1)], 4, 3),                          # other activations / none
    ((5, 5), 56, [(72, 112, 1, "relu6", "relu6", 1)], 9, 3),                     # four output chunks, whole CU's LDS
    ((40, 40), 8, [(48, 8, 1, "relu6", "relu6", 1)], 2, 3),                      # row tiles with halo, residual
    ((41, 37), 8, [(48, 16, 2, "relu6", "relu6", 1)], 2, 3),                     # row tiles, stride 2, odd sizes
    ((12, 12), 16, [(96, 16, 1, "relu6", "relu6", 1), (96, 24, 2, "relu6", "relu6", 1)], 6, 3),  # two blocks in a row: one launch
    ((9, 9), 8, [(48, 8, 1, "relu6", "relu6", 0)], 3, 5),                        # pad-0 depthwise: not the pattern, unfused
    ((1, 1), 8, [(16, 8, 1, "relu6", "relu6", 1)], 7, 3),                        # one pixel, one half-filled expanded chunk
    ((2, 3), 5, [(30, 128, 2, "relu6", "relu6", 1)], 1, 3),                      # batch 1, ragged input channels, 128 outputs
    ((3, 3), 8, [(48, 8, 1, "relu6", "relu6", 1)], 1030, 3),                     # more images than one pass of tiles
    ((24, 24), 40, [(240, 40, 1, "relu6", "relu6", 1)], 2, 3),                   # three input blocks, many expanded chunks
    ((17, 5), 8, [(16, 24, 2, None, "leaky", 1)], 3, 3),                         # tall narrow map, stride 2
]


@pytest.mark.parametrize("hw,c0,blocks,batch,launches", CASES)
def test_fused_block_matches_the_oracle(G, hw, c0, blocks, batch, launches):
    from zant_amd import networks as nets
    arch = _arch(hw, c0, blocks)
    params = nets.int8_params(arch, seed=3)
    rng = np.random.default_rng(11)
    quant = int8_ref.calibrate(arch, params, rng.integers(0, 256, (2,) + arch["input"], dtype=np.uint8))
    x = rng.integers(0, 256, (batch,) + arch["input"], dtype=np.uint8)
    ref = int8_ref.forward(arch, params, quant, x)
    m = nets.build_int8_model(G.tm.context(), arch, params, quant, batch)
    assert m.num_launches == launches
    np.testing.assert_array_equal(m.predict_host(x), ref)
    # a second pass over other data reuses the packed weights
    x2 = rng.integers(0, 256, x.shape, dtype=np.uint8)
    np.testing.assert_array_equal(m.predict_host(x2), int8_ref.forward(arch, params, quant, x2))
    m.close()


def test_fused_block_saturates_like_the_oracle(G):
    """Scales far off calibration drive every stage into saturation at both ends."""
    from zant_amd import networks as nets
    arch = _arch((10, 10), 8, [(48, 8, 1, "relu6", "relu6", 1)])
    params = nets.int8_params(arch, seed=5)
    rng = np.random.default_rng(2)
    quant = int8_ref.calibrate(arch, params, rng.integers(0, 256, (2,) + arch["input"], dtype=np.uint8))
    for q in quant["layers"]:
        if q:
            q[0] = float(np.float32(q[0]) * np.float32(0.2))
    x = rng.integers(0, 256, (4,) + arch["input"], dtype=np.uint8)
    ref = int8_ref.forward(arch, params, quant, x)
    assert (ref == 0).any() and (ref == 255).any()
    m = nets.build_int8_model(G.tm.context(), arch, params, quant, 4)
    np.testing.assert_array_equal(m.predict_host(x), ref)
    m.close()
