"""Bit-exact parity of the patch-stationary int8 convolution kernel (3x3, stride 1, at least 32 input and 33 output
channels) with the CPU oracle: every path of its tiling and of its epilogues."""
import numpy as np
import pytest

from oracle import oracle as zo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def _operands(seed, N, C, H, W, K):
    g = np.random.default_rng(seed)
    x = g.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = g.integers(-127, 128, (K, C, 3, 3), dtype=np.int8)
    ws = (g.uniform(0.5, 1.5, K) * 0.08 / np.sqrt(9 * C)).astype(np.float32)
    b = g.integers(-1000, 1001, K, dtype=np.int32)
    return x, w, ws, b


PS_CASES = [
    # N, C, H, W, K, pads                    what the shape exercises
    (3, 64, 12, 12, 96, [1, 1, 1, 1]),       # several whole images per tile; 96 channels in a pass of 128
    (2, 32, 9, 13, 40, [0, 1, 0, 1]),        # one channel chunk, a pass of 64 channels, asymmetric padding
    (1, 160, 6, 6, 256, [1, 1, 1, 1]),       # two output-channel passes, five channel chunks
    (5, 48, 30, 30, 64, [1, 1, 1, 1]),       # odd number of 16-channel blocks, row tiles with a short last tile
    (2, 128, 28, 28, 128, [0, 0, 0, 0]),     # no padding
    (7, 40, 5, 5, 72, [1, 1, 1, 1]),         # channels not a multiple of 16, images not a multiple of the tile
    (2, 256, 7, 9, 200, [1, 0, 1, 0]),       # eight chunks, ragged output channels
]


@pytest.mark.parametrize("case", PS_CASES, ids=[str(i) for i in range(len(PS_CASES))])
@pytest.mark.parametrize("act", [None, "leaky"])
def test_patch_stationary_shapes_bit_exact(G, case, act):
    N, C, H, W, K, pads = case
    x, w, ws, b = _operands(11 * N + C + K, N, C, H, W, K)
    kw = dict(act=act, act_alpha=0.1, act_scale=0.04, act_zp=30) if act else {}
    ref = zo.qlinearconv(x, 0.02, 128, w, ws, None, 0.05, 128, b, [1, 1], pads, [1, 1], 1, **kw)
    y = G.tm.qlinearconv(G.dev(x), 0.02, 128, G.dev(w), G.dev(ws), None, 0.05, 128, G.dev(b), [1, 1], pads, [1, 1], 1, **kw)
    np.testing.assert_array_equal(G.host(y), ref)
    assert len(np.unique(ref)) > 8


@pytest.mark.parametrize("C", [32, 64])
def test_more_tiles_than_compute_units(G, C):
    """Every workgroup walks several tiles: with one channel chunk the next tile's patch goes in at once, with two it
    streams in during the last step of the current tile."""
    N, H, K = 1100, 14, 64
    x, w, ws, b = _operands(C, N, C, H, H, K)
    ref = zo.qlinearconv(x, 0.02, 128, w, ws, None, 0.05, 128, b, [1, 1], [1, 1, 1, 1], [1, 1], 1)
    y = G.host(G.tm.qlinearconv(G.dev(x), 0.02, 128, G.dev(w), G.dev(ws), None, 0.05, 128, G.dev(b), [1, 1], [1, 1, 1, 1], [1, 1], 1))
    np.testing.assert_array_equal(y, ref)


def test_blocked_in_and_out_inside_a_model(G):
    """Three convolutions in a row: the middle one reads and writes the channel-blocked layout (once without and once
    with a fused activation), the first reads NCHW, the last writes it."""
    from zant_amd.model import Model, U8
    N, C, H = 6, 64, 20
    g = np.random.default_rng(5)
    x = g.integers(0, 256, (N, C, H, H), dtype=np.uint8)
    layers = [_operands(100 + i, 1, C, 4, 4, C)[1:] for i in range(3)]
    for act in (None, "relu6"):
        m = Model(G.tm.context())
        t = m.input((N, C, H, H), U8, 0.02, 128)
        ref, s, z = x, 0.02, 128
        for i, (w, ws, b) in enumerate(layers):
            t = m.qlinearconv(t, w, ws, b, 0.05, 120 + i, [1, 1], [1, 1, 1, 1])
            ref = zo.qlinearconv(ref, s, z, w, ws, None, 0.05, 120 + i, b, [1, 1], [1, 1, 1, 1], [1, 1], 1)
            s, z = 0.05, 120 + i
            if act and i == 1:
                t = m.qlinear_act(t, act, 0.0, 0.03, 10)
                ref = zo.qlinear_act(ref, s, z, act, 0.0, 0.03, 10)
                s, z = 0.03, 10
        m.finalize()
        y = m.predict_host(x)
        np.testing.assert_array_equal(y, ref)


# An NCHW input with whole 16-channel blocks and rows of whole, aligned dwords is regrouped by the kernel itself (no
# blocked copy is written first): a tile's whole patch goes to LDS before the tile's first step.
DIRECT_CASES = [
    # N, C, H, W, K, pads, x_zp
    (3, 64, 12, 12, 96, [1, 1, 1, 1], 128),    # several whole images per tile, two channel chunks
    (2, 128, 28, 28, 128, [0, 0, 0, 0], 128),  # no padding: the patch has no halo columns
    (5, 48, 14, 28, 96, [1, 1, 1, 1], 3),      # odd number of 16-channel blocks (the last half chunk is padding), row tiles
    (600, 64, 8, 8, 64, [1, 1, 1, 1], 200),    # several tiles per workgroup: the patch is refilled tile after tile
    (7, 32, 8, 16, 40, [1, 0, 1, 0], 77),      # one chunk, padding on the top / left only, images not a multiple of the tile
    (2, 96, 12, 12, 200, [1, 1, 1, 1], 0),     # two output-channel passes over one patch, three chunks
]


@pytest.mark.parametrize("case", DIRECT_CASES, ids=[str(i) for i in range(len(DIRECT_CASES))])
def test_nchw_input_read_directly_bit_exact(G, case):
    N, C, H, W, K, pads, x_zp = case
    x, w, ws, b = _operands(13 * N + C + K, N, C, H, W, K)
    y = G.tm.qlinearconv(G.dev(x), 0.02, x_zp, G.dev(w), G.dev(ws), None, 0.05, 128, G.dev(b), [1, 1], pads, [1, 1], 1)
    name = G.tm.context().kernel_name()
    assert name.startswith("qconv_ps_kernel<") and name.endswith(",true>"), name
    pick = list(range(N)) if N <= 8 else [0, 1, N // 2, N - 2, N - 1]
    ref = zo.qlinearconv(x[pick], 0.02, x_zp, w, ws, None, 0.05, 128, b, [1, 1], pads, [1, 1], 1)
    np.testing.assert_array_equal(G.host(y)[pick], ref)


def test_nchw_input_that_needs_the_blocked_copy(G):
    """Rows that are not whole dwords, or an input that is not 4-byte aligned, take the blocked copy as before."""
    import torch
    N, C, H, W, K = 3, 64, 10, 14, 64
    x, w, ws, b = _operands(5, N, C, H, W, K)
    ref = zo.qlinearconv(x, 0.02, 128, w, ws, None, 0.05, 128, b, [1, 1], [1, 1, 1, 1], [1, 1], 1)
    y = G.tm.qlinearconv(G.dev(x), 0.02, 128, G.dev(w), G.dev(ws), None, 0.05, 128, G.dev(b), [1, 1], [1, 1, 1, 1], [1, 1], 1)
    assert G.tm.context().kernel_name().endswith(",false>"), G.tm.context().kernel_name()
    np.testing.assert_array_equal(G.host(y), ref)
    # the same tensor of 16-column rows, one byte off alignment
    N, C, H, W, K = 2, 32, 8, 16, 64
    x, w, ws, b = _operands(6, N, C, H, W, K)
    ref = zo.qlinearconv(x, 0.02, 128, w, ws, None, 0.05, 128, b, [1, 1], [1, 1, 1, 1], [1, 1], 1)
    buf = torch.zeros(x.size + 1, dtype=torch.uint8, device="cuda:0")
    xo = buf[1:].view(N, C, H, W)
    xo.copy_(G.dev(x))
    y = G.tm.qlinearconv(xo, 0.02, 128, G.dev(w), G.dev(ws), None, 0.05, 128, G.dev(b), [1, 1], [1, 1, 1, 1], [1, 1], 1)
    assert G.tm.context().kernel_name().endswith(",false>"), G.tm.context().kernel_name()
    np.testing.assert_array_equal(G.host(y), ref)


# NCHW output whose plane runs are made of aligned 4- or 8-byte units is staged through LDS and written out as whole
# runs: a staging region of its own, or -- one tile per workgroup, one pass -- the one laid over the dead ring and patch.
STAGED_CASES = [
    # N, C, H, W, K, pads
    (4, 32, 8, 8, 64, [1, 1, 1, 1]),         # 8-byte units, a staging region of its own
    (300, 32, 8, 8, 64, [1, 1, 1, 1]),       # the same with several tiles per workgroup: staging rows are rewritten
    (2, 64, 12, 12, 200, [1, 1, 1, 1]),      # two output-channel passes, ragged channels
    (3, 32, 9, 12, 40, [1, 1, 1, 1]),        # planes of 108 bytes: 4-byte units
    (2, 128, 28, 28, 128, [1, 1, 1, 1]),     # too large for a region of its own: laid over ring, slot table and patch
    (5, 48, 14, 28, 96, [1, 1, 1, 1]),       # row tiles that do not divide the rows (short last tile), whole-unit rows
]


@pytest.mark.parametrize("case", STAGED_CASES, ids=[str(i) for i in range(len(STAGED_CASES))])
@pytest.mark.parametrize("act", [None, "relu6"])
def test_staged_nchw_write_out_bit_exact(G, case, act):
    N, C, H, W, K, pads = case
    x, w, ws, b = _operands(7 * N + C + K, N, C, H, W, K)
    kw = dict(act=act, act_alpha=0.0, act_scale=0.03, act_zp=0) if act else {}
    y = G.tm.qlinearconv(G.dev(x), 0.02, 128, G.dev(w), G.dev(ws), None, 0.05, 128, G.dev(b), [1, 1], pads, [1, 1], 1, **kw)
    assert G.tm.context().kernel_name().startswith("qconv_ps_kernel<"), G.tm.context().kernel_name()
    assert G.tm.context().kernel_name().rstrip(">").split(",")[1] in ("4", "5"), "the staged write-out did not run"
    pick = list(range(N)) if N <= 8 else [0, 1, N // 2, N - 2, N - 1]
    ref = zo.qlinearconv(x[pick], 0.02, 128, w, ws, None, 0.05, 128, b, [1, 1], pads, [1, 1], 1, **kw)
    np.testing.assert_array_equal(G.host(y)[pick], ref)


# The fused 2x2/2 max pool (blocked tensors on both sides, inside a model): the pool is taken on the accumulators, one
# value in four is requantised, and the pooled bytes are staged and written out as whole 16-byte units.
POOL_CASES = [
    # N, C, H, W, K                what the shape exercises
    (6, 32, 24, 24, 64),           # one image per tile, a pass of 64 channels, several tiles per workgroup at larger N
    (5, 64, 12, 12, 128),          # several images per tile, two channel chunks, a pass of 128 channels
    (3, 48, 20, 28, 72),           # row tiles (TH < OH), ragged channels on both sides
    (700, 32, 8, 8, 40),           # many tiles per workgroup: the staging rows are rewritten tile after tile
]


@pytest.mark.parametrize("case", POOL_CASES, ids=[str(i) for i in range(len(POOL_CASES))])
@pytest.mark.parametrize("act", ["leaky", None])
def test_fused_pool_bit_exact_inside_a_model(G, case, act):
    from zant_amd.model import Model, U8
    N, C, H, W, K = case
    x, w, ws, b = _operands(3 * N + C + K, N, C, H, W, K)
    g = np.random.default_rng(N)
    w0 = g.integers(-127, 128, (C, 3, 3, 3), dtype=np.int8)   # a first layer brings the input into the blocked layout
    ws0 = (g.uniform(0.5, 1.5, C) * 0.08 / np.sqrt(27)).astype(np.float32)
    x0 = g.integers(0, 256, (N, 3, H, W), dtype=np.uint8)
    m = Model(G.tm.context())
    t = m.input((N, 3, H, W), U8, 0.02, 128)
    t = m.qlinearconv(t, w0, ws0, None, 0.05, 128, [1, 1], [1, 1, 1, 1])
    t = m.qlinearconv(t, w, ws, b, 0.05, 128, [1, 1], [1, 1, 1, 1])
    if act:
        t = m.qlinear_act(t, act, 0.1, 0.04, 30)
    t = m.maxpool(t, [2, 2], [2, 2])
    t = m.qlinearconv(t, np.ones((16, K, 1, 1), np.int8), np.full(16, 0.01, np.float32), None, 0.5, 0, [1, 1], [0, 0, 0, 0])
    m.finalize()
    m.profile()
    assert any(k.startswith("qconv_ps_kernel<") and ",6," in k for k in m.launch_kernels()), m.launch_kernels()
    pick = list(range(N)) if N <= 8 else [0, 1, N // 2, N - 1]
    r = zo.qlinearconv(x0[pick], 0.02, 128, w0, ws0, None, 0.05, 128, None, [1, 1], [1, 1, 1, 1], [1, 1], 1)
    kw = dict(act=act, act_alpha=0.1, act_scale=0.04, act_zp=30) if act else {}
    r = zo.qlinearconv(r, 0.05, 128, w, ws, None, 0.05, 128, b, [1, 1], [1, 1, 1, 1], [1, 1], 1, **kw)
    r = zo.onnx_maxpool(r, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
    s_in, zp_in = (0.04, 30) if act else (0.05, 128)
    r = zo.qlinearconv(r, s_in, zp_in, np.ones((16, K, 1, 1), np.int8), np.full(16, 0.01, np.float32), None, 0.5, 0, None,
                       [1, 1], [0, 0, 0, 0], [1, 1], 1)
    np.testing.assert_array_equal(m.predict_host(x0)[pick], r)
    m.close()
