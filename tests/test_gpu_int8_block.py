"""The fused inverted residual block (1x1 expansion -> depthwise 3x3 -> 1x1 projection [-> quantised add]) against the
oracle's layer-by-layer result, bit for bit, over the shapes that select each variant of the kernel: many and few
position tiles per workgroup tile (the latter deal (position tile, channel chunk) units to the waves and add their
partial sums up in LDS), one to four blocks of 32 output channels, stride 1 and 2, with and without the residual, a last
channel chunk that is half padding, and batches that leave a partial last tile."""
import numpy as np
import pytest

from oracle import oracle as zo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


#        N, Cin, H,  Ce,  Co, stride, residual
CASES = [(8, 8, 48, 48, 8, 1, True),       # large map: three position tiles per wave
         (5, 8, 24, 48, 8, 2, False),      # stride 2
         (32, 8, 12, 48, 8, 1, True),
         (64, 32, 6, 192, 32, 1, True),    # one position tile per workgroup tile: units dealt to the waves
         (70, 24, 6, 144, 24, 1, True),    # 144 = 4 x 32 + 16: the last chunk is half padding
         (64, 32, 6, 192, 56, 2, False),   # two blocks of output channels
         (64, 56, 3, 336, 56, 1, True),
         (33, 56, 3, 336, 112, 1, False),  # four blocks of output channels
         (1024, 56, 3, 336, 56, 1, True),  # the benchmark's batch: several images per tile, two position tiles
         (1024, 32, 6, 192, 32, 1, True)]


@pytest.mark.parametrize("N,Cin,H,Ce,Co,stride,res", CASES)
def test_block_matches_the_layers_bit_for_bit(G, N, Cin, H, Ce, Co, stride, res):
    from zant_amd.model import Model, U8
    g = np.random.default_rng(N + Cin + H + Ce + Co)
    m = Model(G.tm.context())
    t = m.input((N, Cin, H, H), U8, 0.02, 128)
    layers = []

    def conv(t, cin, cout, k, s, grp, act):
        w = g.integers(-127, 128, (cout, cin // grp, k, k), dtype=np.int8)
        ws = g.uniform(0.001, 0.004, cout).astype(np.float32)
        b = g.integers(-100, 100, cout, dtype=np.int32)
        layers.append((w, ws, b, s, k // 2, grp, act))
        t = m.qlinearconv(t, w, ws, b, 0.05, 128, [s, s], [k // 2] * 4, [1, 1], grp)
        return m.qlinear_act(t, "relu6", 0.0, 0.03, 0) if act else t

    t = conv(t, Cin, Cin, 1, 1, 1, False)   # keeps the block's input a blocked tensor inside the model
    block_in = t
    t = conv(t, Cin, Ce, 1, 1, 1, True)
    t = conv(t, Ce, Ce, 3, stride, Ce, True)
    t = conv(t, Ce, Co, 1, 1, 1, False)
    if res:
        t = m.qlinear_add(t, block_in, 0.07, 100)
    conv(t, Co, Co, 1, 1, 1, False)
    m.finalize()
    assert m.num_launches == 3 and "InvertedResidual" in m.profile()[1][0]
    x = g.integers(0, 256, (N, Cin, H, H), dtype=np.uint8)
    y = m.predict_host(x)
    m.close()

    sample = np.unique(np.r_[0:min(N, 6), max(N - 6, 0):N])  # the oracle on both ends of the batch (every image alone)
    v, sc, zp = x[sample], 0.02, 128
    outs = []
    for i, (w, ws, b, s, p, grp, act) in enumerate(layers):
        if i == 4 and res:
            v, sc, zp = zo.qlinear_add(v, sc, zp, outs[0][0], outs[0][1], outs[0][2], 0.07, 100), 0.07, 100
        v, sc, zp = zo.qlinearconv(v, sc, zp, w, ws, None, 0.05, 128, b, [s, s], [p] * 4, [1, 1], grp), 0.05, 128
        if act:
            v, sc, zp = zo.qlinear_act(v, sc, zp, "relu6", 0.0, 0.03, 0), 0.03, 0
        outs.append((v, sc, zp))
    np.testing.assert_array_equal(y[sample], v)


#             N,  H, blocks: (Cin, Ce, Co, stride, residual)
CHAIN_CASES = [(300, 12, [(16, 96, 16, 1, True), (16, 96, 24, 2, False), (24, 144, 24, 1, True), (24, 144, 32, 1, False)]),
               (7, 6, [(32, 192, 56, 2, False), (56, 336, 56, 1, True), (56, 336, 56, 1, True)]),  # two blocks of output channels
               (130, 6, [(24, 144, 24, 1, True), (24, 144, 24, 1, True)])]


@pytest.mark.parametrize("N,H,blocks", CHAIN_CASES, ids=["12to6", "6to3", "two"])
def test_blocks_in_a_row_run_as_one_launch_bit_for_bit(G, N, H, blocks):
    """Consecutive blocks on tiles of whole images become one launch (a workgroup stays on its images through all of
    them).  Their tensors differ in shape, so storage reused between them would let a fast workgroup overwrite what a
    slow one still reads: the result must match the oracle image by image, and every intermediate tensor, read back
    (which replays the blocks one by one), must match too."""
    from zant_amd.model import Model, U8
    g = np.random.default_rng(N + H)
    m = Model(G.tm.context())
    cin0 = blocks[0][0]
    x = g.integers(0, 256, (N, cin0, H, H), dtype=np.uint8)
    sample = np.unique(np.r_[0:min(N, 5), max(N - 5, 0):N])
    ref = [x[sample], 0.02, 128]  # the oracle's tensor, scale, zero point, advanced with every node added to the model

    def conv(t, cin, cout, k, s, grp, act):
        w = g.integers(-127, 128, (cout, cin // grp, k, k), dtype=np.int8)
        ws = g.uniform(0.001, 0.004, cout).astype(np.float32)
        b = g.integers(-100, 100, cout, dtype=np.int32)
        t = m.qlinearconv(t, w, ws, b, 0.05, 128, [s, s], [k // 2] * 4, [1, 1], grp)
        ref[:] = [zo.qlinearconv(ref[0], ref[1], ref[2], w, ws, None, 0.05, 128, b, [s, s], [k // 2] * 4, [1, 1], grp), 0.05, 128]
        if act:
            t = m.qlinear_act(t, "relu6", 0.0, 0.03, 0)
            ref[:] = [zo.qlinear_act(ref[0], ref[1], ref[2], "relu6", 0.0, 0.03, 0), 0.03, 0]
        return t

    t = m.input((N, cin0, H, H), U8, 0.02, 128)
    t = conv(t, cin0, cin0, 1, 1, 1, False)
    ends = []
    for cin, ce, co, s, res in blocks:
        block_in, ref_in = t, list(ref)
        t = conv(t, cin, ce, 1, 1, 1, True)
        t = conv(t, ce, ce, 3, s, ce, True)
        t = conv(t, ce, co, 1, 1, 1, False)
        if res:
            t = m.qlinear_add(t, block_in, 0.07, 100)
            ref[:] = [zo.qlinear_add(ref[0], ref[1], ref[2], ref_in[0], ref_in[1], ref_in[2], 0.07, 100), 0.07, 100]
        ends.append((t, ref[0]))
    conv(t, blocks[-1][2], blocks[-1][2], 1, 1, 1, False)
    m.finalize()
    names = [p[0] for p in m.profile()]
    assert m.num_launches == 3 and names[1] == "InvertedResidualChain", names
    assert m.launch_kernels()[1].startswith("qblock_chain_kernel<"), m.launch_kernels()
    y = m.predict_host(x)
    np.testing.assert_array_equal(y[sample], ref[0])
    for tid, r in ends[:-1]:
        np.testing.assert_array_equal(m.read_tensor(tid, (N,) + r.shape[1:], np.uint8)[sample], r)
    np.testing.assert_array_equal(m.predict_host(x), y)  # the arena is as the pass left it
    m.close()
