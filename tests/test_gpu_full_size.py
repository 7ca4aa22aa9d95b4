"""Parity at the benchmark's full sizes (configs 1, 2a, 2b, 3), where the oracle cannot run the whole input in a test:
sampled slices against the oracle, plus properties that hold whatever the size -- a permuted batch permutes the output
(bit for bit: every image takes the same arithmetic path wherever it sits), and the Gemm is linear in B."""
import numpy as np
import pytest
import torch

from oracle import oracle as zo
from test_gpu_model import oracle_readme_cnn, readme_cnn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def test_config1_readme_cnn_batch_4096(G):
    """1600 window-packed tiles over 512 persistent workgroups (three rounds and a last one dealt out by workgroup number),
    256 Gemm tiles: the tilings only the full batch exercises."""
    from zant_amd import networks
    B = 4096
    params = networks.readme_cnn_params(seed=0)
    m = readme_cnn(G, B, params)
    g = np.random.default_rng(11)
    x = g.random((B, 1, 28, 28), dtype=np.float32)
    y = m.predict_host(x)
    assert y.shape == (B, 10) and np.isfinite(y).all()
    np.testing.assert_allclose(y.sum(axis=1), 1.0, rtol=0, atol=1e-5)  # every row is a softmax
    # sampled images against the oracle: both ends, tile boundaries of the convolutions (4 images per workgroup; 64
    # pooling windows per tile of the second one, so images 2, 5, 7 ... straddle two tiles), images of the last round's
    # tiles (every eighth run of 200 tiles ends with eight of them: images 491-511, 1003-1023, ... 4075-4095), of the Gemm
    # (128 rows per tile) and of the classifier head (16 rows per workgroup), and a random draw
    pick = sorted(set([0, 1, 2, 3, 4, 5, 7, 15, 16, 127, 128, 491, 500, 511, 1010, 2047, 2048, 3580, 4079, 4080, 4090, 4094, 4095] +
                      g.integers(0, B, 24).tolist()))
    ref = np.concatenate([oracle_readme_cnn(x[i:i + 1], params) for i in pick])
    np.testing.assert_allclose(y[pick], ref, rtol=G.RTOL, atol=G.ATOL)
    # batch-permutation equivariance over the whole batch, bit for bit
    perm = g.permutation(B)
    yp = m.predict_host(x[perm])
    assert np.array_equal(yp, y[perm])
    m.close()


def test_config2a_conv_256x64x56x56(G):
    N, C, H, K = 256, 64, 56, 64
    torch.manual_seed(2)
    x = torch.randn(N, C, H, H, device="cuda:0")
    w = torch.randn(K, C, 3, 3, device="cuda:0") * (2.0 / (C * 9)) ** 0.5
    b = torch.randn(K, device="cuda:0") * 0.1
    y = torch.zeros(N, K, H, H, device="cuda:0")
    G.tm.conv_lean(x, w, y, b, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
    yh = G.host(y)
    pick = [0, 101, 255]
    ref = zo.Conv(G.host(x[pick]), G.host(w), G.host(b), [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
    np.testing.assert_allclose(yh[pick], ref, rtol=G.RTOL, atol=G.ATOL)
    perm = torch.randperm(N, device="cuda:0")
    yp = torch.zeros_like(y)
    G.tm.conv_lean(x[perm].contiguous(), w, yp, b, [1, 1], [1, 1, 1, 1], [1, 1], 1, "NOTSET")
    assert torch.equal(yp, y[perm])


def test_config2b_gemm_4096x1600x512(G):
    M, Kd, N = 4096, 1600, 512
    torch.manual_seed(3)
    a = torch.randn(1, 1, M, Kd, device="cuda:0")
    b1 = torch.randn(1, 1, Kd, N, device="cuda:0") * (2.0 / Kd) ** 0.5
    b2 = torch.randn(1, 1, Kd, N, device="cuda:0") * (2.0 / Kd) ** 0.5
    c = torch.randn(1, 1, 1, N, device="cuda:0") * 0.1
    y1 = torch.zeros(1, 1, M, N, device="cuda:0")
    G.tm.gemm_lean(a, b1, c, 1.0, 1.0, False, False, y1)
    # row blocks against the oracle: the first and last tile of 128 rows and two from the middle
    rows = np.r_[0:128, 1984:2112, 3968:4096]
    ref = zo.gemm(G.host(a[:, :, rows]), G.host(b1), G.host(c), 1.0, 1.0, False, False)
    np.testing.assert_allclose(G.host(y1)[:, :, rows], ref, rtol=G.RTOL, atol=G.ATOL)
    # row-permutation equivariance, bit for bit
    perm = torch.randperm(M, device="cuda:0")
    yp = torch.zeros_like(y1)
    G.tm.gemm_lean(a[:, :, perm].contiguous(), b1, c, 1.0, 1.0, False, False, yp)
    assert torch.equal(yp, y1[:, :, perm])
    # linearity in B (no C, so both sides are pure products): A(B1 + B2) = A B1 + A B2 within f32 rounding of a
    # 1600-term sum of O(1) products
    y2 = torch.zeros_like(y1)
    y12 = torch.zeros_like(y1)
    y1n = torch.zeros_like(y1)
    G.tm.gemm_lean(a, b1, None, 1.0, 1.0, False, False, y1n)
    G.tm.gemm_lean(a, b2, None, 1.0, 1.0, False, False, y2)
    G.tm.gemm_lean(a, b1 + b2, None, 1.0, 1.0, False, False, y12)
    np.testing.assert_allclose(G.host(y12), G.host(y1n + y2), rtol=1e-4, atol=2e-5)
    # and alpha scales the product exactly when it is a power of two
    y4 = torch.zeros_like(y1)
    G.tm.gemm_lean(a, b1, None, 4.0, 1.0, False, False, y4)
    assert torch.equal(y4, 4.0 * y1n)


def test_config3_qlinearconv_128x128x28x28(G):
    N, C, H, K = 128, 128, 28, 128
    g = np.random.default_rng(5)
    x = g.integers(0, 256, (N, C, H, H), dtype=np.uint8)
    w = g.integers(-127, 128, (K, C, 3, 3), dtype=np.int8)
    ws = g.uniform(0.001, 0.01, K).astype(np.float32)
    bias = g.integers(-1000, 1001, K, dtype=np.int32)
    xd, wd, wsd, bd = G.dev(x), G.dev(w), G.dev(ws), G.dev(bias)
    y = torch.zeros(N, K, H, H, dtype=torch.uint8, device="cuda:0")
    run = lambda xin, out: G.tm.qlinearconv_lean(xin, 0.02, 128, wd, wsd, None, 0.05, 128, bd, out, [1, 1], [1, 1, 1, 1], [1, 1])
    run(xd, y)
    yh = G.host(y)
    assert 0.02 < (yh == 0).mean() + (yh == 255).mean() < 0.9  # the scales put some, not all, outputs at the rails
    pick = [0, 63, 127]
    ref = zo.qlinearconv(x[pick], 0.02, 128, w, ws, None, 0.05, 128, bias, [1, 1], [1, 1, 1, 1], [1, 1])
    assert np.array_equal(yh[pick], ref)
    perm = torch.randperm(N, device="cuda:0")
    yp = torch.zeros_like(y)
    run(xd[perm].contiguous(), yp)
    assert torch.equal(yp, y[perm])
