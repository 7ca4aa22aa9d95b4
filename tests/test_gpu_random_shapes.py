"""Seeded random shapes through the C ABI against the oracle: tilings, tails and borders nobody picked by hand.

Integer paths are compared bit for bit, the f32 Gemm within the tolerance the operator states (rtol 1e-4, atol 1e-5
against the oracle's k-ascending f32 sums).
"""
import numpy as np
import pytest

from oracle import oracle as zo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def _qconv_case(G, g, N, C, H, W, K, stride, pad, group, act):
    x = g.integers(0, 256, (N, C, H, W), dtype=np.uint8)
    w = g.integers(-127, 128, (K, C // group, 3, 3), dtype=np.int8)
    ws = (g.uniform(0.5, 1.5, K) * 0.08 / np.sqrt((C // group) * 9)).astype(np.float32)
    b = g.integers(-1000, 1001, K, dtype=np.int32)
    kw = dict(act=act, act_alpha=0.1, act_scale=0.04, act_zp=30) if act else {}
    p = [pad] * 4
    ref = zo.qlinearconv(x, 0.02, 128, w, ws, None, 0.05, 128, b, [stride, stride], p, [1, 1], group, **kw)
    y = G.tm.qlinearconv(G.dev(x), 0.02, 128, G.dev(w), G.dev(ws), None, 0.05, 128, G.dev(b), [stride, stride], p, [1, 1],
                         group, **kw)
    np.testing.assert_array_equal(G.host(y), ref, err_msg=f"N{N} C{C} {H}x{W} K{K} s{stride} p{pad} g{group} {act}")


def test_dense_3x3_layers_of_many_channels(G):
    """32 channels and up in, 33 and up out: the patch-stationary kernel, NCHW output (dword and byte epilogues)."""
    g = np.random.default_rng(101)
    for _ in range(16):
        N, C, K = int(g.integers(1, 5)), int(g.integers(32, 70)), int(g.integers(33, 140))
        H, W, pad = int(g.integers(3, 20)), int(g.integers(3, 24)), int(g.integers(0, 2))
        _qconv_case(G, g, N, C, H, W, K, 1, pad, 1, [None, "leaky", "relu6"][int(g.integers(0, 3))])


def test_first_layers_and_depthwise_layers(G):
    """1 to 4 input channels (first-layer kernel) and depthwise layers, strides 1 and 2, with and without padding."""
    g = np.random.default_rng(102)
    done = 0
    while done < 30:
        first = done % 2 == 0
        N, H, W = int(g.integers(1, 40)), int(g.integers(4, 30)), int(g.integers(4, 30))
        s, pad = int(g.integers(1, 3)), int(g.integers(0, 2))
        if first:
            C, K, group = int(g.integers(1, 5)), int(g.integers(3, 40)), 1
        else:
            C = K = group = int(g.integers(1, 5)) * 16 + int(g.integers(0, 2)) * 8
        if (H + 2 * pad - 3) // s + 1 < 1 or (W + 2 * pad - 3) // s + 1 < 1:
            continue
        _qconv_case(G, g, N, C, H, W, K, s, pad, group, [None, "leaky", "relu6"][int(g.integers(0, 3))])
        done += 1


def test_gemm_with_a_column_count_that_is_a_multiple_of_four(G):
    """All four transpositions; B stored [K][N] takes the 16-byte column copies, the others the k-contiguous ones."""
    import torch
    g = np.random.default_rng(103)
    for _ in range(24):
        M, K, N = int(g.integers(1, 400)), int(g.integers(1, 300)), int(g.integers(9, 60)) * 4
        ta, tb = int(g.integers(0, 2)), int(g.integers(0, 2))
        a = g.standard_normal((1, 1, K, M) if ta else (1, 1, M, K), dtype=np.float32)
        b = (g.standard_normal((1, 1, N, K) if tb else (1, 1, K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
        c = (g.standard_normal((1, 1, 1, N)) * 0.1).astype(np.float32)
        ref = zo.gemm(a, b, c, 1.0, 1.0, ta, tb)
        y = torch.full(ref.shape, -7.0, device="cuda:0")
        G.tm.gemm_lean(G.dev(a), G.dev(b), G.dev(c), 1.0, 1.0, ta, tb, y)
        np.testing.assert_allclose(G.host(y), ref, rtol=G.RTOL, atol=G.ATOL, err_msg=f"M{M} K{K} N{N} ta{ta} tb{tb}")
