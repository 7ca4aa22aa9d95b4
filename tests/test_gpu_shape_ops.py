"""Sigmoid, ReduceMean, Concat and Resize(nearest) on the GPU against the oracle: the reference's known answers, seeded
random cases of every kernel variant, error codes, and large-size properties."""
import numpy as np
import pytest
import torch

from conftest import cases_for
from oracle import oracle as zo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def G():
    import gpu_util
    return gpu_util


def T(d, dtype=np.float32):
    return np.array(d["data"], dtype=dtype).reshape(d["shape"])


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("c", cases_for("sigmoid"))
def test_sigmoid_known_answers(G, c):
    y = G.tm.sigmoid(dev(T(c["x"]))).cpu().numpy()
    assert np.all(np.abs(y - T(c["expect"])) < c["atol"])


@pytest.mark.parametrize("n", [1, 3, 1024, 4099, 1 << 20])
def test_sigmoid_matches_oracle(G, n):
    x = (np.random.default_rng(n).standard_normal(n) * 6).astype(np.float32)
    x[:1] = -200.0
    y = G.tm.sigmoid(dev(x)).cpu().numpy()
    np.testing.assert_allclose(y, zo.sigmoid(x), rtol=1e-4, atol=1e-5)  # the f32 tolerance of the whole path
    xd = dev(np.concatenate([x, x]))[1:n + 1]  # a base that is not 16-byte aligned
    np.testing.assert_allclose(G.tm.sigmoid(xd).cpu().numpy(), zo.sigmoid(xd.cpu().numpy()), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("c", cases_for("reduce_mean"))
def test_reduce_mean_known_answers(G, c):
    y = G.tm.reduce_mean(dev(T(c["x"])), c["axes"], c["keepdims"], c["noop"]).cpu().numpy()
    if "expect" in c:
        assert list(y.shape) == c["expect"]["shape"]
        assert np.all(np.abs(y - T(c["expect"])) <= c["atol"])
    else:
        assert list(y.shape) == c["expect_shape"]
        assert np.all(np.abs(y.ravel()[:3] - np.array(c["expect_first"], np.float32)) <= c["atol"])


@pytest.mark.parametrize("shape,axes,keep", [
    ((4, 6, 7, 9), [2, 3], True),         # global average pool, short odd runs
    ((3, 5, 16, 16), [2, 3], False),      # 256-element runs: 16-byte loads
    ((2, 3, 56, 56), [-1, -2], True),     # 3136-element runs
    ((5, 1280, 3, 3), [2, 3], True),      # the MobileNet pooling shape
    ((3, 4, 5), [1], True),               # kept innermost axis
    ((3, 4, 5), [0, 2], False),           # reduced - kept - reduced
    ((2, 3, 4, 5), [3, 0], True),
    ((2, 3, 4, 5), [1, 3], False),
    ((7, 33), [0], False),
    ((6,), [0], False),
    ((1, 8, 1, 4), [2], True),            # reducing an axis of extent one: a copy
    ((3, 1 << 17), [1], False),           # long runs, few results: segmented
    ((1 << 18,), None, False),            # everything, one result
    ((2, 3, 4), None, True),
])
def test_reduce_mean_matches_oracle(G, shape, axes, keep):
    x = np.random.default_rng(len(shape)).standard_normal(shape).astype(np.float32) + 0.5
    y = G.tm.reduce_mean(dev(x), axes, keep, False).cpu().numpy()
    ref = zo.reduce_mean(x, axes, keep, False)
    assert y.shape == ref.shape
    np.testing.assert_allclose(y, ref, rtol=1e-4, atol=1e-5)


def test_reduce_mean_noop_and_errors(G):
    x = np.random.default_rng(0).standard_normal((3, 4)).astype(np.float32)
    np.testing.assert_array_equal(G.tm.reduce_mean(dev(x), None, True, True).cpu().numpy(), x)
    np.testing.assert_array_equal(G.tm.reduce_mean(dev(x), [], False, True).cpu().numpy(), x)
    for axes in ([2], [-3], [1, 1]):
        with pytest.raises(G.tm.ZantError) as e:
            G.tm.reduce_mean(dev(x), axes, True, False)
        assert e.value.name == "InvalidAxes"


def test_reduce_mean_at_full_size_is_linear_and_exact_on_constants(G):
    x = torch.randn(256, 64, 56, 56, device="cuda")
    m = G.tm.reduce_mean(x, [2, 3], True, False)
    assert m.shape == (256, 64, 1, 1)
    torch.testing.assert_close(m, x.double().mean(dim=(2, 3), keepdim=True).float(), rtol=1e-4, atol=1e-5)
    c = torch.full((64, 32, 28, 28), 3.25, device="cuda")
    assert torch.all(G.tm.reduce_mean(c, [2, 3], False, False) == 3.25)  # sums of 784 x 3.25 are exact in f32


@pytest.mark.parametrize("c", cases_for("concatenate"))
def test_concatenate_known_answers(G, c):
    ts = [dev(T(t)) for t in c["tensors"]]
    if "error" in c:
        with pytest.raises(G.tm.ZantError) as e:
            G.tm.concatenate(ts, c["axis"])
        assert e.value.name == c["error"]
        return
    y = G.tm.concatenate(ts, c["axis"]).cpu().numpy()
    if "expect" in c:
        np.testing.assert_array_equal(y, T(c["expect"]))
    else:
        assert list(y.shape) == c["expect_shape"]


@pytest.mark.parametrize("c", cases_for("concatenate_shape"))
def test_concatenate_shape_known_answers(G, c):
    if "error" in c:
        with pytest.raises(G.tm.ZantError) as e:
            G.tm.get_concatenate_output_shape(c["shapes"], c["axis"])
        assert e.value.name == c["error"]
    else:
        assert list(G.tm.get_concatenate_output_shape(c["shapes"], c["axis"])) == c["expect_shape"]


@pytest.mark.parametrize("shapes,axis,dtype", [
    ([(2, 8, 6, 6), (2, 4, 6, 6)], 1, np.float32),            # channel concat, 16-byte units
    ([(2, 3, 5, 5), (2, 2, 5, 5), (2, 1, 5, 5)], 1, np.float32),  # odd chunk sizes: 4-byte units
    ([(2, 3, 5, 5), (2, 2, 5, 5)], 1, np.uint8),              # byte units
    ([(3, 4), (5, 4)], 0, np.float32),                        # one slice: plain copies
    ([(2, 3, 4, 5), (2, 3, 4, 2)], -1, np.float32),           # innermost axis
    ([(2, 3, 4, 16), (2, 3, 4, 32)], 3, np.uint8),
    ([(1, 2, 3), (3,)], 1, np.float32),                       # rank padding with leading ones
    ([(4, 6), (4, 2)], 1, np.float64),
    ([(4, 6), (4, 0), (4, 2)], 1, np.float32),                # an empty input
])
def test_concatenate_matches_oracle(G, shapes, axis, dtype):
    g = np.random.default_rng(7)
    ts = [(g.standard_normal(s) * 40).astype(dtype) for s in shapes]
    y = G.tm.concatenate([dev(t) for t in ts], axis).cpu().numpy()
    np.testing.assert_array_equal(y, zo.concatenate(ts, axis))


def test_concatenate_at_full_size_splits_back(G):
    a = torch.randint(0, 255, (512, 128, 12, 12), dtype=torch.uint8, device="cuda")
    b = torch.randint(0, 255, (512, 256, 12, 12), dtype=torch.uint8, device="cuda")
    y = G.tm.concatenate([a, b], 1)
    assert y.shape == (512, 384, 12, 12) and torch.equal(y[:, :128], a) and torch.equal(y[:, 128:], b)


@pytest.mark.parametrize("c", cases_for("resize", "resize_shape"))
def test_resize_known_answers(G, c):
    x = T(c["x"], np.uint8) if "x" in c else np.zeros(c["shape"], np.uint8)
    args = (dev(x), c.get("mode", "nearest"), c["scales"], c["sizes"], c.get("coord", "half_pixel"))
    if "error" in c:
        with pytest.raises(G.tm.ZantError) as e:
            G.tm.resize(*args)
        assert e.value.name == c["error"]
        return
    y = G.tm.resize(*args).cpu().numpy()
    assert list(y.shape) == c["expect_shape"]
    if "expect_first" in c:
        assert list(y.ravel()[:len(c["expect_first"])]) == c["expect_first"]


@pytest.mark.parametrize("shape,scales,sizes,dtype", [
    ((2, 3, 6, 6), [1, 1, 2, 2], None, np.float32),
    ((2, 3, 6, 6), [1, 1, 2, 2], None, np.uint8),
    ((1, 2, 5, 7), None, [1, 2, 9, 13], np.float32),
    ((2, 3, 8, 16), [1, 1, 2, 2], None, np.uint8),    # 16 outputs per thread
    ((2, 3, 8, 11), None, [2, 3, 5, 24], np.int16),   # 8 outputs per thread, gather within a row
    ((24,), [2.0], None, np.float32),                  # rank 1 through the vector kernel
    ((1, 2, 9, 13), None, [1, 2, 5, 7], np.uint8),
    ((3, 5), [1.7, 0.6], None, np.float64),
    ((11,), [3.3], None, np.int16),
    ((2, 1, 4, 4), None, [2, 1, 1, 1], np.float32),   # one-element outputs (0 / 0 under align_corners)
    ((2, 2, 3, 3, 3), [1, 1, 2, 2, 2], None, np.float32),
    ((3000, 2, 8), None, [3000, 3, 16], np.float32),  # the outermost axis' table is too long for LDS: looked up in global memory
    ((2, 1100), None, [3, 4400], np.float32),          # even the innermost one is
    ((2100, 4), None, [2100, 8], np.uint8),
])
@pytest.mark.parametrize("coord", ["half_pixel", "align_corners", "asymmetric"])
def test_resize_matches_oracle(G, shape, scales, sizes, dtype, coord):
    x = (np.random.default_rng(9).standard_normal(shape) * 50).astype(dtype)
    y = G.tm.resize(dev(x), "nearest", scales, sizes, coord).cpu().numpy()
    np.testing.assert_array_equal(y, zo.resize(x, "nearest", scales, sizes, coord))


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.float32, np.float64])
@pytest.mark.parametrize("shape,sizes", [
    ((3, 5, 7, 16), [3, 5, 14, 32]),    # rows and columns doubled
    ((2, 3, 5, 32), [2, 3, 15, 64]),    # rows tripled
    ((2, 3, 5, 32), [2, 3, 5, 64]),     # rows kept
    ((9, 48), [36, 96]),                # rank 2, rows x4
    ((2, 3, 5, 32), [4, 3, 10, 64]),    # a leading axis resized too
    ((1, 1300, 2, 16), [1, 1300, 4, 32]),  # more rows than one workgroup covers
])
@pytest.mark.parametrize("coord", ["half_pixel", "align_corners", "asymmetric"])
def test_resize_integer_upsampling_matches_oracle(G, shape, sizes, dtype, coord):
    # under half_pixel an integer factor repeats elements; asymmetric and align_corners round differently at the same sizes
    x = (np.random.default_rng(11).standard_normal(shape) * 90).astype(dtype)
    y = G.tm.resize(dev(x), "nearest", None, sizes, coord).cpu().numpy()
    np.testing.assert_array_equal(y, zo.resize(x, "nearest", None, sizes, coord))
    if coord == "half_pixel" and tuple(sizes[:-2]) == shape[:-2]:
        np.testing.assert_array_equal(y, x.repeat(sizes[-2] // shape[-2], axis=-2).repeat(2, axis=-1))


@pytest.mark.parametrize("shape", [(512, 128, 6, 6), (256, 64, 28, 32)])
def test_resize_at_full_size_repeats_elements(G, shape):
    x = torch.randint(0, 255, shape, dtype=torch.uint8, device="cuda")
    y = G.tm.resize(x, "nearest", [1.0, 1.0, 2.0, 2.0], None, "half_pixel")
    assert torch.equal(y, x.repeat_interleave(2, dim=2).repeat_interleave(2, dim=3))
