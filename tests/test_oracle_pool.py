"""Pins the pooling oracle: bit-for-bit against the compiled reference objects (oracle/_ref), against
committed golden vectors (which came from those objects), against torch's pooling autograd where the
result is unique, and against brute force on tiny inputs.

Cases follow matlab/xtest/suite/nnpool.m:34-112 (pool sizes, pads, strides, rectangular windows,
asymmetric pads) plus what that suite never exercises: ties, NaN, -inf."""
import itertools
import os

import numpy as np
import pytest
import torch

from util import F, bits_equal, rel_max

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "pool_golden.npz")

# (H, W, C, N, pool, stride, pad)
GEOMS = [
    (5, 6, 2, 3, 2, 1, 0), (5, 6, 2, 3, 3, 2, 1), (8, 8, 1, 2, 3, 3, 2), (7, 9, 3, 1, (2, 3), (1, 2), (1, 0, 2, 1)),
    (9, 7, 2, 2, (3, 2), (2, 1), (0, 1, 1, 0)), (4, 4, 1, 1, 4, 4, 3), (6, 6, 2, 2, 2, 2, (0, 1, 0, 1)),
    (12, 12, 2, 2, 3, 2, 1), (5, 5, 1, 1, 1, 1, 0), (10, 3, 1, 2, (5, 3), (3, 1), (2, 2, 1, 1)),
]


def _inputs(shape, seed, mode):
    r = np.random.default_rng(seed)
    n = int(np.prod(shape))
    if mode == "distinct":  # random permutation: every max is unique (nnpool.m:22-31)
        x = r.permutation(n).astype(np.float32).reshape(shape)
    elif mode == "ties":
        x = r.integers(0, 3, size=shape).astype(np.float32)
    elif mode == "special":
        x = r.integers(0, 3, size=shape).astype(np.float32)
        flat = x.reshape(-1)
        flat[r.random(n) < 0.25] = np.nan
        flat[r.random(n) < 0.25] = -np.inf
        flat[r.random(n) < 0.05] = np.inf
    else:
        x = r.standard_normal(shape).astype(np.float32)
    return F(x)


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("method", ["max", "avg"])
@pytest.mark.parametrize("mode", ["distinct", "ties", "special", "normal"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_oracle_equals_reference_bitwise(ref, geom, method, mode, dtype):
    H, W, C, N, pool, stride, pad = geom
    g = ref.pool_geom((H, W, C, N), pool, stride, pad, method)
    x = F(_inputs((H, W, C, N), 11, mode), dtype)
    dy = F(np.random.default_rng(12).standard_normal(ref.pool_out_shape(g)), dtype)
    assert bits_equal(ref.pool_forward(x, g), ref.ref_pool_forward(x, g))
    assert bits_equal(ref.pool_backward(x, dy, g), ref.ref_pool_backward(x, dy, g))


def test_oracle_equals_reference_overlapping_large(ref):
    # overlapping, clipped windows on a plane big enough to have interior + all four borders
    for method in ("max", "avg"):
        g = ref.pool_geom((37, 29, 3, 2), 3, 2, 1, method)
        x = _inputs((37, 29, 3, 2), 5, "ties")
        dy = F(np.random.default_rng(6).standard_normal(ref.pool_out_shape(g)))
        assert bits_equal(ref.pool_backward(x, dy, g), ref.ref_pool_backward(x, dy, g))


@pytest.mark.parametrize("geom", GEOMS)
def test_max_backward_vs_torch_autograd_on_distinct_input(ob, geom):
    """With all-distinct inputs the routing is unique, so torch's max_pool2d gradient must agree
    (symmetric pads only: torch has no asymmetric padding)."""
    H, W, C, N, pool, stride, pad = geom
    pad4 = ob._quad(pad)
    ph, pw = ob._pair(pool)
    if pad4[0] != pad4[1] or pad4[2] != pad4[3] or pad4[0] > ph // 2 or pad4[2] > pw // 2:
        pytest.skip("torch max_pool2d needs symmetric pad <= pool/2")
    g = ob.pool_geom((H, W, C, N), pool, stride, pad, "max")
    x = F(_inputs((H, W, C, N), 3, "distinct"), np.float64)
    dy = F(np.random.default_rng(4).standard_normal(ob.pool_out_shape(g)), np.float64)
    xt = torch.from_numpy(np.ascontiguousarray(x.T)).requires_grad_(True)  # (N,C,W,H)
    sy, sx = ob._pair(stride)
    yt = torch.nn.functional.max_pool2d(xt, (pw, ph), (sx, sy), (pad4[2], pad4[0]))
    yt.backward(torch.from_numpy(np.ascontiguousarray(dy.T)))
    assert np.array_equal(ob.pool_forward(x, g), yt.detach().numpy().T)
    assert rel_max(ob.pool_backward(x, dy, g), xt.grad.numpy().T) < 1e-14


@pytest.mark.parametrize("geom", GEOMS)
def test_avg_backward_vs_torch_autograd(ob, geom):
    """avg pooling excludes padding from the count = torch's count_include_pad=False."""
    H, W, C, N, pool, stride, pad = geom
    pad4 = ob._quad(pad)
    ph, pw = ob._pair(pool)
    if pad4[0] != pad4[1] or pad4[2] != pad4[3] or pad4[0] > ph // 2 or pad4[2] > pw // 2:
        pytest.skip("torch avg_pool2d needs symmetric pad <= pool/2")
    g = ob.pool_geom((H, W, C, N), pool, stride, pad, "avg")
    x = F(_inputs((H, W, C, N), 3, "normal"), np.float64)
    dy = F(np.random.default_rng(4).standard_normal(ob.pool_out_shape(g)), np.float64)
    xt = torch.from_numpy(np.ascontiguousarray(x.T)).requires_grad_(True)
    sy, sx = ob._pair(stride)
    yt = torch.nn.functional.avg_pool2d(xt, (pw, ph), (sx, sy), (pad4[2], pad4[0]), count_include_pad=False)
    yt.backward(torch.from_numpy(np.ascontiguousarray(dy.T)))
    assert rel_max(ob.pool_forward(x, g), yt.detach().numpy().T) < 1e-13
    assert rel_max(ob.pool_backward(x, dy, g), xt.grad.numpy().T) < 1e-13


def _brute_max_backward(x, dy, H, W, ph, pw, sy, sx, pt, pl, oh_n, ow_n):
    """Independent statement of the routing rule for one plane: first maximum in memory (column-major)
    order, NaN never wins, -inf never beats the start value."""
    dx = np.zeros((H, W), x.dtype)
    for ow in range(ow_n):
        for oh in range(oh_n):
            cells = [(h, w) for w in range(max(ow * sx - pl, 0), min(ow * sx - pl + pw, W))
                     for h in range(max(oh * sy - pt, 0), min(oh * sy - pt + ph, H))]
            vals = [x[h, w] for h, w in cells]
            finite_or_inf = [v for v in vals if not np.isnan(v) and v > -np.inf]
            if not finite_or_inf:
                continue
            m = max(finite_or_inf)
            h, w = cells[vals.index(m)]
            dx[h, w] = dx[h, w] + dy[oh, ow]
    return dx


@pytest.mark.parametrize("mode", ["ties", "special"])
def test_max_backward_brute_force_tiny(ob, mode):
    H, W = 7, 6
    g = ob.pool_geom((H, W, 1, 1), 3, 2, 1, "max")
    x = _inputs((H, W, 1, 1), 21, mode)
    oshape = ob.pool_out_shape(g)
    dy = F(np.random.default_rng(22).standard_normal(oshape))
    want = _brute_max_backward(x[:, :, 0, 0], dy[:, :, 0, 0], H, W, 3, 3, 2, 2, 1, 1, oshape[0], oshape[1])
    assert bits_equal(ob.pool_backward(x, dy, g)[:, :, 0, 0].copy(), want)


def test_ties_go_to_the_first_maximum_in_memory_order(ob):
    # 2x2 stride-2 max pooling of columns [1 1 1 1],[2 2 2 2],[3 3 3 3],[4 4 4 4]: winners at offsets 4,6,12,14
    x = F(np.tile(np.array([1, 2, 3, 4], np.float32), (4, 1)).reshape(4, 4, 1, 1))
    g = ob.pool_geom(x.shape, 2, 2, 0, "max")
    dy = F(np.array([10, 20, 30, 40], np.float32).reshape(2, 2, 1, 1, order="F"))
    dx = ob.pool_backward(x, dy, g).ravel(order="F")
    assert list(np.nonzero(dx)[0]) == [4, 6, 12, 14]
    assert list(dx[[4, 6, 12, 14]]) == [10, 20, 30, 40]


def test_backward_accumulates_into_existing(ob):
    g = ob.pool_geom((6, 6, 1, 1), 2, 2, 0, "avg")
    x = _inputs((6, 6, 1, 1), 1, "normal")
    dy = F(np.random.default_rng(2).standard_normal(ob.pool_out_shape(g)))
    base = F(np.random.default_rng(3).standard_normal((6, 6, 1, 1)))
    got = ob.pool_backward(x, dy, g, dx=base.copy(order="F"))
    assert rel_max(got, base + ob.pool_backward(x, dy, g)) < 1e-6


def test_oracle_matches_golden_vectors(ob):
    """Golden vectors written from the compiled reference (tests/golden/make_golden.py)."""
    z = np.load(GOLDEN)
    for i in range(int(z["count"])):
        geom = [int(v) for v in z["geom_%d" % i]]
        H, W, C, N, ph, pw, sy, sx, pt, pb, pl, pr, method = geom
        g = ob.pool_geom((H, W, C, N), (ph, pw), (sy, sx), (pt, pb, pl, pr), "max" if method == 0 else "avg")
        x, dy = F(z["x_%d" % i]), F(z["dy_%d" % i])
        assert bits_equal(ob.pool_forward(x, g), F(z["y_%d" % i])), i
        assert bits_equal(ob.pool_backward(x, dy, g), F(z["dx_%d" % i])), i
