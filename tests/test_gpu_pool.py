"""GPU parity, pooling: the HIP kernels (through the C ABI) against the CPU oracle and the golden vectors
from the compiled reference.  Bar: bit-exact, max AND average (tolerance stated by the task for average is
1e-5 relative; the gather order makes it exact, so exactness is what is asserted)."""
import os

import numpy as np
import pytest

from matconvnet_amd import workloads
from util import F, bits_equal, count_bit_mismatches

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "pool_golden.npz")

GEOMS = [
    (5, 6, 2, 3, 2, 1, 0), (5, 6, 2, 3, 3, 2, 1), (8, 8, 1, 2, 3, 3, 2), (7, 9, 3, 1, (2, 3), (1, 2), (1, 0, 2, 1)),
    (9, 7, 2, 2, (3, 2), (2, 1), (0, 1, 1, 0)), (4, 4, 1, 1, 4, 4, 3), (6, 6, 2, 2, 2, 2, (0, 1, 0, 1)),
    (12, 12, 2, 2, 3, 2, 1), (5, 5, 1, 1, 1, 1, 0), (10, 3, 1, 2, (5, 3), (3, 1), (2, 2, 1, 1)),
    (28, 28, 5, 3, 3, 2, 1), (56, 56, 4, 2, 2, 2, 0), (33, 47, 3, 2, (3, 5), (2, 3), (1, 2, 4, 0)),
    (224, 8, 2, 1, 3, 2, 1), (8, 224, 2, 1, 3, 2, 1),
]


def _inputs(shape, seed, mode):
    r = np.random.default_rng(seed)
    n = int(np.prod(shape))
    if mode == "distinct":
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


def _run(capi, ob, x, dy, shape, pool, stride, pad, method, accumulate_into=None):
    g = capi.pool_geom(shape, pool, stride, pad, method)
    og = ob.pool_geom(shape, pool, stride, pad, method)
    xd, dyd = capi.to_device(x), capi.to_device(dy)
    if accumulate_into is None:
        got = capi.to_host(capi.pool_backward(xd, dyd, g))
        want = ob.pool_backward(x, dy, og)
    else:
        got = capi.to_host(capi.pool_backward(xd, dyd, g, dx=capi.to_device(accumulate_into)))
        want = ob.pool_backward(x, dy, og, dx=accumulate_into.copy(order="F"))
    return got, want


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("method", ["max", "avg"])
@pytest.mark.parametrize("mode", ["distinct", "ties", "special", "normal"])
def test_backward_bit_exact_small(capi, ob, geom, method, mode):
    H, W, C, N, pool, stride, pad = geom
    shape = (H, W, C, N)
    og = ob.pool_geom(shape, pool, stride, pad, method)
    x = _inputs(shape, 11, mode)
    dy = F(np.random.default_rng(12).standard_normal(ob.pool_out_shape(og)))
    got, want = _run(capi, ob, x, dy, shape, pool, stride, pad, method)
    assert bits_equal(got, want), count_bit_mismatches(got, want)


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("method", ["max", "avg"])
def test_forward_bit_exact_small(capi, ob, geom, method):
    H, W, C, N, pool, stride, pad = geom
    shape = (H, W, C, N)
    x = _inputs(shape, 5, "special" if method == "max" else "normal")
    g = capi.pool_geom(shape, pool, stride, pad, method)
    got = capi.to_host(capi.pool_forward(capi.to_device(x), g))
    want = ob.pool_forward(x, ob.pool_geom(shape, pool, stride, pad, method))
    assert bits_equal(got, want)


@pytest.mark.parametrize("method", ["max", "avg"])
@pytest.mark.parametrize("geom", [(40, 36, 3, 2, 3, 2, 1), (112, 112, 4, 2, 3, 2, 1), (21, 17, 2, 1, (7, 3), (1, 1), (3, 3, 1, 1)),
                                  (30, 30, 1, 2, 9, 4, 4), (7, 7, 5, 3, 7, 1, 0), (300, 9, 2, 1, (2, 5), (2, 1), 0),
                                  (56, 56, 4, 2, 2, 2, 0), (8, 6, 3, 2, 3, 2, (1, 0, 1, 0)), (4, 2, 2, 1, 3, 2, 1),
                                  (12, 10, 2, 3, 2, 2, (0, 1, 0, 1)), (42, 36, 2, 2, 3, 2, 1), (40, 35, 2, 2, 3, 2, 1)])
def test_forward_bit_exact_larger_planes(capi, ob, method, geom):
    """Forward pass on planes of several hundred elements, wide windows and whole-plane windows, and the
    down-sampling cases that have a kernel of their own (3x3 / 2x2 windows, stride 2, heights that are and are not
    multiples of 4): the oracle's bits (ties, NaN, infinities and zeros of both signs included)."""
    H, W, C, N, pool, stride, pad = geom
    shape = (H, W, C, N)
    x = _inputs(shape, 51, "special" if method == "max" else "normal")
    g = capi.pool_geom(shape, pool, stride, pad, method)
    want = ob.pool_forward(x, ob.pool_geom(shape, pool, stride, pad, method))
    assert bits_equal(capi.to_host(capi.pool_forward(capi.to_device(x), g)), want)


@pytest.mark.parametrize("method", ["max", "avg"])
def test_backward_accumulate_mode(capi, ob, method):
    """accumulate != 0 is the vl::nn::Pooling::backward contract: derInput += ..., same addition order."""
    shape = (12, 12, 2, 2)
    x = _inputs(shape, 3, "ties")
    og = ob.pool_geom(shape, 3, 2, 1, method)
    dy = F(np.random.default_rng(4).standard_normal(ob.pool_out_shape(og)))
    base = F(np.random.default_rng(5).standard_normal(shape))
    got, want = _run(capi, ob, x, dy, shape, 3, 2, 1, method, accumulate_into=base)
    assert bits_equal(got, want)


@pytest.mark.parametrize("budget", [1024, 4096, 65536])
def test_tile_width_does_not_change_results(capi, ob, budget):
    """Different LDS budgets -> different tile widths (and the non-tiled fallback): identical bits."""
    old = capi.get_tunable("pool_lds_bytes")
    try:
        capi.set_tunable("pool_lds_bytes", budget)
        for method in ("max", "avg"):
            shape = (40, 36, 3, 2)
            x = _inputs(shape, 8, "ties")
            og = ob.pool_geom(shape, 3, 2, 1, method)
            dy = F(np.random.default_rng(9).standard_normal(ob.pool_out_shape(og)))
            got, want = _run(capi, ob, x, dy, shape, 3, 2, 1, method)
            assert bits_equal(got, want)
    finally:
        capi.set_tunable("pool_lds_bytes", old)


@pytest.mark.parametrize("method", ["max", "avg"])
@pytest.mark.parametrize("geom", [(20, 18, 2, 2, 3, 2, 1), (16, 16, 3, 1, 2, 2, 0), (15, 13, 2, 2, (3, 2), (1, 2), (1, 0, 0, 1))])
def test_general_gather_kernels_agree(capi, ob, method, geom):
    """The ordered-pass kernel is the default; the general tiled gather / flag kernels behind it give the
    same bits."""
    H, W, C, N, pool, stride, pad = geom
    shape = (H, W, C, N)
    x = _inputs(shape, 31, "ties")
    og = ob.pool_geom(shape, pool, stride, pad, method)
    dy = F(np.random.default_rng(32).standard_normal(ob.pool_out_shape(og)))
    try:
        capi.set_tunable("pool_force_gather", 1)
        got, want = _run(capi, ob, x, dy, shape, pool, stride, pad, method)
        assert bits_equal(got, want)
        base = F(np.random.default_rng(33).standard_normal(shape))
        got, want = _run(capi, ob, x, dy, shape, pool, stride, pad, method, accumulate_into=base)
        assert bits_equal(got, want)
    finally:
        capi.set_tunable("pool_force_gather", 0)


@pytest.mark.parametrize("method", ["max", "avg"])
@pytest.mark.parametrize("geom", [(24, 20, 2, 2, 5, 1, 2), (30, 30, 1, 2, 9, 4, 4), (21, 17, 2, 1, (7, 3), (1, 1), (3, 3, 1, 1)),
                                   (40, 40, 2, 1, 3, 5, 0)])
def test_large_windows_and_sparse_strides(capi, ob, method, geom):
    """Windows covered by many outputs (more than 16 passes), windows larger than 8, and strides larger than
    the window (inputs no output covers) take the general paths."""
    H, W, C, N, pool, stride, pad = geom
    shape = (H, W, C, N)
    x = _inputs(shape, 41, "ties")
    og = ob.pool_geom(shape, pool, stride, pad, method)
    dy = F(np.random.default_rng(42).standard_normal(ob.pool_out_shape(og)))
    got, want = _run(capi, ob, x, dy, shape, pool, stride, pad, method)
    assert bits_equal(got, want), count_bit_mismatches(got, want)


@pytest.mark.parametrize("geom", [(7, 7, 5, 3, 7, 1, 0), (6, 9, 3, 2, (6, 9), (1, 1), 0), (5, 4, 2, 2, (7, 6), (2, 3), (1, 1, 1, 1)),
                                  (4, 4, 2, 2, (5, 5), (1, 1), (0, 1, 0, 1))])
def test_average_over_the_whole_plane(capi, ob, geom):
    """One window covering the plane (the pooling before a classifier) has a kernel of its own: same bits as the
    oracle and as the general kernel, overwriting and accumulating, zeros of either sign included."""
    H, W, C, N, pool, stride, pad = geom
    shape = (H, W, C, N)
    x = _inputs(shape, 41, "normal")
    og = ob.pool_geom(shape, pool, stride, pad, "avg")
    assert ob.pool_out_shape(og)[:2] == (1, 1)
    dy = F(np.random.default_rng(42).standard_normal(ob.pool_out_shape(og)))
    dy[0, 0, 0, 0] = -0.0
    base = F(np.random.default_rng(43).standard_normal(shape))
    outs = []
    for force in (0, 1):
        try:
            capi.set_tunable("pool_force_gather", force)
            got, want = _run(capi, ob, x, dy, shape, pool, stride, pad, "avg")
            assert bits_equal(got, want)
            got2, want2 = _run(capi, ob, x, dy, shape, pool, stride, pad, "avg", accumulate_into=base)
            assert bits_equal(got2, want2)
            outs.append((got, got2))
        finally:
            capi.set_tunable("pool_force_gather", 0)
    assert bits_equal(outs[0][0], outs[1][0]) and bits_equal(outs[0][1], outs[1][1])


def test_golden_vectors_from_reference(capi):
    z = np.load(GOLDEN)
    for i in range(int(z["count"])):
        v = [int(t) for t in z["geom_%d" % i]]
        g = capi.PoolGeom(*v)
        xd, dyd = capi.to_device(z["x_%d" % i]), capi.to_device(z["dy_%d" % i])
        assert bits_equal(capi.to_host(capi.pool_forward(xd, g)), F(z["y_%d" % i])), i
        assert bits_equal(capi.to_host(capi.pool_backward(xd, dyd, g)), F(z["dx_%d" % i])), i


@pytest.mark.parametrize("ties", [False, True])
def test_baseline_max_pool_full_size_bit_exact(capi, ob, ties):
    """benchmark configuration 3a: 112x112x64x32, 3x3 stride 2 pad 1, and its 8-level tie-stress variant."""
    w = workloads.pool_max_case(ties=ties)
    got, want = _run(capi, ob, w["x"], w["dy"], w["x"].shape, w["pool"], w["stride"], w["pad"], "max")
    assert bits_equal(got, want), count_bit_mismatches(got, want)
    # size-independent property: every dzdy lands on exactly one input when the window has a finite max
    assert np.isclose(got.astype(np.float64).sum(), w["dy"].astype(np.float64).sum(), rtol=1e-6)


@pytest.mark.parametrize("shape,pad", [((224, 8, 2, 1), 1), ((8, 224, 2, 1), 1), ((16, 16, 3, 2), 1), ((112, 30, 2, 2), 1),
                                       ((40, 41, 1, 9), (1, 0, 1, 0)), ((8, 6, 70, 1), (1, 0, 1, 0))])
@pytest.mark.parametrize("mode", ["ties", "special", "normal"])
def test_table_kernel_small_planes(capi, ob, shape, pad, mode):
    """The kernel for 3x3 / stride 2 / padding 1 (`pool_pairs` = 1) on small planes: tall, wide, one column behind the
    last window (odd width), fewer planes than XCDs and more than workgroups; ties, NaN and infinities; bit-exact."""
    og = ob.pool_geom(shape, 3, 2, pad, "max")
    x = _inputs(shape, 21, mode)
    dy = F(np.random.default_rng(22).standard_normal(ob.pool_out_shape(og)))
    capi.set_tunable("pool_pairs", 1)
    try:
        capi.profile_begin("pool_backward_pairs")
        got, want = _run(capi, ob, x, dy, shape, 3, 2, pad, "max")
        launches, _ = capi.profile_end()
    finally:
        capi.set_tunable("pool_pairs", 0)
    assert launches >= 1
    assert bits_equal(got, want), count_bit_mismatches(got, want)


@pytest.mark.parametrize("ties", [False, True])
def test_baseline_max_pool_by_the_table_kernel_as_well(capi, ob, ties):
    """The same configuration through the kernel for 3x3 windows at stride 2 behind one row and column of padding (tiles
    by direct-to-LDS loads, one winner table, sums in registers; switched on by `pool_pairs`): the same bits, and the
    launches counted, so both kernels stay checked at the benchmarked size."""
    w = workloads.pool_max_case(ties=ties)
    capi.set_tunable("pool_pairs", 1)
    try:
        capi.profile_begin("pool_backward_pairs")
        got, want = _run(capi, ob, w["x"], w["dy"], w["x"].shape, w["pool"], w["stride"], w["pad"], "max")
        launches, _ = capi.profile_end()
    finally:
        capi.set_tunable("pool_pairs", 0)
    assert launches >= 1
    assert bits_equal(got, want), count_bit_mismatches(got, want)


def test_baseline_avg_pool_full_size_bit_exact(capi, ob):
    """benchmark configuration 3b: 56x56x256x32, 2x2 stride 2."""
    w = workloads.pool_avg_case()
    got, want = _run(capi, ob, w["x"], w["dy"], w["x"].shape, w["pool"], w["stride"], w["pad"], "avg")
    assert bits_equal(got, want), count_bit_mismatches(got, want)


def test_errors(capi):
    g = capi.pool_geom((8, 8, 1, 1), 3, 0, 0, "max")
    with pytest.raises(capi.McnError) as e:
        capi.pool_out_shape(g)
    assert e.value.code == capi.ILLEGAL_ARGUMENT
    g = capi.pool_geom((2, 2, 1, 1), 5, 1, 0, "max")
    with pytest.raises(capi.McnError):
        capi.pool_out_shape(g)
