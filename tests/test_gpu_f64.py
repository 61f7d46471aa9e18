"""GPU parity, double precision (the operators' VLDT_Double instantiation): the HIP kernels through the C ABI against
the CPU oracle's double instantiation.  Gates: pooling bit-exact (the kernels keep the order of the reference's
loops); convolution and batch normalisation 1e-12 (max|diff|/max|ref|; only the order of the sums differs, and
every accumulator is a double)."""
import os

import numpy as np
import pytest

from util import F, bits_equal, count_bit_mismatches, rel_max

pytestmark = pytest.mark.gpu

TOL = 1e-12
D = np.float64
BNORM_GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "bnorm_golden.npz")

CONV_CASES = [
    # x, f, stride, pad, dilate
    ((8, 7, 3, 2), (3, 3, 3, 4), 1, 0, 1),
    ((9, 8, 4, 3), (3, 2, 4, 5), (2, 1), (1, 0, 2, 1), 1),
    ((12, 11, 6, 2), (3, 3, 3, 4), 1, 1, 1),                 # two filter groups
    ((13, 12, 2, 2), (3, 3, 2, 3), (2, 3), (2, 1, 0, 2), (2, 1)),   # stride and dilation
    ((6, 6, 8, 3), (1, 1, 8, 16), 1, 0, 1),
    ((5, 5, 4, 2), (5, 5, 4, 7), 1, 0, 1),                   # fully connected
    ((32, 32, 3, 4), (5, 5, 3, 32), 1, 2, 1),                # benchmark configuration 1, four images
    ((14, 13, 16, 3), (3, 3, 16, 24), 1, 1, 1),              # sixteen and more columns in every product: the matrix instruction
    ((15, 12, 20, 2), (3, 2, 20, 70), (2, 1), (1, 0, 2, 1), (1, 2)),   # the same with stride, dilation, partial tiles
    ((9, 9, 64, 2), (1, 1, 64, 64), 1, 0, 1),                # 1x1
    ((7, 9, 1, 2), (3, 2, 1, 5), 1, (2, 0, 1, 1), 1),        # one, two and four input channels, uneven padding: the
    ((6, 5, 2, 3), (2, 3, 2, 4), 1, (1, 1, 2, 0), 1),        # pixel-per-thread input gradient of first layers
    ((10, 6, 4, 2), (5, 3, 4, 6), 1, (0, 4, 2, 1), 1),
    ((16, 15, 3, 2), (7, 7, 3, 8), 1, 3, 1), ((9, 11, 4, 2), (3, 3, 4, 5), 1, (1, 2, 0, 1), 1),   # square windows: unrolled
]

POOL_GEOMS = [
    (5, 6, 2, 3, 2, 1, 0), (5, 6, 2, 3, 3, 2, 1), (8, 8, 1, 2, 3, 3, 2), (7, 9, 3, 1, (2, 3), (1, 2), (1, 0, 2, 1)),
    (9, 7, 2, 2, (3, 2), (2, 1), (0, 1, 1, 0)), (4, 4, 1, 1, 4, 4, 3), (12, 12, 2, 2, 3, 2, 1),
    (10, 3, 1, 2, (5, 3), (3, 1), (2, 2, 1, 1)), (28, 28, 5, 3, 3, 2, 1), (33, 47, 3, 2, (3, 5), (2, 3), (1, 2, 4, 0)),
]


@pytest.mark.parametrize("xs,fs,stride,pad,dilate", CONV_CASES)
@pytest.mark.parametrize("with_bias", [False, True])
def test_convolution(capi, ob, xs, fs, stride, pad, dilate, with_bias):
    r = np.random.default_rng(sum(xs) + sum(fs))
    x = F(r.standard_normal(xs), D)
    f = F(r.standard_normal(fs), D)
    b = r.standard_normal(fs[3]) if with_bias else None
    g = ob.conv_geom(xs, fs, stride, pad, dilate)
    cg = capi.conv_geom(xs, fs, stride, pad, dilate)
    xd, fd = capi.to_device(x, D), capi.to_device(f, D)
    bd = None if b is None else capi.to_device(b, D)
    y = capi.conv_forward(xd, fd, bd, cg)
    want = ob.conv_forward(x, f, b, g)
    got = capi.to_host(y)
    assert got.dtype == D and rel_max(got, want) < TOL
    # y = outMult*y + inMult*conv + b
    base = F(r.standard_normal(want.shape), D)
    y2 = capi.conv_forward(xd, fd, bd, cg, y=capi.to_device(base, D), out_mult=0.5, in_mult=-2.0)
    assert rel_max(capi.to_host(y2), ob.conv_forward(x, f, b, g, y=base.copy(order="F"), out_mult=0.5, in_mult=-2.0)) < TOL
    dy = F(r.standard_normal(want.shape), D)
    dx, df, db = capi.conv_backward(xd, fd, capi.to_device(dy, D), cg)
    wdx, wdf, wdb = ob.conv_backward(x, f, dy, g)
    assert rel_max(capi.to_host(dx), wdx) < TOL
    assert rel_max(capi.to_host(df), wdf) < TOL
    assert rel_max(capi.to_host(db).reshape(-1), np.asarray(wdb).reshape(-1)) < TOL


def test_convolution_adjoint_identity(capi):
    """<dzdy, conv(x + d) - conv(x)> = <dzdx, d>, and the same for the filters: exact up to rounding, no oracle."""
    r = np.random.default_rng(3)
    xs, fs = (11, 10, 4, 3), (3, 4, 2, 6)
    cg = capi.conv_geom(xs, fs, (2, 1), (1, 2, 0, 1), 1)
    x, d = F(r.standard_normal(xs), D), F(r.standard_normal(xs), D)
    f, e = F(r.standard_normal(fs), D), F(r.standard_normal(fs), D)
    y0 = capi.to_host(capi.conv_forward(capi.to_device(x, D), capi.to_device(f, D), None, cg))
    y1 = capi.to_host(capi.conv_forward(capi.to_device(x + d, D), capi.to_device(f, D), None, cg))
    y2 = capi.to_host(capi.conv_forward(capi.to_device(x, D), capi.to_device(f + e, D), None, cg))
    dy = F(r.standard_normal(y0.shape), D)
    dx, df, _ = capi.conv_backward(capi.to_device(x, D), capi.to_device(f, D), capi.to_device(dy, D), cg)
    lhs_x, rhs_x = float((dy * (y1 - y0)).sum()), float((capi.to_host(dx) * d).sum())
    lhs_f, rhs_f = float((dy * (y2 - y0)).sum()), float((capi.to_host(df) * e).sum())
    assert abs(lhs_x - rhs_x) < 1e-10 * max(abs(lhs_x), 1.0)
    assert abs(lhs_f - rhs_f) < 1e-10 * max(abs(lhs_f), 1.0)


@pytest.mark.parametrize("shape", [(2, 2, 1, 2), (8, 8, 3, 2), (13, 17, 4, 7), (1, 1, 5, 9), (56, 56, 8, 4), (7, 7, 64, 5)])
@pytest.mark.parametrize("eps", [1e-4, 1e-5])
def test_batch_normalisation(capi, ob, shape, eps):
    r = np.random.default_rng(sum(shape))
    Cc = shape[2]
    x = F(r.standard_normal(shape) * r.uniform(0.5, 2, (1, 1, Cc, 1)) + r.standard_normal((1, 1, Cc, 1)), D)
    g, b = r.uniform(0.5, 1.5, Cc), r.standard_normal(Cc) * 0.1
    dy = F(r.standard_normal(shape), D)
    xd, gd, bd, dyd = (capi.to_device(v, D) for v in (x, g, b, dy))
    y, mom = [capi.to_host(t) for t in capi.bnorm_forward(xd, gd, bd, eps)]
    wy, wmom = ob.bnorm_forward(x, g, b, eps)
    assert y.dtype == D and rel_max(y, wy) < TOL and rel_max(mom, wmom) < TOL
    dx, dg, db, mom2 = [capi.to_host(t) for t in capi.bnorm_backward(xd, gd, dyd, eps)]
    wdx, wdg, wdb, wmom2 = ob.bnorm_backward(x, g, dy, eps)
    # dzdg is a difference of two sums of ~m terms: its error scales with the sums, not with the (smaller) result
    slack = max(1.0, float(np.abs(x).max() * np.abs(dy).sum(axis=(0, 1, 3)).max() / max(np.abs(wdg).max(), 1e-300)) * 1e-3)
    assert rel_max(dx, wdx) < TOL * slack and rel_max(dg, wdg) < TOL * slack
    assert rel_max(db, wdb) < TOL and rel_max(mom2, wmom2) < TOL
    # moments given (DagNN's mode) and moments not requested
    given = F(np.stack([np.linspace(-1, 1, Cc), np.linspace(0.5, 2, Cc)], axis=1), D)
    gvd = capi.to_device(given, D)
    y3, _ = capi.bnorm_forward(xd, gd, bd, eps, moments=gvd)
    assert rel_max(capi.to_host(y3), ob.bnorm_forward(x, g, b, eps, moments=given)[0]) < TOL
    dx3, dg3, db3, _ = [capi.to_host(t) for t in capi.bnorm_backward(xd, gd, dyd, eps, moments=gvd)]
    wdx3, wdg3, wdb3, _ = ob.bnorm_backward(x, g, dy, eps, moments=given)
    assert rel_max(dx3, wdx3) < TOL * slack and rel_max(dg3, wdg3) < TOL * slack and rel_max(db3, wdb3) < TOL
    dx4, _, _, none = capi.bnorm_backward(xd, gd, dyd, eps, want_moments=False)
    assert none is None and bits_equal(capi.to_host(dx4), dx)


def test_batch_normalisation_golden_vectors_from_reference(capi):
    """Outputs of the compiled reference's double instantiation, on its own double inputs."""
    z = np.load(BNORM_GOLDEN)
    checked = 0
    for k in range(int(z["count"])):
        if z["x_%d" % k].dtype != np.float64:
            continue
        x, g, b, dy, eps = z["x_%d" % k], z["g_%d" % k], z["b_%d" % k], z["dy_%d" % k], float(z["eps_%d" % k])
        xd, gd, bd, dyd = (capi.to_device(v, D) for v in (x, g, b, dy))
        y, mom = [capi.to_host(t) for t in capi.bnorm_forward(xd, gd, bd, eps)]
        assert rel_max(y, z["y_%d" % k]) < 1e-11 and rel_max(mom, z["mom_%d" % k]) < 1e-11
        dx, dg, db, mom2 = [capi.to_host(t) for t in capi.bnorm_backward(xd, gd, dyd, eps)]
        assert rel_max(dx, z["dx_%d" % k]) < 1e-10 and rel_max(dg, z["dg_%d" % k]) < 1e-10
        assert rel_max(db, z["db_%d" % k]) < 1e-11 and rel_max(mom2, z["mom2_%d" % k]) < 1e-11
        given = capi.to_device(z["given_%d" % k], D)
        dxg, dgg, dbg, _ = [capi.to_host(t) for t in capi.bnorm_backward(xd, gd, dyd, eps, moments=given)]
        assert rel_max(dxg, z["dxg_%d" % k]) < 1e-10 and rel_max(dgg, z["dgg_%d" % k]) < 1e-10
        assert rel_max(dbg, z["dbg_%d" % k]) < 1e-11
        checked += 1
    assert checked >= 4


def _pool_inputs(shape, seed, mode):
    r = np.random.default_rng(seed)
    n = int(np.prod(shape))
    if mode == "ties":
        x = r.integers(0, 3, size=shape).astype(D)
    elif mode == "special":
        x = r.integers(0, 3, size=shape).astype(D)
        flat = x.reshape(-1)
        flat[r.random(n) < 0.25] = np.nan
        flat[r.random(n) < 0.25] = -np.inf
        flat[r.random(n) < 0.05] = np.inf
    else:
        x = r.standard_normal(shape)
    return F(x, D)


@pytest.mark.parametrize("geom", POOL_GEOMS)
@pytest.mark.parametrize("method", ["max", "avg"])
@pytest.mark.parametrize("mode", ["ties", "special", "normal"])
def test_pooling_bit_exact(capi, ob, geom, method, mode):
    H, W, Cc, N, pool, stride, pad = geom
    shape = (H, W, Cc, N)
    g = capi.pool_geom(shape, pool, stride, pad, method)
    og = ob.pool_geom(shape, pool, stride, pad, method)
    x = _pool_inputs(shape, 11, mode if method == "max" else "normal")
    r = np.random.default_rng(12)
    dy = F(r.standard_normal(ob.pool_out_shape(og)), D)
    xd, dyd = capi.to_device(x, D), capi.to_device(dy, D)
    y = capi.to_host(capi.pool_forward(xd, g))
    assert y.dtype == D and bits_equal(y, ob.pool_forward(x, og))
    got = capi.to_host(capi.pool_backward(xd, dyd, g))
    want = ob.pool_backward(x, dy, og)
    assert bits_equal(got, want), count_bit_mismatches(got, want)
    # accumulating into a caller's buffer (the contract of vl::nn::Pooling::backward)
    base = F(r.standard_normal(shape), D)
    got = capi.to_host(capi.pool_backward(xd, dyd, g, dx=capi.to_device(base, D)))
    want = ob.pool_backward(x, dy, og, dx=base.copy(order="F"))
    assert bits_equal(got, want), count_bit_mismatches(got, want)


@pytest.mark.parametrize("switch", ["conv64_no_mfma", "pool64_no_tiles"])
def test_general_double_kernels_stay_checked(capi, ob, switch):
    """With the matrix-instruction convolutions / the LDS strips of max-pool backward switched off, the one-accumulator
    kernels serve the same shapes: against the oracle as above."""
    capi.set_tunable(switch, 1)
    try:
        if switch == "conv64_no_mfma":
            test_convolution(capi, ob, (14, 13, 16, 3), (3, 3, 16, 24), 1, 1, 1, True)
        else:
            test_pooling_bit_exact(capi, ob, (28, 28, 5, 3, 3, 2, 1), "max", "ties")
    finally:
        capi.set_tunable(switch, 0)


@pytest.mark.parametrize("geom", [(112, 112, 3, 2, 3, 2, (0, 1, 0, 1)), (56, 40, 4, 2, 2, 2, 0), (30, 17, 2, 3, 3, 2, 1),
                                  (64, 64, 2, 2, (3, 2), (2, 2), (1, 1, 0, 0)), (6, 5, 3, 2, 3, 1, 1)])
@pytest.mark.parametrize("mode", ["ties", "special"])
def test_max_pool_backward_streaming_and_strips(capi, ob, geom, mode):
    """Heights of whole 16-byte cells take single precision's streaming kernel (several tiles per plane, the frame's
    borders, ties and non-finite values); with that kernel switched off the same shapes go through the LDS strips."""
    test_pooling_bit_exact(capi, ob, geom, "max", mode)
    capi.set_tunable("pool_force_gather", 1)
    try:
        test_pooling_bit_exact(capi, ob, geom, "max", mode)
    finally:
        capi.set_tunable("pool_force_gather", 0)


@pytest.mark.parametrize("geom", [(56, 56, 5, 2, 2, 2, 0), (8, 12, 3, 2, (2, 3), (2, 3), 0), (12, 9, 2, 3, (6, 3), (6, 3), 0)])
def test_average_pooling_over_exact_tiles(capi, ob, geom):
    """Windows that tile the plane exactly, columns of whole 16-byte cells: the streaming pass in memory order; with it
    switched off, the one-thread-per-element kernel.  Same bits either way."""
    test_pooling_bit_exact(capi, ob, geom, "avg", "normal")
    capi.set_tunable("pool64_no_tiles", 1)
    try:
        test_pooling_bit_exact(capi, ob, geom, "avg", "normal")
    finally:
        capi.set_tunable("pool64_no_tiles", 0)


def test_mixed_precision_is_refused(capi):
    """All tensors of a call are single or all are double (bits/data.hpp:260-266)."""
    x = capi.to_device(np.zeros((4, 4, 1, 1)), D)
    f = capi.to_device(np.zeros((3, 3, 1, 1)))
    with pytest.raises(TypeError):
        capi.conv_forward(x, f, None, capi.conv_geom((4, 4, 1, 1), (3, 3, 1, 1)))


# ---- through the C++ operator layer and the MEX-convention front-end -----------------------------------------------

def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(np.asfortranarray(a, dtype=D).T)).cuda()


def _host(t):
    return np.asfortranarray(t.detach().cpu().numpy().T)


def test_front_end_double_tensors(vl, ob):
    """vl_nnconv / vl_nnbnorm / vl_nnpool called with double arrays, as the reference's tests call every operator for
    both data types (matlab/xtest/suite/nntest.m: dataType 'single' and 'double'): outputs are double and match the
    oracle's double instantiation."""
    import torch
    r = np.random.default_rng(1)
    x = F(r.standard_normal((14, 12, 6, 3)), D)
    f = F(r.standard_normal((3, 3, 6, 8)) * 0.2, D)
    b = r.standard_normal(8)
    g = ob.conv_geom(x.shape, f.shape, (2, 1), (1, 0, 2, 1), 1)
    y = vl.vl_nnconv(_dev(x), _dev(f), _dev(b), "pad", [1, 0, 2, 1], "stride", [2, 1])
    want = ob.conv_forward(x, f, b, g)
    assert y.dtype == torch.float64 and tuple(reversed(y.shape)) == want.shape and rel_max(_host(y), want) < TOL
    dy = F(r.standard_normal(want.shape), D)
    dx, df, db = vl.vl_nnconv(_dev(x), _dev(f), _dev(b), _dev(dy), "pad", [1, 0, 2, 1], "stride", [2, 1])
    wdx, wdf, wdb = ob.conv_backward(x, f, dy, g)
    assert dx.dtype == torch.float64
    assert rel_max(_host(dx), wdx) < TOL and rel_max(_host(df), wdf) < TOL and rel_max(_host(db).ravel(), wdb) < TOL

    gm, bs = r.uniform(0.5, 1.5, 6), r.standard_normal(6) * 0.1
    yb, mom = vl.vl_nnbnorm(_dev(x), _dev(gm), _dev(bs), "epsilon", 1e-5, nout=2)
    wy, wmom = ob.bnorm_forward(x, gm, bs, 1e-5)
    assert yb.dtype == torch.float64 and rel_max(_host(yb), wy) < TOL and rel_max(_host(mom), wmom) < TOL
    dyb = F(r.standard_normal(x.shape), D)
    dxb, dgb, dbb = vl.vl_nnbnorm(_dev(x), _dev(gm), _dev(bs), _dev(dyb), "epsilon", 1e-5)
    wdx, wdg, wdb, _ = ob.bnorm_backward(x, gm, dyb, 1e-5)
    assert rel_max(_host(dxb), wdx) < 1e-10 and rel_max(_host(dgb).ravel(), wdg) < 1e-10 and rel_max(_host(dbb).ravel(), wdb) < TOL

    for method in ("max", "avg"):
        og = ob.pool_geom(x.shape, (3, 2), (2, 1), (1, 0, 0, 1), method)
        yp = vl.vl_nnpool(_dev(x), [3, 2], "stride", [2, 1], "pad", [1, 0, 0, 1], "method", method)
        assert yp.dtype == torch.float64 and bits_equal(_host(yp), ob.pool_forward(x, og))
        dyp = F(r.standard_normal(ob.pool_out_shape(og)), D)
        dxp = vl.vl_nnpool(_dev(x), [3, 2], _dev(dyp), "stride", [2, 1], "pad", [1, 0, 0, 1], "method", method)
        assert bits_equal(_host(dxp), ob.pool_backward(x, dyp, og))


def test_front_end_double_companions(vl, ob):
    """The other operators of the front-end in double: vl_nnconv with empty filters (subsampling with bias),
    vl_nnconvt, vl_taccum."""
    import torch
    r = np.random.default_rng(2)
    x = F(r.standard_normal((9, 8, 4, 2)), D)
    b = r.standard_normal(4)
    none = torch.empty((0,), dtype=torch.float64, device="cuda")
    y = vl.vl_nnconv(_dev(x), none, _dev(b), "stride", [2, 3], "pad", [1, 0, 2, 1])
    want = ob.subsample_forward(x, b, (2, 3), (1, 0, 2, 1))
    assert y.dtype == torch.float64 and bits_equal(_host(y), want)
    dy = F(r.standard_normal(want.shape), D)
    dx, df, db = vl.vl_nnconv(_dev(x), none, _dev(b), _dev(dy), "stride", [2, 3], "pad", [1, 0, 2, 1])
    wdx = ob.subsample_backward(x.shape, dy, (2, 3), (1, 0, 2, 1))
    assert bits_equal(_host(dx), wdx) and rel_max(_host(db).ravel(), dy.sum(axis=(0, 1, 3))) < TOL and df.numel() == 0

    f = F(r.standard_normal((3, 3, 5, 4)) * 0.3, D)   # FH x FW x K x C
    bt = r.standard_normal(5)
    yt = vl.vl_nnconvt(_dev(x), _dev(f), _dev(bt), "upsample", 2, "crop", [1, 0, 0, 1])
    wt = ob.convt_forward(x, f, bt, 2, (1, 0, 0, 1))
    assert yt.dtype == torch.float64 and tuple(reversed(yt.shape)) == wt.shape and rel_max(_host(yt), wt) < TOL
    dyt = F(r.standard_normal(wt.shape), D)
    dxt, dft, dbt = vl.vl_nnconvt(_dev(x), _dev(f), _dev(bt), _dev(dyt), "upsample", 2, "crop", [1, 0, 0, 1])
    wdx, wdf, wdb = ob.convt_backward(x, f, dyt, 2, (1, 0, 0, 1))
    assert rel_max(_host(dxt), wdx) < TOL and rel_max(_host(dft), wdf) < TOL and rel_max(_host(dbt).ravel(), wdb) < TOL

    a, c = F(r.standard_normal((5, 4, 3, 2)), D), F(r.standard_normal((5, 4, 3, 2)), D)
    got = vl.vl_taccum(0.9, _dev(a), -0.37, _dev(c))
    assert got.dtype == torch.float64 and bits_equal(_host(got), ob.taccum(0.9, a, -0.37, c))


def test_mixed_precision_is_refused_by_the_front_end(vl):
    import torch
    x = torch.zeros((2, 4, 8, 8), dtype=torch.float64, device="cuda")
    f = torch.zeros((5, 4, 3, 3), dtype=torch.float32, device="cuda")
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnconv(x, f, torch.zeros((5,), device="cuda"))
    assert e.value.message == "DATA and FILTERS do not have compatible formats."
