"""GPU parity, batch normalisation.  Gate (max|diff|/max|ref| over each output): 1e-5 against the double
instantiation of the reference algorithm fed the same float inputs.  The float instantiation sums ~1e5
terms sequentially in float and is itself further than 1e-5 from the double one at the benchmark sizes, so the
distance to it is asserted only to the looser bound it can support."""
import os

import numpy as np
import pytest

from matconvnet_amd import workloads
from util import F, rel_max

pytestmark = pytest.mark.gpu

TOL = 1e-5
GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "bnorm_golden.npz")
SHAPES = [(2, 2, 1, 2), (8, 8, 3, 2), (13, 17, 4, 7), (8, 2, 3, 7), (1, 1, 5, 9), (56, 56, 8, 4), (7, 7, 64, 5), (30, 30, 3, 70),
          (7, 7, 130, 6), (14, 14, 256, 4)]   # the last two: many small channels (one launch per call)


def _case(shape, seed):
    w = workloads.bnorm_case(seed=seed, H=shape[0], W=shape[1], C=shape[2], N=shape[3])
    return w["x"], w["g"], w["b"], w["dy"]


def _d(a):
    return F(a, np.float64) if a.ndim > 1 else a.astype(np.float64)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("eps", [1e-4, 1e-5])
def test_backward_batch_moments(capi, ob, shape, eps):
    x, g, b, dy = _case(shape, 7)
    dx, dg, db, mom = [capi.to_host(t) for t in capi.bnorm_backward(capi.to_device(x), capi.to_device(g), capi.to_device(dy), eps)]
    wdx, wdg, wdb, wmom = ob.bnorm_backward(_d(x), _d(g), _d(dy), eps)
    assert rel_max(dx, wdx) < TOL and rel_max(dg, wdg) < TOL and rel_max(db, wdb) < TOL and rel_max(mom, wmom) < TOL


@pytest.mark.parametrize("shape", SHAPES)
def test_backward_given_moments(capi, ob, shape):
    x, g, b, dy = _case(shape, 8)
    C = shape[2]
    given = F(np.stack([np.linspace(-1, 1, C), np.linspace(0.5, 2, C)], axis=1))
    dx, dg, db, _ = [capi.to_host(t) for t in capi.bnorm_backward(capi.to_device(x), capi.to_device(g), capi.to_device(dy), 1e-4, moments=capi.to_device(given))]
    wdx, wdg, wdb, _ = ob.bnorm_backward(_d(x), _d(g), _d(dy), 1e-4, moments=_d(given))
    assert rel_max(dx, wdx) < TOL and rel_max(dg, wdg) < TOL and rel_max(db, wdb) < TOL


@pytest.mark.parametrize("shape", SHAPES)
def test_forward_both_modes(capi, ob, shape):
    x, g, b, dy = _case(shape, 9)
    y, mom = [capi.to_host(t) for t in capi.bnorm_forward(capi.to_device(x), capi.to_device(g), capi.to_device(b), 1e-4)]
    wy, wmom = ob.bnorm_forward(_d(x), _d(g), _d(b), 1e-4)
    assert rel_max(y, wy) < TOL and rel_max(mom, wmom) < TOL
    y2, _ = capi.bnorm_forward(capi.to_device(x), capi.to_device(g), capi.to_device(b), 1e-4, moments=capi.to_device(wmom))
    assert rel_max(capi.to_host(y2), wy) < TOL


def test_moments_not_requested(capi, ob):
    """vl_nnbnorm with three outputs: no moments tensor is passed (vl_nnbnorm.cu:105,210-213)."""
    x, g, b, dy = _case((8, 8, 3, 2), 3)
    dx, dg, db, mom = capi.bnorm_backward(capi.to_device(x), capi.to_device(g), capi.to_device(dy), 1e-4, want_moments=False)
    assert mom is None
    wdx, wdg, wdb, _ = ob.bnorm_backward(_d(x), _d(g), _d(dy), 1e-4)
    assert rel_max(capi.to_host(dx), wdx) < TOL


def test_golden_vectors_from_reference(capi):
    """Outputs of the compiled reference (its double instantiation: entries with float64 dtype)."""
    z = np.load(GOLDEN)
    checked = 0
    for k in range(int(z["count"])):
        if z["x_%d" % k].dtype != np.float64:
            continue
        x, g, b, dy, eps = z["x_%d" % k], z["g_%d" % k], z["b_%d" % k], z["dy_%d" % k], float(z["eps_%d" % k])
        xd, gd, bd, dyd = capi.to_device(x), capi.to_device(g), capi.to_device(b), capi.to_device(dy)
        y, mom = [capi.to_host(t) for t in capi.bnorm_forward(xd, gd, bd, eps)]
        assert rel_max(y, z["y_%d" % k]) < TOL and rel_max(mom, z["mom_%d" % k]) < TOL
        dx, dg, db, mom2 = [capi.to_host(t) for t in capi.bnorm_backward(xd, gd, dyd, eps)]
        assert rel_max(dx, z["dx_%d" % k]) < TOL and rel_max(dg, z["dg_%d" % k]) < TOL
        assert rel_max(db, z["db_%d" % k]) < TOL and rel_max(mom2, z["mom2_%d" % k]) < TOL
        given = capi.to_device(z["given_%d" % k])
        dxg, dgg, dbg, _ = [capi.to_host(t) for t in capi.bnorm_backward(xd, gd, dyd, eps, moments=given)]
        assert rel_max(dxg, z["dxg_%d" % k]) < TOL and rel_max(dgg, z["dgg_%d" % k]) < TOL and rel_max(dbg, z["dbg_%d" % k]) < TOL
        checked += 1
    assert checked >= 4


EDGE = os.path.join(os.path.dirname(__file__), "golden", "bnorm_edge_golden.npz")


def test_edge_golden_vectors_from_reference(capi):
    """The corners of the one-pass variance (bits/nnbnorm.cu:64-70,118-132), outputs of the compiled reference: a
    constant channel (variance 0: the max(0, .) clamp, sigma = sqrt(epsilon)), a channel with standard deviation
    1e-2 around a mean of 1e3 ('cancel': E[x^2] - mean^2 cancels ten digits) or of 30 ('cancel_mild': seven), one element
    per channel.

    The device result is compared with the reference's DOUBLE instantiation run on the same float data, at the usual
    1e-5, on every output.  Why not the float one: in these corners the float instantiation is not a result to
    match -- its sigma of the constant channel is a rounding residue (0.00341 for sqrt(1e-5) = 0.00316), its variance of
    the large-mean channel is 0 or noise (sigma 0.0100 or 0.50 for 0.0140 and 0.0106), and which of these comes out
    depends on the summation order.  The device kernels widen each float to double before squaring and summing, so they
    keep what the double instantiation keeps.  The distance to the float instantiation is printed, not gated.
    In the 'cancel' cases the double instantiation is itself only good to about six digits (its sigma is 5e-6 from the
    two-pass value): any two summation orders differ by that much there, and the gate for those cases is 1e-4."""
    z = np.load(EDGE)
    checked = set()
    for k in range(int(z["count"])):
        if z["x_%d" % k].dtype != np.float64:
            continue
        kind = str(z["kind_%d" % k])
        x, g, b, dy, eps = z["x_%d" % k], z["g_%d" % k], z["b_%d" % k], z["dy_%d" % k], float(z["eps_%d" % k])
        xd, gd, bd, dyd = capi.to_device(x), capi.to_device(g), capi.to_device(b), capi.to_device(dy)
        y, mom = [capi.to_host(t) for t in capi.bnorm_forward(xd, gd, bd, eps)]
        dx, dg, db, mom2 = [capi.to_host(t) for t in capi.bnorm_backward(xd, gd, dyd, eps)]
        errs = dict(y=rel_max(y, z["y_%d" % k]), mom=rel_max(mom, z["mom_%d" % k]), dx=rel_max(dx, z["dx_%d" % k]),
                    dg=rel_max(dg, z["dg_%d" % k]), db=rel_max(db, z["db_%d" % k]), mom2=rel_max(mom2, z["mom2_%d" % k]))
        # per channel as well: the corner channel must not hide behind a larger neighbour
        sig, want_sig = mom2[:, 1].astype(np.float64), z["mom2_%d" % k][:, 1]
        errs["sigma_per_channel"] = float(np.abs(sig / want_sig - 1).max())
        for c in range(x.shape[2]):
            errs["dx_c%d" % c] = rel_max(dx[:, :, c, :], z["dx_%d" % k][:, :, c, :]) if np.abs(z["dx_%d" % k][:, :, c, :]).max() > 0 else float(np.abs(dx[:, :, c, :]).max())
        f = k - 1  # the float instantiation of the same case
        assert str(z["kind_%d" % f]) == kind and z["x_%d" % f].dtype == np.float32
        print("bnorm edge", kind, x.shape, "vs double:", {n: "%.1e" % v for n, v in errs.items()},
              "| vs float: dx %.1e sigma %.1e" % (rel_max(dx, z["dx_%d" % f]), np.abs(sig / z["mom2_%d" % f][:, 1] - 1).max()))
        # the forward output is normalised with the moments as they are stored, in float (so that a later pass given
        # them reproduces it bit for bit; the reference's float instantiation does the same): the stored mean is within
        # half an ulp of the double one, which moves y by up to that times |g|/sigma.  Only the 'cancel' kinds notice.
        want_mom = z["mom2_%d" % k]
        half_ulp = 0.5 * np.spacing(np.abs(want_mom[:, 0]).astype(np.float32)).astype(np.float64)
        y_gate = max(TOL, 2 * float((half_ulp * np.abs(g) / want_mom[:, 1]).max()) / float(np.abs(z["y_%d" % k]).max()))
        assert errs.pop("y") < y_gate, (kind, y_gate)
        assert max(errs.values()) < (1e-4 if kind == "cancel" else TOL), (kind, errs)
        checked.add(kind)
    assert checked == {"constant", "cancel", "cancel_mild", "single"}


def test_baseline_config_full_size(capi, ob):
    """benchmark configuration 2: 56x56x256x32, eps 1e-4, moments from the batch."""
    w = workloads.bnorm_case()
    x, g, dy = w["x"], w["g"], w["dy"]
    dx, dg, db, mom = [capi.to_host(t) for t in capi.bnorm_backward(capi.to_device(x), capi.to_device(g), capi.to_device(dy), w["eps"])]
    wdx, wdg, wdb, wmom = ob.bnorm_backward(_d(x), _d(g), _d(dy), w["eps"])
    d = dict(dzdx=rel_max(dx, wdx), dzdg=rel_max(dg, wdg), dzdb=rel_max(db, wdb), moments=rel_max(mom, wmom))
    print("bnorm cfg2 vs double oracle:", d)
    assert max(d.values()) < TOL, d
    # distance to the float instantiation (what the reference's float CPU path returns): reported, loosely bounded
    fdx, fdg, fdb, fmom = ob.bnorm_backward(x, g, dy, w["eps"])
    df = dict(dzdx=rel_max(dx, fdx), dzdg=rel_max(dg, fdg), dzdb=rel_max(db, fdb), moments=rel_max(mom, fmom))
    print("bnorm cfg2 vs float oracle:", df)
    assert max(df.values()) < 5e-4, df
    # size-independent invariants of the gradient, per channel
    s = dx.astype(np.float64).sum(axis=(0, 1, 3))
    assert np.abs(s).max() / np.abs(dx).astype(np.float64).sum(axis=(0, 1, 3)).max() < 1e-5


def test_bottleneck_shapes(capi, ob):
    """The two bnorm shapes of benchmark configuration 4 (eps 1e-5)."""
    for C in (64, 256):
        w = workloads.bnorm_case(seed=20 + C, C=C, N=8, eps=1e-5)
        x, g, dy = w["x"], w["g"], w["dy"]
        dx, dg, db, mom = [capi.to_host(t) for t in capi.bnorm_backward(capi.to_device(x), capi.to_device(g), capi.to_device(dy), 1e-5)]
        wdx, wdg, wdb, wmom = ob.bnorm_backward(_d(x), _d(g), _d(dy), 1e-5)
        assert rel_max(dx, wdx) < TOL and rel_max(dg, wdg) < TOL and rel_max(db, wdb) < TOL and rel_max(mom, wmom) < TOL


@pytest.mark.parametrize("shape", [(7, 7, 130, 6), (14, 14, 256, 4), (2, 2, 128, 9), (4, 6, 192, 32)])
def test_small_channels_in_one_launch_give_the_same_bits(capi, shape):
    """Channels of a few thousand elements are summed and normalised by one launch (one workgroup per channel does
    both); with that switched off the usual two launches run: every output of every entry point has the same bits."""
    from util import bits_equal
    H, W, C, N = shape
    w = workloads.bnorm_case(seed=21, H=H, W=W, C=C, N=N)
    r = np.random.default_rng(22)
    later = F(r.standard_normal(w["x"].shape))
    later[::3] = 0.0
    res = F(r.standard_normal(w["x"].shape))
    xd, gd, bd, dyd, ld, rd = (capi.to_device(v) for v in (w["x"], w["g"], w["b"], w["dy"], later, res))
    old = capi.get_tunable("bnorm_one_launch_elems")
    outs = []
    try:
        for limit in (old, 0):
            capi.set_tunable("bnorm_one_launch_elems", limit)
            got = []
            y, mom = capi.bnorm_forward(xd, gd, bd, 1e-5)
            got += [y, mom]
            got += list(capi.bnorm_forward_fused(xd, gd, bd, residual=rd, relu=True, eps=1e-5))
            got += list(capi.bnorm_forward_fused(xd, gd, bd, relu=True, eps=1e-5))
            got += list(capi.bnorm_backward(xd, gd, dyd, 1e-5))
            got += list(capi.bnorm_backward(xd, gd, dyd, 1e-5, moments=mom))
            got += list(capi.bnorm_backward_relu(xd, gd, bd, dyd, mom, 1e-5))
            got += list(capi.bnorm_backward_masked(xd, gd, dyd, ld, mom, 1e-5))
            outs.append([capi.to_host(t) for t in got if t is not None])
    finally:
        capi.set_tunable("bnorm_one_launch_elems", old)
    assert len(outs[0]) == len(outs[1]) and len(outs[0]) >= 20
    for a, b_ in zip(*outs):
        assert bits_equal(a, b_)


def test_relu_mask_as_bits_matches_the_float_mask_paths(capi, ob):
    """The residual unit's last ReLU with its mask kept as one bit per element: the forward pass that writes the bits
    gives the same y and moments as the one that does not, the bits say y > 0 element by element, and the batch-norm
    derivative that reads them is bit-identical to the one that reads the ReLU's output (mcn_bnorm_backward_masked)."""
    import torch
    from util import bits_equal
    H, W, Cc, N = 56, 56, 32, 6
    assert capi.lib().mcn_bnorm_mask_bits_supported(H, W, Cc, N) == 1
    assert capi.lib().mcn_bnorm_mask_bits_supported(14, 14, Cc, N) == 0      # planes of 196 elements: not whole words
    r = np.random.default_rng(21)
    x = capi.to_device(F(r.standard_normal((H, W, Cc, N)) * 1.5 + 0.2))
    res = capi.to_device(F(r.standard_normal((H, W, Cc, N))))
    dy = capi.to_device(F(r.standard_normal((H, W, Cc, N))))
    g = capi.to_device(F(r.uniform(0.5, 1.5, Cc)).ravel())
    b = capi.to_device(F(r.standard_normal(Cc) * 0.1).ravel())
    # partial sums in the layout a summing convolution leaves them: [channel][group][2]
    xd = x.double()
    groups = 3
    cuts = [0, 2, 4, N]
    sums = torch.stack([torch.stack([xd[cuts[k]:cuts[k + 1]].sum(dim=(0, 2, 3)), (xd[cuts[k]:cuts[k + 1]] ** 2).sum(dim=(0, 2, 3))], dim=1)
                        for k in range(groups)], dim=1).contiguous()
    y0, m0 = capi.bnorm_forward_sums(x, g, b, sums, residual=res, relu=True, eps=1e-5)
    y1, bits, m1 = capi.bnorm_forward_sums_mask(x, g, b, sums, residual=res, eps=1e-5)
    assert torch.equal(y0, y1) and torch.equal(m0, m1)
    want = (y1.reshape(-1) > 0).to(torch.int64).reshape(-1, 32)
    weights = (1 << torch.arange(32, device="cuda", dtype=torch.int64))
    words = (want * weights).sum(dim=1)
    assert torch.equal(words, bits.to(torch.int64) & 0xffffffff)
    got = capi.bnorm_backward_bits(x, g, dy, bits, m1, eps=1e-5)
    ref = capi.bnorm_backward_masked(x, g, dy, y1, m1, eps=1e-5)
    for a, c in zip(got, ref[:3]):
        assert bits_equal(capi.to_host(a), capi.to_host(c))
