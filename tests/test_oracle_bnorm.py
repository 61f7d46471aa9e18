"""Pins the batch-normalisation oracle: bit-for-bit against the compiled reference (float and double,
both moment modes), against committed golden vectors, against the closed forms of doc/blocks.tex
(restated with numpy two-pass statistics, as matlab/xtest/suite/nnbnorm.m:19-30 does), against torch's
batch_norm autograd in double, and against the invariants of the gradient."""
import os

import numpy as np
import pytest
import torch

from util import F, bits_equal, rel_max

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "bnorm_golden.npz")
SHAPES = [(2, 2, 1, 2), (8, 8, 3, 2), (13, 17, 4, 7), (8, 2, 3, 7), (1, 1, 5, 9)]  # rows, cols, C, N (nnbnorm.m sizes)


def _case(shape, seed, dtype):
    H, W, C, N = shape
    r = np.random.default_rng(seed)
    mu, sd = r.standard_normal(C), r.uniform(0.5, 2.0, C)
    x = F((r.standard_normal(shape) * sd[None, None, :, None] + mu[None, None, :, None]).astype(np.float32), dtype)
    g = r.uniform(0.5, 1.5, C).astype(np.float32).astype(dtype)
    b = (0.1 * r.standard_normal(C)).astype(np.float32).astype(dtype)
    dy = F(r.standard_normal(shape).astype(np.float32), dtype)
    return x, g, b, dy


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("eps", [1e-4, 1e-5])
def test_oracle_equals_reference_bitwise(ref, shape, dtype, eps):
    x, g, b, dy = _case(shape, 7, dtype)
    y, mom = ref.bnorm_forward(x, g, b, eps)
    ry, rmom = ref.ref_bnorm_forward(x, g, b, eps)
    assert bits_equal(y, ry) and bits_equal(mom, rmom)
    got = ref.bnorm_backward(x, g, dy, eps)
    want = ref.ref_bnorm_backward(x, g, b, dy, eps)
    for a, w in zip(got, want):
        assert bits_equal(a, w)
    # given-moments mode (vl_nnbnorm 'moments' option; nnbnorm.m:53-79)
    given = F(np.stack([np.linspace(-1, 1, shape[2]), np.linspace(0.5, 2, shape[2])], axis=1), dtype)
    assert bits_equal(ref.bnorm_forward(x, g, b, eps, moments=given)[0], ref.ref_bnorm_forward(x, g, b, eps, moments=given)[0])
    got = ref.bnorm_backward(x, g, dy, eps, moments=given)
    want = ref.ref_bnorm_backward(x, g, b, dy, eps, moments=given)
    for a, w in zip(got[:3], want[:3]):
        assert bits_equal(a, w)


def test_oracle_matches_golden_vectors(ob):
    z = np.load(GOLDEN)
    for k in range(int(z["count"])):
        x, g, b, dy, eps = F(z["x_%d" % k], None), z["g_%d" % k], z["b_%d" % k], F(z["dy_%d" % k], None), float(z["eps_%d" % k])
        y, mom = ob.bnorm_forward(x, g, b, eps)
        assert bits_equal(y, F(z["y_%d" % k], None)) and bits_equal(mom, F(z["mom_%d" % k], None))
        dx, dg, db, mom2 = ob.bnorm_backward(x, g, dy, eps)
        assert bits_equal(dx, F(z["dx_%d" % k], None)) and bits_equal(dg, z["dg_%d" % k])
        assert bits_equal(db, z["db_%d" % k]) and bits_equal(mom2, F(z["mom2_%d" % k], None))
        given = F(z["given_%d" % k], None)
        assert bits_equal(ob.bnorm_forward(x, g, b, eps, moments=given)[0], F(z["yg_%d" % k], None))
        dxg, dgg, dbg, _ = ob.bnorm_backward(x, g, dy, eps, moments=given)
        assert bits_equal(dxg, F(z["dxg_%d" % k], None)) and bits_equal(dgg, z["dgg_%d" % k]) and bits_equal(dbg, z["dbg_%d" % k])


EDGE = os.path.join(os.path.dirname(__file__), "golden", "bnorm_edge_golden.npz")


def test_oracle_matches_edge_golden_vectors(ob):
    """Outputs of the compiled reference at the corners of its one-pass variance (bits/nnbnorm.cu:64-70,118-132):
    a constant channel (the max(0, .) clamp, sigma = sqrt(epsilon) or a float rounding residue next to it), a channel
    with mean 1e3 and standard deviation 1e-2 (the float instantiation loses the variance, the double one keeps it)
    and one element per channel.  The oracle reproduces every bit, float and double."""
    z = np.load(EDGE)
    kinds = set()
    for k in range(int(z["count"])):
        x, g, b, dy, eps = F(z["x_%d" % k], None), z["g_%d" % k], z["b_%d" % k], F(z["dy_%d" % k], None), float(z["eps_%d" % k])
        y, mom = ob.bnorm_forward(x, g, b, eps)
        assert bits_equal(y, F(z["y_%d" % k], None)) and bits_equal(mom, F(z["mom_%d" % k], None))
        dx, dg, db, mom2 = ob.bnorm_backward(x, g, dy, eps)
        assert bits_equal(dx, F(z["dx_%d" % k], None)) and bits_equal(dg, z["dg_%d" % k])
        assert bits_equal(db, z["db_%d" % k]) and bits_equal(mom2, F(z["mom2_%d" % k], None))
        kinds.add(str(z["kind_%d" % k]))
    assert kinds == {"constant", "cancel", "cancel_mild", "single"}


def test_edge_golden_vectors_say_what_they_are_meant_to(ob):
    """The double outputs obey the closed forms (sigma of a constant channel is sqrt(epsilon); the 'cancel' channel
    has the two-pass variance); the float outputs of the same cases are off by what the one-pass formula loses in
    float.  So the fixtures do sit in the regime they are named for."""
    z = np.load(EDGE)
    for k in range(int(z["count"])):
        kind, x, eps, mom = str(z["kind_%d" % k]), z["x_%d" % k], float(z["eps_%d" % k]), z["mom2_%d" % k]
        c = {"constant": 1, "cancel": 0, "cancel_mild": 0, "single": 0}[kind]
        x64 = x[:, :, c, :].astype(np.float64)
        sigma = np.sqrt(x64.var() + eps)
        if x.dtype == np.float64:
            # (ten digits cancel in the 'cancel' channel: the double instantiation itself keeps about six)
            assert abs(mom[c, 1] - sigma) / sigma < (1e-4 if kind == "cancel" else 1e-7), (kind, mom[c, 1], sigma)
            if kind in ("constant", "single"):
                assert abs(mom[c, 1] - np.sqrt(eps)) / np.sqrt(eps) < 1e-6
        elif kind in ("cancel", "cancel_mild"):
            # float: nothing of the variance is left ('cancel'), or a digit or two ('cancel_mild')
            assert abs(mom[c, 1] - sigma) / sigma > (0.2 if kind == "cancel" else 1e-3)
        elif kind == "constant":
            assert 1e-4 < abs(mom[c, 1] - sigma) / sigma < 0.2   # float: a rounding residue under the root


@pytest.mark.parametrize("shape", SHAPES)
def test_closed_form_and_torch_autograd_double(ob, shape):
    """y = g (x - mu)/sqrt(var + eps) + b with the biased variance; gradients from torch autograd of the
    library batch_norm (training mode).  A dropped eps, an unbiased variance, sigma without the square
    root or a wrong sign in G2 each fail this."""
    eps = 1e-4
    x, g, b, dy = _case(shape, 9, np.float64)
    H, W, C, N = shape
    mu = x.mean(axis=(0, 1, 3))
    var = ((x - mu[None, None, :, None]) ** 2).mean(axis=(0, 1, 3))
    y, mom = ob.bnorm_forward(x, g, b, eps)
    assert rel_max(mom[:, 0], mu) < 1e-12
    assert rel_max(mom[:, 1], np.sqrt(var + eps)) < 1e-10
    want_y = g[None, None, :, None] * (x - mu[None, None, :, None]) / np.sqrt(var + eps)[None, None, :, None] + b[None, None, :, None]
    assert rel_max(y, want_y) < 1e-10

    xt = torch.from_numpy(np.ascontiguousarray(x.T)).requires_grad_(True)  # (N,C,W,H)
    gt = torch.from_numpy(g.copy()).requires_grad_(True)
    bt = torch.from_numpy(b.copy()).requires_grad_(True)
    yt = torch.nn.functional.batch_norm(xt, None, None, gt, bt, training=True, eps=eps)
    yt.backward(torch.from_numpy(np.ascontiguousarray(dy.T)))
    assert rel_max(y, yt.detach().numpy().T) < 1e-10
    dx, dg, db, _ = ob.bnorm_backward(x, g, dy, eps)
    assert rel_max(dx, xt.grad.numpy().T) < 1e-9
    assert rel_max(dg, gt.grad.numpy()) < 1e-9
    assert rel_max(db, bt.grad.numpy()) < 1e-12


def test_gradient_invariants(ob):
    """Per channel: sum dzdx = 0 and sum dzdx*(x - mu) = 0 (both up to the eps term); dzdy = 1 with any g
    gives dzdx = 0."""
    x, g, b, dy = _case((13, 17, 4, 7), 10, np.float64)
    dx, dg, db, mom = ob.bnorm_backward(x, g, dy, 1e-4)
    s = dx.sum(axis=(0, 1, 3))
    assert np.abs(s).max() < 1e-9
    dx1, _, _, _ = ob.bnorm_backward(x, g, F(np.ones_like(dy), np.float64), 1e-4)
    assert np.abs(dx1).max() < 1e-12


def test_given_moments_equal_batch_moments(ob):
    """Passing the moments returned by the batch mode reproduces the batch-mode result (nnbnorm.m:53-79)."""
    x, g, b, dy = _case((8, 8, 3, 2), 11, np.float64)
    y, mom = ob.bnorm_forward(x, g, b, 1e-4)
    y2, _ = ob.bnorm_forward(x, g, b, 1e-4, moments=mom)
    assert rel_max(y2, y) < 1e-13
    dx, dg, db, mom_b = ob.bnorm_backward(x, g, dy, 1e-4)
    dx2, dg2, db2, _ = ob.bnorm_backward(x, g, dy, 1e-4, moments=mom_b)
    assert rel_max(dx2, dx) < 1e-12 and rel_max(dg2, dg) < 1e-12 and rel_max(db2, db) < 1e-13


def test_known_moments_of_a_four_by_four_ramp(ob):
    # 4x4 ramp, C = N = 1, g = 2, eps = 1e-4: moments = (8.5, 4.60978)
    x = F(np.arange(1, 17, dtype=np.float32).reshape(4, 4, 1, 1, order="F"))
    _, mom = ob.bnorm_forward(x, np.array([2], np.float32), np.array([0], np.float32), 1e-4)
    assert abs(mom[0, 0] - 8.5) < 1e-6 and abs(mom[0, 1] - 4.60978) < 1e-5
