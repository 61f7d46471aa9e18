"""Pins of the oracle's subsample (vl_nnconv with empty FILTERS) and convolution-transpose restatements.

Neither bits/nnsubsample.cu nor bits/nnconv.cu can be compiled here (both include MATLAB's <blas.h>), so:
  * subsample is pinned by the reference's own definition -- empty FILTERS "pretend the identity filter bank"
    (matlab/src/vl_nnconv.cu:316-321) -- against the separately pinned convolution oracle, by brute force, and
    by the adjoint identity;
  * convolution transpose (composed as bits/nnconv.cu:323-421 composes it) is pinned by torch's
    conv_transpose2d and its autograd in double, and by the equivalences of matlab/xtest/suite/nnconvt.m
    (upsample = zero insertion, crop = cropping the full output, groups = block-diagonal filters).
"""
import numpy as np
import pytest
import torch

from util import F, bits_equal, rel_max

CASES = [  # (H, W, C, N, stride, pad)
    (9, 7, 3, 2, 1, 0),
    (9, 7, 3, 2, (2, 3), 0),
    (8, 8, 4, 1, 2, (1, 0, 2, 1)),
    (5, 6, 2, 3, (3, 1), (2, 2, 0, 3)),
    (1, 1, 5, 2, 4, 0),
    (7, 5, 1, 1, 10, (0, 1, 1, 0)),
]


@pytest.mark.parametrize("H,W,C,N,stride,pad", CASES)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_subsample_is_convolution_with_the_identity_bank(ob, H, W, C, N, stride, pad, dtype):
    r = np.random.default_rng(H * 100 + W)
    x = F(r.standard_normal((H, W, C, N)), dtype)
    b = r.standard_normal(C).astype(dtype)
    eye = F(np.eye(C).reshape(1, 1, C, C), dtype)
    g = ob.conv_geom(x.shape, eye.shape, stride, pad, 1)
    y = ob.subsample_forward(x, b, stride, pad)
    assert y.shape == ob.conv_out_shape(g) == ob.subsample_out_shape(x.shape, stride, pad)
    # values: x*1 + sum of exact zeros + b -- identical up to the sign of zero, so compare numerically and exactly
    assert np.array_equal(y, ob.conv_forward(x, eye, b, g))
    assert np.array_equal(ob.subsample_forward(x, None, stride, pad), ob.conv_forward(x, eye, None, g))
    dy = F(r.standard_normal(y.shape), dtype)
    dx = ob.subsample_backward(x.shape, dy, stride, pad)
    wdx, _, wdb = ob.conv_backward(x, eye, dy, g, want=(True, False, True))
    assert np.array_equal(dx, wdx)
    assert rel_max(dy.sum(axis=(0, 1, 3)), wdb) < 1e-5


def test_subsample_brute_force_and_adjoint(ob):
    r = np.random.default_rng(3)
    x = F(r.standard_normal((6, 5, 2, 2)), np.float64)
    sy, sx, pt, pb, pl, pr = 2, 3, 1, 2, 2, 0
    y = ob.subsample_forward(x, None, (sy, sx), (pt, pb, pl, pr))
    oh, ow = (6 + pt + pb - 1) // sy + 1, (5 + pl + pr - 1) // sx + 1
    assert y.shape == (oh, ow, 2, 2)
    for i in range(oh):
        for j in range(ow):
            h, w = i * sy - pt, j * sx - pl
            want = x[h, w] if 0 <= h < 6 and 0 <= w < 5 else np.zeros((2, 2))
            assert np.array_equal(y[i, j], want)
    dy = F(r.standard_normal(y.shape), np.float64)
    dx = ob.subsample_backward(x.shape, dy, (sy, sx), (pt, pb, pl, pr))
    assert abs((y * dy).sum() - (x * dx).sum()) < 1e-12  # <S x, dy> = <x, S' dy>


def to_t(a):
    return torch.tensor(np.ascontiguousarray(np.transpose(a, (3, 2, 0, 1))), requires_grad=True)


def from_t(t):
    return np.asfortranarray(np.transpose(t.detach().numpy(), (2, 3, 1, 0)))


CONVT = [  # (H, W, Cin, N, FH, FW, out channels per group, groups, upsample, crop)
    (5, 4, 4, 2, 3, 3, 3, 1, 2, (1, 0, 1, 1)),
    (6, 5, 6, 2, 4, 3, 2, 2, (2, 3), (0, 1, 2, 0)),
    (4, 4, 2, 1, 1, 1, 5, 1, 1, 0),
    (3, 3, 4, 3, 5, 5, 1, 4, 1, 2),
    (7, 2, 3, 1, 2, 4, 2, 3, (3, 1), (1, 1, 0, 0)),
]


@pytest.mark.parametrize("H,W,Cin,N,FH,FW,Cog,groups,up,crop", CONVT)
def test_convt_against_torch_double(ob, H, W, Cin, N, FH, FW, Cog, groups, up, crop):
    r = np.random.default_rng(H + 10 * W + 100 * Cin)
    x = F(r.standard_normal((H, W, Cin, N)), np.float64)
    f = F(r.standard_normal((FH, FW, Cog, Cin)), np.float64)
    b = r.standard_normal(Cog * groups)
    y = ob.convt_forward(x, f, b, up, crop, groups)
    assert y.shape == ob.convt_out_shape(x.shape, f.shape, up, crop, groups)
    xt, ft, bt = to_t(x), to_t(f), torch.tensor(b, requires_grad=True)
    uy, ux = ob._pair(up)
    ct, cb, cl, cr = ob._quad(crop)
    full = torch.nn.functional.conv_transpose2d(xt, ft, bt, stride=(uy, ux), groups=groups)
    yt = full[:, :, ct:full.shape[2] - cb, cl:full.shape[3] - cr]
    assert rel_max(y, from_t(yt)) < 1e-13
    dy = F(r.standard_normal(y.shape), np.float64)
    yt.backward(torch.tensor(np.ascontiguousarray(np.transpose(dy, (3, 2, 0, 1)))))
    dx, df, db = ob.convt_backward(x, f, dy, up, crop, groups)
    assert rel_max(dx, from_t(xt.grad)) < 1e-13
    assert rel_max(df, from_t(ft.grad)) < 1e-13
    assert rel_max(db, bt.grad.numpy()) < 1e-13
    # float instantiation stays within the conv gate of the double one
    yf = ob.convt_forward(F(x), F(f), b.astype(np.float32), up, crop, groups)
    assert rel_max(yf, y) < 2e-5


def test_convt_upsample_is_zero_insertion(ob):
    """matlab/xtest/suite/nnconvt.m: convt with upsample u equals convt with upsample 1 of the zero-stuffed input."""
    r = np.random.default_rng(9)
    x = F(r.standard_normal((4, 5, 3, 2)), np.float64)
    f = F(r.standard_normal((3, 2, 2, 3)), np.float64)
    uy, ux = 2, 3
    stuffed = np.zeros(((4 - 1) * uy + 1, (5 - 1) * ux + 1, 3, 2), order="F")
    stuffed[::uy, ::ux] = x
    assert rel_max(ob.convt_forward(x, f, None, (uy, ux), 0), ob.convt_forward(F(stuffed, np.float64), f, None, 1, 0)) < 1e-13


def test_taccum_is_the_scal_axpy_pair(ob):
    """vl_taccummex.cu:57-74: every element is fl(fl(alpha*a) + fl(beta*b)); numpy's float32 arithmetic rounds each
    operation separately, so the restatement must agree with it bit for bit; and the SGD momentum update it serves
    (cnn_train_dag.m:350-366) comes out as the closed form in double."""
    r = np.random.default_rng(2)
    a = F(r.standard_normal((7, 5, 3, 2)))
    b = F(r.standard_normal((7, 5, 3, 2)))
    alpha, beta = np.float32(0.9), np.float32(-0.0123)
    got = ob.taccum(float(alpha), a, float(beta), b)
    want = (alpha * a) + (beta * b)
    assert got.dtype == np.float32 and np.array_equal(got, want)
    got64 = ob.taccum(0.9, F(a, np.float64), -0.0123, F(b, np.float64))
    assert np.allclose(got64, 0.9 * a.astype(np.float64) - 0.0123 * b.astype(np.float64), rtol=1e-15, atol=0)
    assert np.array_equal(ob.taccum(1.0, a, 0.0, b), a) and np.array_equal(ob.taccum(0.0, a, 1.0, b), b)
