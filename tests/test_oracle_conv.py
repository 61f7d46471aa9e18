"""Pins the convolution oracle.

vl::nn::Convolution itself cannot be compiled here (it needs MATLAB's <blas.h> / libmwblas), so:
  * im2row / row2im are compared bit-for-bit with the reference's own impl/im2row_cpu.cpp (oracle/_ref)
    and with golden vectors written from it;
  * the GEMM is compared with numpy's matmul (a library routine) in all transpose modes used;
  * conv forward/backward are compared with torch's conv2d autograd in double (library routine, incl.
    stride, dilation, symmetric padding, groups), with a direct loop-nest gradient on tiny shapes
    (asymmetric padding), with the adjoint identities, and with the equivalences the reference's own
    tests assert (matlab/xtest/suite/nnconv.m:88-161).
A transposed filter, a flipped tap, a wrong pad side, a wrong group slice or a missing image in the
accumulation each fail at least one of these."""
import os

import numpy as np
import pytest
import torch

from util import F, bits_equal, rel_max

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "im2row_golden.npz")

# H, W, C, FH, FW, stride, pad, dilate
IM2ROW = [
    (6, 7, 2, 3, 3, 1, 1, 1), (9, 8, 2, 3, 2, (2, 3), (1, 0, 2, 1), 1), (11, 10, 1, 3, 3, (3, 2), (2, 2, 3, 3), (2, 1)),
    (5, 5, 3, 1, 1, 1, 0, 1), (8, 8, 2, 5, 5, 1, 2, 1), (10, 9, 2, 2, 3, 2, (3, 0, 0, 2), (3, 2)),
    (64, 64, 2, 11, 11, (3, 2), (5, 5, 8, 8), 1),  # nnconv.m:163-202 geometry
    (4, 4, 1, 3, 3, 1, (0, 4, 0, 4), 1),           # pad larger than needed on one side
]


@pytest.mark.parametrize("case", IM2ROW)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_im2row_equals_reference_bitwise(ref, case, dtype):
    H, W, C, FH, FW, stride, pad, dilate = case
    g = ref.conv_geom((H, W, C, 1), (FH, FW, C, 1), stride, pad, dilate)
    r = np.random.default_rng(1)
    x = F(r.standard_normal((H, W, C)), dtype)
    st = ref.im2row_forward(x, g)
    assert bits_equal(st, ref.ref_im2row_forward(x, g))
    t = F(r.standard_normal(st.shape), dtype)
    assert bits_equal(ref.im2row_backward(t, g), ref.ref_im2row_backward(t, g))


def test_im2row_matches_golden_vectors(ob):
    z = np.load(GOLDEN)
    for i in range(int(z["count"])):
        v = [int(t) for t in z["geom_%d" % i]]
        g = ob.ConvGeom(*v)
        assert bits_equal(ob.im2row_forward(F(z["x_%d" % i]), g), F(z["stacked_%d" % i])), i
        assert bits_equal(ob.im2row_backward(F(z["t_%d" % i]), g), F(z["back_%d" % i])), i


@pytest.mark.parametrize("ta,tb", [("n", "n"), ("n", "t"), ("t", "n"), ("t", "t")])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_gemm_vs_numpy(ob, ta, tb, dtype):
    r = np.random.default_rng(3)
    m, n, k = 37, 29, 53
    A = F(r.standard_normal((k, m) if ta == "t" else (m, k)), dtype)
    B = F(r.standard_normal((n, k) if tb == "t" else (k, n)), dtype)
    C0 = F(r.standard_normal((m, n)), dtype)
    want = 0.7 * (A.T if ta == "t" else A).astype(np.float64) @ (B.T if tb == "t" else B).astype(np.float64) + 1.3 * C0
    got = ob.gemm(ta, tb, 0.7, A, B, 1.3, C0.copy(order="F"))
    assert rel_max(got, want) < (1e-5 if dtype == np.float32 else 1e-13)
    # beta = 0 must ignore (not propagate) what is in C
    Cn = F(np.full((m, n), np.nan), dtype)
    got = ob.gemm(ta, tb, 1.0, A, B, 0.0, Cn)
    assert np.isfinite(got).all()


# H, W, C, N, FH, FW, FC, K, stride, pad, dilate   (symmetric pads: torch-compatible)
TORCH_CASES = [
    (8, 9, 3, 2, 3, 3, 3, 4, 1, 1, 1),
    (9, 8, 4, 3, 3, 2, 4, 6, (2, 1), (1, 1, 0, 0), 1),
    (12, 11, 2, 2, 3, 3, 2, 3, (2, 3), (2, 2, 1, 1), (2, 1)),
    (7, 7, 6, 2, 1, 1, 6, 5, 1, 0, 1),
    (10, 10, 6, 2, 3, 3, 2, 9, 1, 1, 1),           # 3 filter groups (nnconv.m:144-161)
    (10, 9, 4, 2, 5, 3, 2, 4, (1, 2), (2, 2, 1, 1), 1),  # 2 groups, rectangular filter
    (32, 32, 3, 2, 5, 5, 3, 8, 1, 2, 1),           # benchmark configuration 1 geometry, reduced N and K
]


def _torch_conv(x, f, b, stride, pad4, dilate, groups):
    """x (H,W,C,N), f (FH,FW,FC,K) Fortran arrays -> torch tensors in NCHW with torch-H := MATLAB-W."""
    xt = torch.from_numpy(np.ascontiguousarray(x.T)).requires_grad_(True)   # (N,C,W,H)
    ft = torch.from_numpy(np.ascontiguousarray(f.T)).requires_grad_(True)   # (K,FC,FW,FH)
    bt = torch.from_numpy(b.copy()).requires_grad_(True)
    sy, sx = stride
    dy_, dx_ = dilate
    yt = torch.nn.functional.conv2d(xt, ft, bt, stride=(sx, sy), padding=(pad4[2], pad4[0]),
                                    dilation=(dx_, dy_), groups=groups)
    return xt, ft, bt, yt


@pytest.mark.parametrize("case", TORCH_CASES)
def test_conv_vs_torch_autograd_double(ob, case):
    H, W, C, N, FH, FW, FC, K, stride, pad, dilate = case
    g = ob.conv_geom((H, W, C, N), (FH, FW, FC, K), stride, pad, dilate)
    r = np.random.default_rng(5)
    x = F(r.standard_normal((H, W, C, N)), np.float64)
    f = F(r.standard_normal((FH, FW, FC, K)), np.float64)
    b = r.standard_normal(K)
    dy = F(r.standard_normal(ob.conv_out_shape(g)), np.float64)
    xt, ft, bt, yt = _torch_conv(x, f, b, ob._pair(stride), ob._quad(pad), ob._pair(dilate), C // FC)
    yt.backward(torch.from_numpy(np.ascontiguousarray(dy.T)))
    y = ob.conv_forward(x, f, b, g)
    assert rel_max(y, yt.detach().numpy().T) < 1e-12
    dx, df, db = ob.conv_backward(x, f, dy, g)
    assert rel_max(dx, xt.grad.numpy().T) < 1e-12
    assert rel_max(df, ft.grad.numpy().T) < 1e-12
    assert rel_max(db, bt.grad.numpy()) < 1e-12
    # float instantiation sits within float rounding of the same numbers
    dx32, df32, db32 = ob.conv_backward(F(x, np.float32), F(f, np.float32), F(dy, np.float32), g)
    assert rel_max(dx32, dx) < 2e-5 and rel_max(df32, df) < 2e-5 and rel_max(db32, db) < 2e-5


def _direct_gradients(x, f, dy, sy, sx, pt, pl, dly, dlx):
    """Loop-nest statement of the three gradients (no im2row, no GEMM), groups = 1."""
    H, W, C, N = x.shape
    FH, FW, FC, K = f.shape
    OH, OW = dy.shape[:2]
    dx = np.zeros_like(x)
    df = np.zeros_like(f)
    for n in range(N):
        for k in range(K):
            for ow in range(OW):
                for oh in range(OH):
                    d = dy[oh, ow, k, n]
                    for j in range(FW):
                        w = ow * sx + j * dlx - pl
                        if w < 0 or w >= W:
                            continue
                        for i in range(FH):
                            h = oh * sy + i * dly - pt
                            if h < 0 or h >= H:
                                continue
                            dx[h, w, :, n] += d * f[i, j, :, k]
                            df[i, j, :, k] += d * x[h, w, :, n]
    return dx, df, dy.sum(axis=(0, 1, 3))


@pytest.mark.parametrize("stride,pad,dilate", [((1, 1), (0, 2, 1, 0), (1, 1)), ((2, 1), (3, 0, 0, 2), (1, 2)), ((3, 2), (1, 2, 2, 1), (2, 2))])
def test_conv_backward_direct_loops_asymmetric_pad(ob, stride, pad, dilate):
    H, W, C, N, FH, FW, K = 7, 8, 2, 2, 3, 2, 3
    g = ob.conv_geom((H, W, C, N), (FH, FW, C, K), stride, pad, dilate)
    r = np.random.default_rng(6)
    x = F(r.standard_normal((H, W, C, N)), np.float64)
    f = F(r.standard_normal((FH, FW, C, K)), np.float64)
    dy = F(r.standard_normal(ob.conv_out_shape(g)), np.float64)
    dx, df, db = ob.conv_backward(x, f, dy, g)
    wdx, wdf, wdb = _direct_gradients(x, f, dy, stride[0], stride[1], pad[0], pad[2], dilate[0], dilate[1])
    assert rel_max(dx, wdx) < 1e-13 and rel_max(df, wdf) < 1e-13 and rel_max(db, wdb) < 1e-13


def test_adjoint_identities(ob):
    """<dzdy, conv(x+d) - conv(x)> = <dzdx, d>, and likewise for f and b (conv is bilinear)."""
    g = ob.conv_geom((9, 10, 4, 3), (3, 3, 2, 6), (2, 1), (1, 2, 0, 1), (1, 2))
    r = np.random.default_rng(8)
    x = F(r.standard_normal((9, 10, 4, 3)), np.float64)
    f = F(r.standard_normal((3, 3, 2, 6)), np.float64)
    b = r.standard_normal(6)
    dy = F(r.standard_normal(ob.conv_out_shape(g)), np.float64)
    dx, df, db = ob.conv_backward(x, f, dy, g)
    y0 = ob.conv_forward(x, f, b, g)
    d = F(r.standard_normal(x.shape), np.float64)
    assert abs((dy * (ob.conv_forward(F(x + d, np.float64), f, b, g) - y0)).sum() - (dx * d).sum()) < 1e-9
    d = F(r.standard_normal(f.shape), np.float64)
    assert abs((dy * (ob.conv_forward(x, F(f + d, np.float64), b, g) - y0)).sum() - (df * d).sum()) < 1e-9
    d = r.standard_normal(6)
    assert abs((dy * (ob.conv_forward(x, f, b + d, g) - y0)).sum() - (db * d).sum()) < 1e-9


def test_stride_is_subsampling_and_pad_is_cropping(ob):
    """nnconv.m:88-125: strided output = subsampled dense output; padded output cropped = unpadded; and
    the gradients agree when dzdy is zero-stuffed / zero-padded accordingly."""
    r = np.random.default_rng(9)
    x = F(r.standard_normal((9, 9, 2, 2)), np.float64)
    f = F(r.standard_normal((3, 3, 2, 3)), np.float64)
    b = r.standard_normal(3)
    g1 = ob.conv_geom(x.shape, f.shape, 1, 0, 1)
    g2 = ob.conv_geom(x.shape, f.shape, (2, 3), 0, 1)
    y1, y2 = ob.conv_forward(x, f, b, g1), ob.conv_forward(x, f, b, g2)
    assert rel_max(y2, y1[::2, ::3]) < 1e-14
    dy2 = F(r.standard_normal(y2.shape), np.float64)
    dy1 = F(np.zeros(y1.shape), np.float64)
    dy1[::2, ::3] = dy2
    for a, w in zip(ob.conv_backward(x, f, dy2, g2), ob.conv_backward(x, f, dy1, g1)):
        assert rel_max(a, w) < 1e-13
    gp = ob.conv_geom(x.shape, f.shape, 1, (1, 2, 2, 1), 1)
    yp = ob.conv_forward(x, f, b, gp)
    assert rel_max(yp[1:-2, 2:-1], y1) < 1e-14
    dyp = F(np.zeros(yp.shape), np.float64)
    dy1 = F(r.standard_normal(y1.shape), np.float64)
    dyp[1:-2, 2:-1] = dy1
    for a, w in zip(ob.conv_backward(x, f, dyp, gp), ob.conv_backward(x, f, dy1, g1)):
        assert rel_max(a, w) < 1e-13


def test_filter_groups_equal_block_diagonal_dense(ob):
    """nnconv.m:144-161: grouped filters = dense filters with the off-group blocks zeroed."""
    r = np.random.default_rng(10)
    x = F(r.standard_normal((7, 7, 6, 2)), np.float64)
    fg = F(r.standard_normal((3, 3, 2, 9)), np.float64)  # 3 groups, 3 filters each
    b = r.standard_normal(9)
    fd = F(np.zeros((3, 3, 6, 9)), np.float64)
    for gi in range(3):
        fd[:, :, 2 * gi:2 * gi + 2, 3 * gi:3 * gi + 3] = fg[:, :, :, 3 * gi:3 * gi + 3]
    gg = ob.conv_geom(x.shape, fg.shape, 1, 1, 1)
    gd = ob.conv_geom(x.shape, fd.shape, 1, 1, 1)
    assert rel_max(ob.conv_forward(x, fg, b, gg), ob.conv_forward(x, fd, b, gd)) < 1e-14
    dy = F(r.standard_normal(ob.conv_out_shape(gg)), np.float64)
    dxg, dfg, dbg = ob.conv_backward(x, fg, dy, gg)
    dxd, dfd, dbd = ob.conv_backward(x, fd, dy, gd)
    assert rel_max(dxg, dxd) < 1e-13 and rel_max(dbg, dbd) < 1e-13
    for gi in range(3):
        assert rel_max(dfg[:, :, :, 3 * gi:3 * gi + 3], dfd[:, :, 2 * gi:2 * gi + 2, 3 * gi:3 * gi + 3]) < 1e-13


def test_known_derivatives_of_a_four_by_four_ramp(ob):
    # 4x4 ramp, 3x3 ones filter, pad 1, dzdy = ones
    x = F(np.arange(1, 17, dtype=np.float32).reshape(4, 4, 1, 1, order="F"))
    f = F(np.ones((3, 3, 1, 1)))
    g = ob.conv_geom(x.shape, f.shape, 1, 1, 1)
    dx, df, db = ob.conv_backward(x, f, F(np.ones(ob.conv_out_shape(g))), g)
    assert list(dx.ravel(order="F")) == [4, 6, 6, 4, 6, 9, 9, 6, 6, 9, 9, 6, 4, 6, 6, 4]
    assert list(df.ravel(order="F")) == [54, 78, 63, 96, 136, 108, 90, 126, 99]
    assert list(db) == [16]


def test_out_mult_and_skipped_outputs(ob):
    r = np.random.default_rng(12)
    x = F(r.standard_normal((6, 6, 2, 2)), np.float64)
    f = F(r.standard_normal((3, 3, 2, 3)), np.float64)
    g = ob.conv_geom(x.shape, f.shape, 1, 1, 1)
    y0 = ob.conv_forward(x, f, None, g)
    base = F(r.standard_normal(y0.shape), np.float64)
    y = ob.conv_forward(x, f, None, g, y=base.copy(order="F"), out_mult=0.5, in_mult=2.0)
    assert rel_max(y, 0.5 * base + 2.0 * y0) < 1e-13
    dy = F(r.standard_normal(y0.shape), np.float64)
    dx, df, db = ob.conv_backward(x, f, dy, g, want=(False, True, False))
    assert dx is None and db is None and df is not None
