"""vl_nnconv with empty FILTERS (subsample + bias) and vl_nnconvt on the GPU, through the MEX-convention
front-end and the C ABI, against the CPU oracle.  Subsampling moves data and adds one bias: bit-exact.
Convolution transpose is the convolution products with exchanged roles: the convolution gate (2e-4)."""
import ctypes as C

import numpy as np
import pytest
import torch

from util import F, bits_equal, rel_max

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def vl():
    from matconvnet_amd import vlapi
    vlapi.lib()
    return vlapi


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(np.asfortranarray(a, dtype=np.float32).T)).cuda()


def host(t):
    return np.asfortranarray(t.detach().cpu().numpy().T)


def hw4(a, shape):
    return np.asarray(a).reshape(shape, order="F")


EMPTY = lambda: torch.empty((0,), dtype=torch.float32, device="cuda")

SUB = [  # (H, W, C, N, stride, pad)
    (9, 7, 3, 2, 1, 0),
    (9, 7, 3, 2, (2, 3), 0),
    (8, 8, 4, 1, 2, (1, 0, 2, 1)),
    (5, 6, 2, 3, (3, 1), (2, 2, 0, 3)),
    (56, 56, 64, 4, 2, 0),
    (1, 1, 5, 2, 4, 0),
]


@pytest.mark.parametrize("H,W,Cc,N,stride,pad", SUB)
def test_vl_nnconv_without_filters_is_subsample_plus_bias(vl, ob, H, W, Cc, N, stride, pad):
    r = np.random.default_rng(H * 7 + W)
    x = F(r.standard_normal((H, W, Cc, N)))
    b = r.standard_normal(Cc).astype(np.float32)
    opts = ("stride", list(np.atleast_1d(stride)), "pad", list(np.atleast_1d(pad)))
    y = vl.vl_nnconv(dev(x), EMPTY(), dev(b), *opts)
    want = ob.subsample_forward(x, b, stride, pad)
    assert bits_equal(hw4(host(y), want.shape), want)
    y0 = vl.vl_nnconv(dev(x), EMPTY(), EMPTY(), *opts)
    assert bits_equal(hw4(host(y0), want.shape), ob.subsample_forward(x, None, stride, pad))
    dy = F(r.standard_normal(want.shape))
    dx, df, db = vl.vl_nnconv(dev(x), EMPTY(), dev(b), dev(dy), *opts)
    assert df.numel() == 0
    assert bits_equal(hw4(host(dx), x.shape), ob.subsample_backward(x.shape, dy, stride, pad))
    assert rel_max(host(db).ravel(), dy.astype(np.float64).sum(axis=(0, 1, 3))) < 1e-5
    dx, df, db = vl.vl_nnconv(dev(x), EMPTY(), EMPTY(), dev(dy), *opts)
    assert db.numel() == 0 and dx.numel() == x.size


def test_subsample_c_abi_rejects_bad_arguments(capi):
    L = capi.lib()
    assert L.mcn_subsample_forward(None, None, None, None, 4, 4, 1, 1, 0, 1, 0, 0, 0, 0) == 7
    assert b"STRIDE" in L.mcn_last_error_message()
    assert L.mcn_subsample_backward(None, None, None, 4, 4, 1, 1, 1, 1, -1, 0, 0, 0) == 7
    oh, ow = C.c_int(), C.c_int()
    assert L.mcn_subsample_output_size(9, 7, 2, 3, 1, 0, 0, 2, C.byref(oh), C.byref(ow)) == 0
    assert (oh.value, ow.value) == ((9 + 1 - 1) // 2 + 1, (7 + 2 - 1) // 3 + 1)


def test_bias_add_c_abi(capi):
    r = np.random.default_rng(4)
    for shape in ((6, 5, 3, 2), (8, 8, 4, 3)):
        y = F(r.standard_normal(shape))
        b = r.standard_normal(shape[2]).astype(np.float32)
        yd, bd = capi.to_device(y), capi.to_device(b)
        capi.check(capi.lib().mcn_bias_add(capi.stream(), capi.ptr(yd), capi.ptr(bd), *shape))
        assert bits_equal(capi.to_host(yd), F(y + b.reshape(1, 1, -1, 1)))


CONVT = [  # (H, W, Cin, N, FH, FW, out channels per group, groups, upsample, crop)
    (5, 4, 4, 2, 3, 3, 3, 1, 2, (1, 0, 1, 1)),
    (6, 5, 6, 2, 4, 3, 2, 2, (2, 3), (0, 1, 2, 0)),
    (4, 4, 2, 1, 1, 1, 5, 1, 1, 0),
    (3, 3, 4, 3, 5, 5, 1, 4, 1, 2),
    (14, 14, 32, 4, 3, 3, 16, 1, 1, 1),   # upsample 1: every product runs on the matrix cores
    (14, 14, 32, 4, 4, 4, 16, 1, 2, 1),   # the FCN-style 2x upsampling layer
]


@pytest.mark.parametrize("H,W,Cin,N,FH,FW,Cog,groups,up,crop", CONVT)
def test_vl_nnconvt_forward_backward(vl, ob, H, W, Cin, N, FH, FW, Cog, groups, up, crop):
    r = np.random.default_rng(H + 10 * W + 100 * Cin)
    x = F(r.standard_normal((H, W, Cin, N)))
    f = F(r.standard_normal((FH, FW, Cog, Cin)) * 0.3)
    b = r.standard_normal(Cog * groups).astype(np.float32)
    opts = ("upsample", list(np.atleast_1d(up)), "crop", list(np.atleast_1d(crop)), "numGroups", groups)
    y = vl.vl_nnconvt(dev(x), dev(f), dev(b), *opts)
    want = ob.convt_forward(x, f, b, up, crop, groups)
    assert rel_max(hw4(host(y), want.shape), want) < 2e-4
    dy = F(r.standard_normal(want.shape))
    dx, df, db = vl.vl_nnconvt(dev(x), dev(f), dev(b), dev(dy), *opts)
    wdx, wdf, wdb = ob.convt_backward(x, f, dy, up, crop, groups)
    assert rel_max(hw4(host(dx), x.shape), wdx) < 2e-4
    assert rel_max(hw4(host(df), f.shape), wdf) < 2e-4
    assert rel_max(host(db).ravel(), wdb) < 2e-4
    # skipped outputs come back empty, like the MEX driver's
    dx, df, db = vl.vl_nnconvt(dev(x), dev(f), EMPTY(), dev(dy), *opts, "NoDerFilters")
    assert df.numel() == 0 and db.numel() == 0 and rel_max(hw4(host(dx), x.shape), wdx) < 2e-4


def test_vl_nnconvt_is_the_adjoint_of_vl_nnconv(vl):
    """<convt(x, f), z> = <x, conv(z, f)> with stride = upsample, pad = crop (bits/nnconv.cu:323-421)."""
    r = np.random.default_rng(12)
    x = F(r.standard_normal((6, 6, 8, 2)))
    f = F(r.standard_normal((3, 3, 5, 8)))
    y = vl.vl_nnconvt(dev(x), dev(f), EMPTY(), "upsample", 2, "crop", 1)
    z = torch.randn_like(y)
    back = vl.vl_nnconv(z, dev(f), EMPTY(), "stride", 2, "pad", 1)
    lhs, rhs = float((y.double() * z.double()).sum()), float((dev(x).double() * back.double()).sum())
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), 1.0)
