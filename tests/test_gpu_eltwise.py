"""GPU parity of the element-wise companions (ReLU, sum, scaled sum, fill): bit-exact against the oracle."""
import numpy as np
import pytest

from util import F, bits_equal

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 3, 4, 5, 255, 1024, 100003])
def test_relu_add_fill(capi, ob, n):
    r = np.random.default_rng(n)
    x = r.standard_normal(n).astype(np.float32)
    x[::7] = 0.0
    if n > 4:
        x[3] = np.nan
        x[4] = -0.0
    dy = r.standard_normal(n).astype(np.float32)
    xd, dyd = capi.to_device(x), capi.to_device(dy)
    assert bits_equal(capi.to_host(capi.relu_forward(xd)), ob.relu_forward(x))
    assert bits_equal(capi.to_host(capi.relu_backward(xd, dyd)), ob.relu_backward(x, dy))
    assert bits_equal(capi.to_host(capi.add(xd, dyd)), ob.add(x, dy))
    t = capi.empty((n,))
    capi.fill(t, 1.5)
    assert np.array_equal(capi.to_host(t), np.full(n, 1.5, np.float32))


def test_unaligned_views(capi, ob):
    """Pointers that are only 4-byte aligned take the scalar path."""
    import torch
    base = torch.randn(1001, device="cuda")
    x = base[1:]
    y = torch.empty(1001, device="cuda")[1:]
    capi.check(capi.lib().mcn_relu_forward(capi.stream(), capi.ptr(y), capi.ptr(x), x.numel()))
    assert torch.equal(y, torch.clamp_min(x, 0))


@pytest.mark.parametrize("n", [1, 5, 1024, 100003])
def test_taccum(capi, ob, n):
    """alpha*a + beta*b, out of place and in place, bit for bit the scal + axpy pair of the oracle."""
    r = np.random.default_rng(n + 1)
    a = r.standard_normal(n).astype(np.float32)
    b = r.standard_normal(n).astype(np.float32)
    want = ob.taccum(0.9, a, -0.0123, b)
    ad, bd = capi.to_device(a), capi.to_device(b)
    assert bits_equal(capi.to_host(capi.taccum(0.9, ad, -0.0123, bd)), want)
    capi.taccum(0.9, ad, -0.0123, bd, out=ad)
    assert bits_equal(capi.to_host(ad), want)


def test_vl_taccum_driver(ob):
    """The MEX conventions: a new array without options, the first array updated with 'InPlace'."""
    import torch
    from matconvnet_amd import vlapi as vl
    r = np.random.default_rng(4)
    a = F(r.standard_normal((6, 5, 4, 3)))
    b = F(r.standard_normal((6, 5, 4, 3)))
    dev = lambda v: torch.from_numpy(np.ascontiguousarray(v.transpose(3, 2, 1, 0))).cuda()
    host = lambda t: np.asfortranarray(t.cpu().numpy().transpose(3, 2, 1, 0))
    want = ob.taccum(0.5, a, 2.0, b)
    ad, bd = dev(a), dev(b)
    y = vl.vl_taccum(0.5, ad, 2.0, bd)
    assert bits_equal(host(y), want) and bits_equal(host(ad), a)
    same = vl.vl_taccum(0.5, ad, 2.0, bd, "inplace")
    assert same is ad and bits_equal(host(ad), want)
