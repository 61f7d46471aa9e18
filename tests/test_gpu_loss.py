"""GPU parity, vl_nnloss: the HIP kernels through the C ABI against the numpy restatement of matlab/vl_nnloss.m.
Gates: error counts exact; the other losses and all derivatives 1e-5 (max|diff|/max|ref|: expf / logf of the device
against numpy's), the oracle run in float32 like the device."""
import numpy as np
import pytest

from oracle import loss as ol
from util import F, rel_max

pytestmark = pytest.mark.gpu

SHAPES = [(4, 5, 3, 3), (1, 1, 1000, 32), (1, 1, 10, 1), (7, 3, 21, 2), (100, 90, 5, 2)]   # the last: a thread per vector


def _inputs(loss, shape, seed, null):
    r = np.random.default_rng(seed)
    H, W, D, N = shape
    if loss in ol.CATEGORICAL:
        c = r.integers(1, D + 1, (H, W, 1, N)).astype(np.float32)
    else:
        c = np.sign(r.standard_normal(shape)).astype(np.float32)
    if loss == "log":
        x = r.random(shape) * 0.6 + 0.2
        x = x / x.sum(axis=2, keepdims=True)
    elif loss == "binarylog":
        x = r.random(shape) * 0.6 + 0.2
    else:
        x = r.standard_normal(shape) * 2
    if null:
        c = c * (r.standard_normal(c.shape) > 0)
    return F(x), F(c), float(r.standard_normal())


@pytest.mark.parametrize("loss", ol.CATEGORICAL + ol.BINARY)
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("null", [False, True])
def test_value_and_derivative(capi, loss, shape, null):
    x, c, dzdy = _inputs(loss, shape, 3, null)
    g = capi.loss_geom(shape, loss)
    xd, cd = capi.to_device(x), capi.to_device(c)
    y = float(capi.to_host(capi.loss_forward(xd, cd, g))[0])
    want = float(ol.vl_nnloss(x, c, None, loss=loss))
    if loss in ("classerror", "topkerror", "binaryerror"):
        assert abs(y - want) <= 1e-6 * max(1.0, abs(want))
    else:
        assert abs(y - want) <= 1e-5 * max(1.0, abs(want))
    dx = capi.to_host(capi.loss_backward(xd, cd, dzdy, g))
    wdx = ol.vl_nnloss(x, c, dzdy, loss=loss)
    assert dx.shape == wdx.shape
    if wdx.any():
        assert rel_max(dx, wdx) < 1e-5
    else:
        assert not dx.any()


@pytest.mark.parametrize("loss", ["softmaxlog", "mshinge", "classerror", "logistic", "hinge"])
def test_instance_weights_and_options(capi, loss):
    shape = (6, 5, 4, 3)
    x, c, dzdy = _inputs(loss, shape, 4, True)
    r = np.random.default_rng(5)
    H, W, D, N = shape
    label_shape = (H, W, 1, N) if loss in ol.CATEGORICAL else shape
    for weights in (r.random(label_shape[:2] + ((1,) if loss in ol.CATEGORICAL else (D,))), r.random(label_shape), np.array([0.25])):
        weights = F(weights)
        g = capi.loss_geom(shape, loss, normalise=False)
        wd = capi.to_device(weights)
        y = float(capi.to_host(capi.loss_forward(capi.to_device(x), capi.to_device(c), g, instance_weights=wd))[0])
        want = float(ol.vl_nnloss(x, c, None, loss=loss, instance_weights=weights, normalise=False))
        assert abs(y - want) <= 1e-5 * max(1.0, abs(want))
        dx = capi.to_host(capi.loss_backward(capi.to_device(x), capi.to_device(c), dzdy, g, instance_weights=wd))
        wdx = ol.vl_nnloss(x, c, dzdy, loss=loss, instance_weights=weights, normalise=False)
        assert (rel_max(dx, wdx) < 1e-5) if wdx.any() else (not dx.any())


def test_one_label_per_image_top_k_and_threshold(capi):
    r = np.random.default_rng(6)
    x = F(r.standard_normal((1, 1, 50, 16)))
    c = F(r.integers(1, 51, 16))
    xd, cd = capi.to_device(x), capi.to_device(c)
    for k in (1, 5, 50):
        y = float(capi.to_host(capi.loss_forward(xd, cd, capi.loss_geom(x.shape, "topkerror", top_k=k)))[0])
        assert y == float(ol.vl_nnloss(x, c, None, loss="topkerror", top_k=k))
    y1 = float(capi.to_host(capi.loss_forward(xd, cd, capi.loss_geom(x.shape, "topkerror", top_k=1)))[0])
    ye = float(capi.to_host(capi.loss_forward(xd, cd, capi.loss_geom(x.shape, "classerror")))[0])
    assert y1 == ye                                            # distinct scores: top-1 error is the class error
    # ties: the first maximum is the prediction, a stable descending sort ranks the classes
    xt = F(np.round(r.standard_normal((2, 3, 6, 4))))
    ct = F(r.integers(1, 7, (2, 3, 1, 4)))
    for loss, k in (("classerror", 5), ("topkerror", 2), ("topkerror", 3)):
        y = float(capi.to_host(capi.loss_forward(capi.to_device(xt), capi.to_device(ct), capi.loss_geom(xt.shape, loss, top_k=k)))[0])
        assert y == float(ol.vl_nnloss(xt, ct, None, loss=loss, top_k=k))
    xa = F(r.standard_normal((3, 3, 4, 2)))
    ca = F(np.sign(r.standard_normal((3, 3, 4, 2))))
    y = float(capi.to_host(capi.loss_forward(capi.to_device(xa), capi.to_device(ca), capi.loss_geom(xa.shape, "binaryerror", threshold=0.3)))[0])
    assert y == float(ol.vl_nnloss(xa, ca, None, loss="binaryerror", threshold=0.3))


def test_argument_errors(capi):
    x = capi.to_device(np.zeros((2, 2, 3, 4)))
    with pytest.raises(capi.McnError):
        capi.loss_forward(x, capi.to_device(np.ones(5)), capi.loss_geom((2, 2, 3, 4)))          # neither N nor H*W*N labels
    with pytest.raises(capi.McnError):
        capi.loss_forward(x, capi.to_device(np.ones(4)), capi.loss_geom((2, 2, 3, 4), "hinge"))   # one label per element
    g = capi.loss_geom((2, 2, 3, 4))
    g.loss = 17
    with pytest.raises(capi.McnError):
        capi.loss_forward(x, capi.to_device(np.ones(4)), g)


def test_front_end_vl_nnloss(vl):
    """vl_nnloss with the reference's argument conventions (matlab/vl_nnloss.m:129-142): positional dzdy, options by
    name without regard to case, labels and weights from the host or the device."""
    import torch
    r = np.random.default_rng(8)
    shape = (4, 5, 3, 3)
    x = F(r.standard_normal(shape))
    c = r.integers(0, 4, (4, 5, 1, 3)).astype(np.float64)       # (zeros: skipped instances)
    w = r.random((4, 5))
    dev = lambda a, dt=np.float32: torch.from_numpy(np.ascontiguousarray(np.asfortranarray(a, dtype=dt).T)).cuda()
    host = lambda a: torch.from_numpy(np.ascontiguousarray(np.asfortranarray(a, dtype=np.float64).T))
    y = vl.vl_nnloss(dev(x), host(c))
    assert tuple(y.shape) == (1, 1) and y.is_cuda
    assert abs(float(y) - float(ol.vl_nnloss(x, c, None))) < 1e-5
    y = vl.vl_nnloss(dev(x), dev(c), "LOSS", "mshinge", "instanceweights", host(w), "normalise", 0.0)
    assert abs(float(y) - float(ol.vl_nnloss(x, c, None, loss="mshinge", instance_weights=w, normalise=False))) < 1e-5
    y = vl.vl_nnloss(dev(x), host(c), torch.empty((0,), dtype=torch.float64), "loss", "topkerror", "topK", 2.0)
    assert float(y) == float(ol.vl_nnloss(x, c, None, loss="topkerror", top_k=2))
    dx = vl.vl_nnloss(dev(x), host(c), 0.7, "loss", "softmaxlog", "instanceWeights", dev(w))
    want = ol.vl_nnloss(x, c, 0.7, loss="softmaxlog", instance_weights=w)
    got = np.asfortranarray(dx.detach().cpu().numpy().T)
    assert got.shape == want.shape and rel_max(got, want) < 1e-5
    for args, message in [((dev(x), host(c), "loss", "bogus"), "Unknown loss 'bogus'."),
                          ((dev(x), host(c), "frobnicate", 1.0), "Unknown option 'frobnicate'."),
                          ((dev(x),), "There are less than two arguments.")]:
        with pytest.raises(vl.VlError) as e:
            vl.vl_nnloss(*args)
        assert e.value.message == message, e.value.message
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnloss(dev(x, np.float64), host(c))
    assert e.value.code == 1


@pytest.mark.parametrize("shape", [(1, 1, 1000, 32), (4, 5, 3, 3), (1, 1, 1, 4), (100, 90, 5, 2)])
def test_softmax(capi, shape):
    r = np.random.default_rng(9)
    x = F(r.standard_normal(shape) * 3)
    dzdy = F(r.standard_normal(shape))
    xd = capi.to_device(x)
    y = capi.to_host(capi.softmax_forward(xd)).reshape(shape, order="F")
    assert rel_max(y, ol.vl_nnsoftmax(x)) < 1e-5 and np.abs(y.sum(axis=2) - 1).max() < 1e-5
    dx = capi.to_host(capi.softmax_backward(xd, capi.to_device(dzdy))).reshape(shape, order="F")
    want = ol.vl_nnsoftmax(x, dzdy)
    assert (rel_max(dx, want) < 1e-5) if shape[2] > 1 else (np.abs(dx).max() < 1e-6)


def test_front_end_vl_nnsoftmax(vl):
    import torch
    r = np.random.default_rng(10)
    x, dzdy = F(r.standard_normal((3, 2, 7, 4))), F(r.standard_normal((3, 2, 7, 4)))
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a.T)).cuda()
    y = vl.vl_nnsoftmax(dev(x))
    assert rel_max(np.asfortranarray(y.cpu().numpy().T), ol.vl_nnsoftmax(x)) < 1e-5
    dx = vl.vl_nnsoftmax(dev(x), dev(dzdy))
    assert rel_max(np.asfortranarray(dx.cpu().numpy().T), ol.vl_nnsoftmax(x, dzdy)) < 1e-5
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnsoftmax(dev(x), dev(dzdy[:, :, :3]))
    assert e.value.message == "X and DZDY do not have the same number of elements."
