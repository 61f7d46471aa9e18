"""Pins oracle/loss.py (the numpy restatement of matlab/vl_nnloss.m) without the reference: numerical derivatives as
in matlab/xtest/suite/nnloss.m:55-72, closed forms, null labels / zero weights (nnloss.m:74-84), brute-force loops."""
import numpy as np
import pytest

from oracle import loss as ol

WITH_DERIVATIVE = ["log", "softmaxlog", "mhinge", "mshinge", "binarylog", "logistic", "hinge"]


def _inputs(loss, seed, null=False, dtype=np.float64):
    """The inputs of nnloss.m:getx (h = 4, w = 5, 3 classes / 5 attributes, 3 images)."""
    r = np.random.default_rng(seed)
    h, w, classes, attributes, images = 4, 5, 3, 5, 3
    if loss in ol.CATEGORICAL:
        c = r.integers(1, classes + 1, (h, w, 1, images)).astype(np.float64)
        weights = r.random((h, w)) / (h * w)
        depth = classes
    else:
        c = np.sign(r.standard_normal((h, w, attributes, images)))
        weights = r.random((h, w, attributes)) / (h * w * attributes)
        depth = attributes
    if loss == "log":
        x = r.random((h, w, depth, images)) * 0.6 + 0.2
        x = x / x.sum(axis=2, keepdims=True)
    elif loss == "binarylog":
        x = r.random((h, w, depth, images)) * 0.6 + 0.2
    else:
        x = r.standard_normal((h, w, depth, images))
    if null:
        c = c * (r.standard_normal(c.shape) > 0)
    return x.astype(dtype), c, weights, float(r.standard_normal())


@pytest.mark.parametrize("loss", WITH_DERIVATIVE)
@pytest.mark.parametrize("weighed", [False, True])
@pytest.mark.parametrize("null", [False, True])
def test_numerical_derivative(loss, weighed, null):
    x, c, weights, dzdy = _inputs(loss, 5, null)
    kw = dict(loss=loss, instance_weights=weights if weighed else None)
    dzdx = ol.vl_nnloss(x, c, dzdy, **kw)
    r = np.random.default_rng(6)
    worst = 0.0
    for _ in range(40):
        i = tuple(int(r.integers(0, s)) for s in x.shape)
        xc = x[i]
        if loss in ("mhinge", "mshinge", "hinge") and abs(abs(xc) - 1) < 1e-3:
            continue
        d = 1e-6
        xp, xm = x.copy(), x.copy()
        xp[i] += d
        xm[i] -= d
        num = (float(ol.vl_nnloss(xp, c, None, **kw)) - float(ol.vl_nnloss(xm, c, None, **kw))) / (2 * d) * dzdy
        worst = max(worst, abs(num - dzdx[i]))
    assert worst < 1e-5 * max(1.0, np.abs(dzdx).max()) + 1e-7


def test_softmaxlog_closed_forms():
    C, N = 7, 4
    x = np.zeros((1, 1, C, N))
    c = np.array([1, 3, 7, 2], dtype=np.float64)
    # uniform scores: the loss of every instance is log C; the sum is divided by N
    assert abs(float(ol.vl_nnloss(x, c, None, loss="softmaxlog")) - np.log(C)) < 1e-12
    assert abs(float(ol.vl_nnloss(x, c, None, loss="softmaxlog", normalise=False)) - N * np.log(C)) < 1e-12
    d = ol.vl_nnloss(x, c, 1.0, loss="softmaxlog")
    assert np.abs(d.sum(axis=2)).max() < 1e-15                       # softmax - onehot sums to zero over the classes
    assert abs(d[0, 0, 0, 0] - (1 / C - 1) / N) < 1e-15 and abs(d[0, 0, 1, 0] - (1 / C) / N) < 1e-15
    # invariance to a shift of the scores of an instance
    r = np.random.default_rng(1)
    x = r.standard_normal((3, 2, C, N))
    cc = r.integers(1, C + 1, (3, 2, 1, N)).astype(np.float64)
    assert abs(float(ol.vl_nnloss(x, cc, None)) - float(ol.vl_nnloss(x + 100.0, cc, None))) < 1e-10


def test_error_counts_by_hand():
    x = np.zeros((1, 1, 4, 3))
    x[0, 0, :, 0] = [0.1, 0.9, 0.3, 0.2]     # prediction 2
    x[0, 0, :, 1] = [0.5, 0.5, 0.1, 0.0]     # tie: the first maximum (class 1) is the prediction
    x[0, 0, :, 2] = [0.0, 0.1, 0.2, 0.3]     # prediction 4
    c = np.array([2.0, 2.0, 1.0])
    assert float(ol.vl_nnloss(x, c, None, loss="classerror", normalise=False)) == 2.0     # images 2 and 3 are wrong
    assert float(ol.vl_nnloss(x, c, None, loss="topkerror", top_k=2, normalise=False)) == 1.0   # image 3: class 1 is last
    assert float(ol.vl_nnloss(x, c, None, loss="topkerror", top_k=4, normalise=False)) == 0.0
    assert float(ol.vl_nnloss(x, c, None, loss="classerror")) == pytest.approx(2.0 / 3)
    assert not ol.vl_nnloss(x, c, 1.0, loss="classerror").any()
    # attribute losses
    xa = np.array([0.5, -0.5, 2.0, -3.0]).reshape(1, 1, 4, 1)
    ca = np.array([1.0, 1.0, -1.0, -1.0]).reshape(1, 1, 4, 1)
    assert float(ol.vl_nnloss(xa, ca, None, loss="binaryerror")) == 2.0
    assert float(ol.vl_nnloss(xa, ca, None, loss="hinge")) == pytest.approx(0.5 + 1.5 + 3.0 + 0.0)
    assert float(ol.vl_nnloss(xa, ca, None, loss="logistic")) == pytest.approx(np.log1p(np.exp(-ca * xa)).sum())


@pytest.mark.parametrize("loss", ol.CATEGORICAL + ol.BINARY)
def test_null_labels_and_zero_weights_remove_instances(loss):
    x, c, weights, dzdy = _inputs(loss, 9, null=True)
    y = float(ol.vl_nnloss(x, c, None, loss=loss, normalise=False))
    # brute force over the instances that count
    total = 0.0
    H, W, D, N = x.shape
    for n in range(N):
        for w in range(W):
            for h in range(H):
                if loss in ol.CATEGORICAL:
                    if c[h, w, 0, n] == 0:
                        continue
                    one = ol.vl_nnloss(x[h:h + 1, w:w + 1, :, n:n + 1], c[h:h + 1, w:w + 1, :, n:n + 1], None, loss=loss, normalise=False)
                    total += float(one)
                else:
                    for d in range(D):
                        if c[h, w, d, n] == 0:
                            continue
                        one = ol.vl_nnloss(x[h:h + 1, w:w + 1, d:d + 1, n:n + 1], c[h:h + 1, w:w + 1, d:d + 1, n:n + 1], None, loss=loss, normalise=False)
                        total += float(one)
    assert abs(y - total) < 1e-9 * max(1.0, abs(total))
    assert float(ol.vl_nnloss(x, c, None, loss=loss, instance_weights=np.zeros_like(weights))) == 0.0
    d = ol.vl_nnloss(x, c, dzdy, loss=loss)
    skipped = np.broadcast_to(c == 0, x.shape)
    assert not d[skipped].any()


def test_one_label_per_image_is_broadcast_over_the_pixels():
    r = np.random.default_rng(2)
    x = r.standard_normal((3, 2, 5, 4))
    c = r.integers(1, 6, 4).astype(np.float64)
    full = np.broadcast_to(c.reshape(1, 1, 1, 4), (3, 2, 1, 4))
    assert float(ol.vl_nnloss(x, c, None)) == float(ol.vl_nnloss(x, full, None))
    assert np.array_equal(ol.vl_nnloss(x, c, 0.5), ol.vl_nnloss(x, full, 0.5))


def test_softmax_properties_and_numerical_derivative():
    r = np.random.default_rng(4)
    x = r.standard_normal((3, 4, 6, 2))
    y = ol.vl_nnsoftmax(x)
    assert np.abs(y.sum(axis=2) - 1).max() < 1e-14 and (y > 0).all()
    assert np.abs(ol.vl_nnsoftmax(x + 7.5) - y).max() < 1e-14
    assert np.abs(ol.vl_nnsoftmax(np.zeros((1, 1, 5, 1))) - 0.2).max() < 1e-16
    dzdy = r.standard_normal(x.shape)
    dzdx = ol.vl_nnsoftmax(x, dzdy)
    assert np.abs(dzdx.sum(axis=2)).max() < 1e-14
    for _ in range(30):
        i = tuple(int(r.integers(0, s)) for s in x.shape)
        xp, xm = x.copy(), x.copy()
        xp[i] += 1e-6
        xm[i] -= 1e-6
        num = ((ol.vl_nnsoftmax(xp) - ol.vl_nnsoftmax(xm)) / 2e-6 * dzdy).sum()
        assert abs(num - dzdx[i]) < 1e-8
