"""vl_nnloss restated in numpy (matlab/vl_nnloss.m:136-317), statement by statement.  TEST INFRASTRUCTURE ONLY.

Arrays are (H, W, C, N) like MATLAB's; the arithmetic runs in the data type of x (float32 or float64), as MATLAB's
does for single / double inputs.

Pinned without running the reference (MATLAB code; no MATLAB here): tests/test_oracle_loss.py checks every loss
against a numerical derivative the way matlab/xtest/suite/nnloss.m:55-72 does, against closed forms (uniform scores
-> log C; derivative of softmaxlog sums to zero over the classes; hinge / error counts on hand-made inputs), that
null labels and zero instance weights remove an instance (nnloss.m:74-84), and against brute-force loops.
"""
import numpy as np

CATEGORICAL = ("classerror", "topkerror", "log", "softmaxlog", "mhinge", "mshinge")
BINARY = ("binaryerror", "binarylog", "logistic", "hinge")


def _prepare(x, c, loss, instance_weights):
    x = np.asarray(x)
    if x.ndim < 4:
        x = x.reshape(x.shape + (1,) * (4 - x.ndim))
    H, W, C, N = x.shape
    T = x.dtype.type
    c = np.asarray(c, dtype=np.float64)
    if c.size == N:                                   # form 1: one label per image (vl_nnloss.m:149-154)
        c = np.broadcast_to(c.reshape(1, 1, 1, N), (H, W, 1, N)).copy()
    elif c.ndim < 4:
        c = c.reshape(c.shape + (1,) * (4 - c.ndim))
    has_ignore = bool((c == 0).any())                 # :156
    assert c.shape[:2] == (H, W) and c.shape[3] == N  # :176-177
    iw = None
    if loss in CATEGORICAL:
        assert c.shape[2] == 1                        # :182
        if has_ignore:
            iw = (c[:, :, :1, :] != 0).astype(x.dtype)    # :184-187
    elif loss in BINARY:
        assert c.shape[2] == C                        # :192
        if has_ignore:
            iw = (c != 0).astype(x.dtype)             # :194-197
    else:
        raise ValueError("Unknown loss '%s'." % loss)
    if instance_weights is not None:                  # :203-211 (bsxfun broadcast to the size of c)
        w = np.asarray(instance_weights, dtype=x.dtype)
        if w.ndim < 4:
            w = w.reshape(w.shape + (1,) * (4 - w.ndim))
        iw = np.broadcast_to(w, c.shape).astype(x.dtype) if iw is None else (iw * w).astype(x.dtype)
    return x, c, iw, T


def _label_values(x, c):
    """x(ci): the score of each instance's label; a null label reads class 1 (uint64(c - 1) saturates at 0, :226)."""
    idx = np.maximum(c.astype(np.int64) - 1, 0)
    return np.take_along_axis(x, idx, axis=2), idx


def vl_nnloss(x, c, dzdy=None, loss="softmaxlog", instance_weights=None, normalise=True, top_k=5, threshold=0.0):
    loss = loss.lower()
    x, c, iw, T = _prepare(x, c, loss, instance_weights)
    H, W, C, N = x.shape
    if loss in ("log", "softmaxlog", "mhinge", "mshinge"):
        xc, idx = _label_values(x, c)
    if dzdy is None:                                                          # :229-271
        if loss == "classerror":
            chat = np.argmax(x, axis=2)[:, :, None, :] + 1                    # first maximum, like MATLAB's max
            t = (c != chat).astype(x.dtype)
        elif loss == "topkerror":
            order = np.argsort(-x, axis=2, kind="stable") + 1                 # sort(x, 3, 'descend') is stable
            t = (1 - (c == order[:, :, :top_k, :]).sum(axis=2, keepdims=True)).astype(x.dtype)
        elif loss == "log":
            t = -np.log(xc)
        elif loss == "softmaxlog":
            xmax = x.max(axis=2, keepdims=True)
            ex = np.exp(x - xmax)
            t = xmax + np.log(ex.sum(axis=2, keepdims=True, dtype=x.dtype)) - xc
        elif loss == "mhinge":
            t = np.maximum(T(0), T(1) - xc)
        elif loss == "mshinge":
            q = x.copy()
            np.put_along_axis(q, idx, -np.inf, axis=2)
            t = np.maximum(T(0), T(1) - xc + q.max(axis=2, keepdims=True))
        elif loss == "binaryerror":
            t = (np.sign(x - T(threshold)) != c).astype(x.dtype)
        elif loss == "binarylog":
            t = -np.log(c.astype(x.dtype) * (x - T(0.5)) + T(0.5))
        elif loss == "logistic":
            a = -c.astype(x.dtype) * x
            b = np.maximum(T(0), a)
            t = b + np.log(np.exp(-b) + np.exp(a - b))
        elif loss == "hinge":
            t = np.maximum(T(0), T(1) - c.astype(x.dtype) * x)
        t = t.astype(x.dtype)
        y = float((iw.ravel(order="F").astype(np.float64) * t.ravel(order="F")).sum()) if iw is not None else float(t.sum(dtype=np.float64))
        if normalise:                                                         # :269-271 (4-D input: N > 1; N = 1 divides by 1)
            y = y / N
        return T(y)
    dz = T(dzdy) if iw is None else (T(dzdy) * iw).astype(x.dtype)            # :275-277
    cc = c.astype(x.dtype)
    if loss in ("classerror", "topkerror", "binaryerror"):
        y = np.zeros_like(x)
    elif loss == "log":
        y = np.zeros_like(x)
        np.put_along_axis(y, idx, (-dz / np.maximum(xc, T(1e-8))) * np.ones_like(xc), axis=2)
    elif loss == "softmaxlog":
        xmax = x.max(axis=2, keepdims=True)
        ex = np.exp(x - xmax)
        y = ex / ex.sum(axis=2, keepdims=True, dtype=x.dtype)
        np.put_along_axis(y, idx, np.take_along_axis(y, idx, axis=2) - T(1), axis=2)
        y = dz * y
    elif loss == "mhinge":
        y = np.zeros_like(x)
        np.put_along_axis(y, idx, -dz * (xc < 1).astype(x.dtype), axis=2)
    elif loss == "mshinge":
        q = x.copy()
        np.put_along_axis(q, idx, -np.inf, axis=2)
        qi = np.argmax(q, axis=2)[:, :, None, :]
        Wt = dz * (xc - np.take_along_axis(x, qi, axis=2) < 1).astype(x.dtype)
        y = np.zeros_like(x)
        np.put_along_axis(y, idx, -Wt, axis=2)
        np.put_along_axis(y, qi, Wt * np.ones_like(xc), axis=2)
    elif loss == "binarylog":
        y = -dz / (x + (cc - T(1)) * T(0.5))
    elif loss == "logistic":
        y = -dz * cc / (T(1) + np.exp(cc * x))
    elif loss == "hinge":
        y = -dz * cc * (cc * x < 1).astype(x.dtype)
    y = y.astype(x.dtype)
    if normalise:                                                             # :313-315
        y = y / T(N)
    return np.asfortranarray(y)


def vl_nnsoftmax(x, dzdy=None):
    """matlab/vl_nnsoftmax.m:20-28, statement by statement.  Pinned by: rows sum to 1, shift invariance, the
    derivative against a numerical one, sum over the channels of dzdx = 0 (tests/test_oracle_loss.py)."""
    x = np.asarray(x)
    e = np.exp(x - x.max(axis=2, keepdims=True))
    y = e / e.sum(axis=2, keepdims=True, dtype=x.dtype)
    if dzdy is None:
        return np.asfortranarray(y.astype(x.dtype))
    dzdy = np.asarray(dzdy, dtype=x.dtype)
    return np.asfortranarray((y * (dzdy - (dzdy * y).sum(axis=2, keepdims=True, dtype=x.dtype))).astype(x.dtype))
