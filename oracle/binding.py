"""ctypes binding of the CPU oracle (liboracle.so) and of the compiled reference objects
(_ref/libmcnref.so).  TEST INFRASTRUCTURE ONLY.

Arrays are numpy, Fortran-ordered, shaped (H, W, C, N) exactly like MATLAB arrays, float32 or float64.
"""
import ctypes as C
import glob
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "liboracle.so")
REF_SO = os.path.join(HERE, "_ref", "libmcnref.so")


class ConvGeom(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "H", "W", "C", "N", "FH", "FW", "FC", "K", "strideY", "strideX",
        "padTop", "padBottom", "padLeft", "padRight", "dilateY", "dilateX")]


class PoolGeom(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "H", "W", "C", "N", "poolH", "poolW", "strideY", "strideX",
        "padTop", "padBottom", "padLeft", "padRight", "method")]


def build(reference="/root/reference"):
    """Compile liboracle.so and, when the reference tree is present, _ref/libmcnref.so."""
    subprocess.check_call(["make", "-C", HERE, "-s", "REFERENCE=" + reference])


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            build()
        _lib = C.CDLL(ORACLE_SO)
        _lib.oracle_num_threads.restype = C.c_int
    return _lib


def ref():
    """The compiled reference bridge, or None when it has not been built (e.g. on the GPU box if the
    prebuilt file is missing)."""
    global _ref
    if _ref is None and os.path.exists(REF_SO):
        _ref = C.CDLL(REF_SO)
    return _ref


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32", C.c_float
    if dtype == np.float64:
        return "f64", C.c_double
    raise TypeError("oracle supports float32 and float64 only, got %s" % dtype)


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def farray(a, dtype=None):
    """Fortran-ordered copy/view with an oracle dtype."""
    return np.asfortranarray(a, dtype=dtype or a.dtype)


def fempty(shape, dtype):
    return np.empty(shape, dtype=dtype, order="F")


def _pair(v):
    v = np.atleast_1d(v).astype(int).ravel()
    return (int(v[0]), int(v[0])) if v.size == 1 else (int(v[0]), int(v[1]))


def _quad(v):
    v = np.atleast_1d(v).astype(int).ravel()
    return (int(v[0]),) * 4 if v.size == 1 else tuple(int(t) for t in v[:4])


def conv_geom(xshape, fshape, stride=1, pad=0, dilate=1):
    """Geometry from MATLAB-style option values: stride [sy sx], pad [top bottom left right],
    dilate [dy dx] (vl_nnconv.cu:136-205)."""
    H, W, Cc, N = (list(xshape) + [1, 1, 1])[:4]
    FH, FW, FC, K = (list(fshape) + [1, 1, 1])[:4]
    sy, sx = _pair(stride)
    pt, pb, pl, pr = _quad(pad)
    dy, dx = _pair(dilate)
    return ConvGeom(H, W, Cc, N, FH, FW, FC, K, sy, sx, pt, pb, pl, pr, dy, dx)


def pool_geom(xshape, pool, stride=1, pad=0, method="max"):
    H, W, Cc, N = (list(xshape) + [1, 1, 1])[:4]
    ph, pw = _pair(pool)
    sy, sx = _pair(stride)
    pt, pb, pl, pr = _quad(pad)
    return PoolGeom(H, W, Cc, N, ph, pw, sy, sx, pt, pb, pl, pr, 0 if method == "max" else 1)


def conv_out_shape(g):
    return (lib().oracle_conv_out_h(C.byref(g)), lib().oracle_conv_out_w(C.byref(g)), g.K, g.N)


def pool_out_shape(g):
    return (lib().oracle_pool_out_h(C.byref(g)), lib().oracle_pool_out_w(C.byref(g)), g.C, g.N)


def num_threads():
    return lib().oracle_num_threads()


_blas_keepalive = []


def use_openblas(enable=True):
    """Route the oracle's GEMM to the ILP64 OpenBLAS that ships inside the numpy wheel (the role MKL
    plays for the reference).  Returns the library path used, or None."""
    L = lib()
    if not enable:
        L.oracle_set_sgemm(None)
        L.oracle_set_dgemm(None)
        return None
    pats = glob.glob(os.path.join(os.path.dirname(np.__file__), "..", "numpy.libs", "libscipy_openblas64_*.so"))
    for path in pats:
        try:
            bl = C.CDLL(path)
            s = C.cast(bl.scipy_sgemm_64_, C.c_void_p)
            d = C.cast(bl.scipy_dgemm_64_, C.c_void_p)
        except (OSError, AttributeError):
            continue
        _blas_keepalive.append(bl)
        L.oracle_set_sgemm(s)
        L.oracle_set_dgemm(d)
        return os.path.realpath(path)
    return None


def gemm(ta, tb, alpha, a, b, beta, c):
    """In-place column-major C = alpha*op(A)*op(B) + beta*C on Fortran-ordered 2-D arrays."""
    s, ct = _sfx(c.dtype)
    m, n = c.shape
    k = a.shape[0] if ta in "tT" else a.shape[1]
    fn = getattr(lib(), "oracle_gemm_" + s)
    fn.argtypes = [C.c_char, C.c_char, C.c_int64, C.c_int64, C.c_int64, ct, C.c_void_p, C.c_int64,
                   C.c_void_p, C.c_int64, ct, C.c_void_p, C.c_int64]
    fn(ta.encode(), tb.encode(), m, n, k, alpha, _p(a), a.shape[0], _p(b), b.shape[0], beta, _p(c), c.shape[0])
    return c


def im2row_forward(x, g):
    s, _ = _sfx(x.dtype)
    oh, ow, _, _ = conv_out_shape(g)
    st = fempty((oh * ow, g.FH * g.FW * g.C), x.dtype)
    getattr(lib(), "oracle_im2row_forward_" + s)(_p(st), _p(x), C.byref(g))
    return st


def im2row_backward(st, g):
    s, _ = _sfx(st.dtype)
    x = fempty((g.H, g.W, g.C), st.dtype)
    getattr(lib(), "oracle_im2row_backward_" + s)(_p(x), _p(st), C.byref(g))
    return x


def conv_forward(x, f, b, g, y=None, out_mult=0.0, in_mult=1.0):
    s, ct = _sfx(x.dtype)
    if y is None:
        y = np.zeros(conv_out_shape(g), dtype=x.dtype, order="F")
    fn = getattr(lib(), "oracle_conv_forward_" + s)
    fn.argtypes = [C.c_void_p, ct, C.c_void_p, ct, C.c_void_p, C.c_void_p, C.c_void_p]
    fn(_p(y), out_mult, _p(x), in_mult, _p(f), _p(b), C.byref(g))
    return y


def conv_backward(x, f, dy, g, want=(True, True, True)):
    s, _ = _sfx(dy.dtype)
    dx = fempty((g.H, g.W, g.C, g.N), dy.dtype) if want[0] else None
    df = fempty((g.FH, g.FW, g.FC, g.K), dy.dtype) if want[1] else None
    db = fempty((g.K,), dy.dtype) if want[2] else None
    fn = getattr(lib(), "oracle_conv_backward_" + s)
    fn.argtypes = [C.c_void_p] * 7
    fn(_p(dx), _p(df), _p(db), _p(x), _p(f), _p(dy), C.byref(g))
    return dx, df, db


def subsample_out_shape(xshape, stride=1, pad=0):
    H, W, Cc, N = (list(xshape) + [1, 1, 1])[:4]
    sy, sx = _pair(stride)
    pt, pb, pl, pr = _quad(pad)
    return ((H + pt + pb - 1) // sy + 1, (W + pl + pr - 1) // sx + 1, Cc, N)


def subsample_forward(x, b, stride=1, pad=0):
    """vl_nnconv(x, [], b, 'stride', s, 'pad', p): bits/nnsubsample.cu:36-117."""
    s, _ = _sfx(x.dtype)
    H, W, Cc, N = (list(x.shape) + [1, 1, 1])[:4]
    sy, sx = _pair(stride)
    pt, pb, pl, pr = _quad(pad)
    y = fempty(subsample_out_shape(x.shape, stride, pad), x.dtype)
    fn = getattr(lib(), "oracle_subsample_forward_" + s)
    fn.argtypes = [C.c_void_p] * 3 + [C.c_int] * 10
    fn(_p(y), _p(x), _p(b), H, W, Cc, N, sy, sx, pt, pb, pl, pr)
    return y


def taccum(alpha, a, beta, b):
    """vl_taccum(alpha, a, beta, b): matlab/src/vl_taccummex.cu:48-78."""
    s, ct = _sfx(a.dtype)
    y = fempty(a.shape, a.dtype)
    fn = getattr(lib(), "oracle_taccum_" + s)
    fn.argtypes = [C.c_void_p, ct, C.c_void_p, ct, C.c_void_p, C.c_size_t]
    fn(_p(y), alpha, _p(a), beta, _p(b), a.size)
    return y


def subsample_backward(xshape, dy, stride=1, pad=0):
    """dzdx of the same call (bits/nnsubsample.cu:125-165); dzdb is the per-channel sum of dzdy."""
    s, _ = _sfx(dy.dtype)
    H, W, Cc, N = (list(xshape) + [1, 1, 1])[:4]
    sy, sx = _pair(stride)
    pt, pb, pl, pr = _quad(pad)
    dx = fempty((H, W, Cc, N), dy.dtype)
    fn = getattr(lib(), "oracle_subsample_backward_" + s)
    fn.argtypes = [C.c_void_p] * 2 + [C.c_int] * 10
    fn(_p(dx), _p(dy), H, W, Cc, N, sy, sx, pt, pb, pl, pr)
    return dx


def convt_out_shape(xshape, fshape, upsample=1, crop=0, groups=1):
    """vl_nnconvt.cu:296-299."""
    H, W, Cc, N = (list(xshape) + [1, 1, 1])[:4]
    FH, FW, FC, K = (list(fshape) + [1, 1, 1])[:4]
    uy, ux = _pair(upsample)
    ct, cb, cl, cr = _quad(crop)
    return ((H - 1) * uy - (ct + cb) + FH, (W - 1) * ux - (cl + cr) + FW, FC * groups, N)


def convt_forward(x, f, b, upsample=1, crop=0, groups=1):
    """ConvolutionTransposeForward, bits/nnconv.cu:323-375: per image, the backward-data product of the
    convolution with stride = upsample and pad = crop, taking x as the output derivative; then the bias."""
    oshape = convt_out_shape(x.shape, f.shape, upsample, crop, groups)
    x4 = farray(x).reshape((list(x.shape) + [1, 1, 1])[:4], order="F")
    y = fempty(oshape, x.dtype)
    for n in range(oshape[3]):
        g = conv_geom(oshape[:3] + (1,), f.shape, upsample, crop, 1)
        dx, _, _ = conv_backward(None, f, farray(x4[:, :, :, n:n + 1]), g, want=(True, False, False))
        y[:, :, :, n] = dx[:, :, :, 0]
    if b is not None:
        y += np.asarray(b, dtype=x.dtype).reshape(1, 1, -1, 1)
    return farray(y)


def convt_backward(x, f, dy, upsample=1, crop=0, groups=1, want=(True, True, True)):
    """ConvolutionTransposeBackward, bits/nnconv.cu:381-421: dzdx = forward convolution of dzdy, dzdf = the
    filter derivative of that convolution with x in the role of its output derivative, dzdb = sums of dzdy."""
    dy4 = farray(dy).reshape((list(dy.shape) + [1, 1, 1])[:4], order="F")
    x4 = farray(x).reshape((list(x.shape) + [1, 1, 1])[:4], order="F")
    g = conv_geom(dy4.shape, f.shape, upsample, crop, 1)
    dx = conv_forward(dy4, f, None, g) if want[0] else None
    df = conv_backward(dy4, None, x4, g, want=(False, True, False))[1] if want[1] else None
    db = None
    if want[2]:
        db = conv_backward(None, None, dy4, conv_geom(dy4.shape, (1, 1, dy4.shape[2], dy4.shape[2])), want=(False, False, True))[2]
    return dx, df, db


def bnorm_forward(x, mult, bias, eps=1e-4, moments=None):
    s, ct = _sfx(x.dtype)
    H, W, Cc, N = (list(x.shape) + [1, 1, 1])[:4]
    y = fempty(x.shape, x.dtype)
    given = moments is not None
    mom = farray(moments, x.dtype).copy(order="F") if given else fempty((Cc, 2), x.dtype)
    fn = getattr(lib(), "oracle_bnorm_forward_" + s)
    fn.argtypes = [C.c_void_p] * 5 + [C.c_int] * 4 + [ct, C.c_int]
    fn(_p(y), _p(mom), _p(x), _p(mult), _p(bias), H, W, Cc, N, eps, int(given))
    return y, mom


def bnorm_backward(x, mult, dy, eps=1e-4, moments=None):
    s, ct = _sfx(x.dtype)
    H, W, Cc, N = (list(x.shape) + [1, 1, 1])[:4]
    dx = fempty(x.shape, x.dtype)
    dg = fempty((Cc,), x.dtype)
    db = fempty((Cc,), x.dtype)
    given = moments is not None
    mom = farray(moments, x.dtype).copy(order="F") if given else fempty((Cc, 2), x.dtype)
    fn = getattr(lib(), "oracle_bnorm_backward_" + s)
    fn.argtypes = [C.c_void_p] * 7 + [C.c_int] * 4 + [ct, C.c_int]
    fn(_p(dx), _p(dg), _p(db), _p(mom), _p(x), _p(mult), _p(dy), H, W, Cc, N, eps, int(given))
    return dx, dg, db, mom


def pool_forward(x, g):
    s, _ = _sfx(x.dtype)
    y = fempty(pool_out_shape(g), x.dtype)
    getattr(lib(), "oracle_pool_forward_" + s)(_p(y), _p(x), C.byref(g))
    return y


def pool_backward(x, dy, g, dx=None):
    """dzdx accumulated into `dx` (zeros when not given), as vl_nnpool does."""
    s, _ = _sfx(x.dtype)
    if dx is None:
        dx = np.zeros((g.H, g.W, g.C, g.N), dtype=x.dtype, order="F")
    getattr(lib(), "oracle_pool_backward_" + s)(_p(dx), _p(x), _p(dy), C.byref(g))
    return dx


def relu_forward(x):
    s, _ = _sfx(x.dtype)
    y = fempty(x.shape, x.dtype)
    fn = getattr(lib(), "oracle_relu_forward_" + s)
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    fn(_p(y), _p(x), x.size)
    return y


def relu_backward(x, dy):
    s, _ = _sfx(x.dtype)
    dx = fempty(x.shape, x.dtype)
    fn = getattr(lib(), "oracle_relu_backward_" + s)
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    fn(_p(dx), _p(x), _p(dy), x.size)
    return dx


def add(a, b):
    s, _ = _sfx(a.dtype)
    y = fempty(a.shape, a.dtype)
    fn = getattr(lib(), "oracle_sum_" + s)
    fn.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    fn(_p(y), _p(a), _p(b), a.size)
    return y


# ---------------------------------------------------------------------------------------------
# The compiled reference objects (present only where oracle/_ref has been built).
# ---------------------------------------------------------------------------------------------

def ref_pool_forward(x, g):
    s, _ = _sfx(x.dtype)
    y = fempty(pool_out_shape(g), x.dtype)
    fn = getattr(ref(), "ref_pool_forward_" + s)
    fn.argtypes = [C.c_void_p, C.c_void_p] + [C.c_int] * 13
    rc = fn(_p(y), _p(x), g.H, g.W, g.C, g.N, g.poolH, g.poolW, g.strideY, g.strideX,
            g.padTop, g.padBottom, g.padLeft, g.padRight, g.method)
    assert rc == 0, rc
    return y


def ref_pool_backward(x, dy, g):
    s, _ = _sfx(x.dtype)
    dx = np.zeros((g.H, g.W, g.C, g.N), dtype=x.dtype, order="F")
    fn = getattr(ref(), "ref_pool_backward_" + s)
    fn.argtypes = [C.c_void_p] * 3 + [C.c_int] * 13
    rc = fn(_p(dx), _p(x), _p(dy), g.H, g.W, g.C, g.N, g.poolH, g.poolW, g.strideY, g.strideX,
            g.padTop, g.padBottom, g.padLeft, g.padRight, g.method)
    assert rc == 0, rc
    return dx


def ref_bnorm_forward(x, mult, bias, eps=1e-4, moments=None):
    s, _ = _sfx(x.dtype)
    H, W, Cc, N = (list(x.shape) + [1, 1, 1])[:4]
    y = fempty(x.shape, x.dtype)
    given = moments is not None
    mom = farray(moments, x.dtype).copy(order="F") if given else fempty((Cc, 2), x.dtype)
    fn = getattr(ref(), "ref_bnorm_forward_" + s)
    fn.argtypes = [C.c_void_p] * 5 + [C.c_int] * 4 + [C.c_double, C.c_int]
    rc = fn(_p(y), _p(mom), _p(x), _p(mult), _p(bias), H, W, Cc, N, eps, int(given))
    assert rc == 0, rc
    return y, mom


def ref_bnorm_backward(x, mult, bias, dy, eps=1e-4, moments=None):
    s, _ = _sfx(x.dtype)
    H, W, Cc, N = (list(x.shape) + [1, 1, 1])[:4]
    dx = fempty(x.shape, x.dtype)
    dg = fempty((Cc,), x.dtype)
    db = fempty((Cc,), x.dtype)
    given = moments is not None
    mom = farray(moments, x.dtype).copy(order="F") if given else fempty((Cc, 2), x.dtype)
    fn = getattr(ref(), "ref_bnorm_backward_" + s)
    fn.argtypes = [C.c_void_p] * 8 + [C.c_int] * 4 + [C.c_double, C.c_int]
    rc = fn(_p(dx), _p(dg), _p(db), _p(mom), _p(x), _p(mult), _p(bias), _p(dy), H, W, Cc, N, eps, int(given))
    assert rc == 0, rc
    return dx, dg, db, mom


def ref_im2row_forward(x, g):
    s, _ = _sfx(x.dtype)
    oh, ow, _, _ = conv_out_shape(g)
    st = fempty((oh * ow, g.FH * g.FW * g.C), x.dtype)
    fn = getattr(ref(), "ref_im2row_forward_" + s)
    fn.argtypes = [C.c_void_p] * 2 + [C.c_int] * 13
    rc = fn(_p(st), _p(x), g.H, g.W, g.C, g.FH, g.FW, g.strideY, g.strideX,
            g.padTop, g.padBottom, g.padLeft, g.padRight, g.dilateY, g.dilateX)
    assert rc == 0, rc
    return st


def ref_im2row_backward(st, g):
    s, _ = _sfx(st.dtype)
    x = fempty((g.H, g.W, g.C), st.dtype)
    fn = getattr(ref(), "ref_im2row_backward_" + s)
    fn.argtypes = [C.c_void_p] * 2 + [C.c_int] * 13
    rc = fn(_p(x), _p(st), g.H, g.W, g.C, g.FH, g.FW, g.strideY, g.strideX,
            g.padTop, g.padBottom, g.padLeft, g.padRight, g.dilateY, g.dilateX)
    assert rc == 0, rc
    return x
