"""ctypes binding of the C ABI in include/mcn_hip.h (libmcn_hip.so).

Fails loudly when the library is missing: there is no fallback path.  Tensors are torch CUDA tensors used
purely as device buffers; a MATLAB array H x W x C x N (column-major) is a contiguous torch tensor of
shape (N, C, W, H).
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmcn_hip.so")

SUCCESS, UNSUPPORTED, DEVICE_ERROR, OUT_OF_MEMORY, OUT_OF_GPU_MEMORY, ILLEGAL_ARGUMENT, UNKNOWN = 0, 1, 2, 5, 6, 7, 8
CONV_FORWARD, CONV_BACKWARD_DATA, CONV_BACKWARD_FILTER, CONV_BACKWARD_BIAS = 0, 1, 2, 3
POOL_MAX, POOL_AVERAGE = 0, 1
BNORM_STATIC_SCRATCH_BYTES = 1 << 20   # MCN_BNORM_STATIC_SCRATCH_BYTES


class ConvGeom(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "H", "W", "C", "N", "FH", "FW", "FC", "K", "strideY", "strideX",
        "padTop", "padBottom", "padLeft", "padRight", "dilateY", "dilateX")]


class PoolGeom(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "H", "W", "C", "N", "poolH", "poolW", "strideY", "strideX",
        "padTop", "padBottom", "padLeft", "padRight", "method")]


class LossGeom(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("H", "W", "C", "N", "loss", "topK", "normalise")] + [("threshold", C.c_double)]


LOSSES = ("classerror", "topkerror", "log", "softmaxlog", "mhinge", "mshinge", "binaryerror", "binarylog", "logistic",
          "hinge")


class McnError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("mcn error %d: %s" % (code, message))
        self.code = code
        self.message = message


# every exported symbol of include/mcn_hip.h: (restype, argtypes)
_vp, _sz, _i, _f, _d = C.c_void_p, C.c_size_t, C.c_int, C.c_float, C.c_double
PROTOTYPES = {
    "mcn_last_error_message": (C.c_char_p, []),
    "mcn_error_name": (C.c_char_p, [_i]),
    "mcn_device_compute_units": (_i, []),
    "mcn_set_tunable": (_i, [C.c_char_p, _i]),
    "mcn_stream_beside": (_i, [_vp, _i]),
    "mcn_get_tunable": (_i, [C.c_char_p, C.POINTER(_i)]),
    "mcn_profile_begin": (_i, [C.c_char_p]),
    "mcn_profile_end": (_i, [C.POINTER(_i), C.POINTER(_d)]),
    "mcn_hbm_yardstick": (_i, [_vp, _vp, _vp, _sz, _i, _i, _i, _i, _i]),
    "mcn_mfma_yardstick": (_i, [_vp, _vp, _i, _i, C.POINTER(_d)]),
    "mcn_conv_output_size": (_i, [C.POINTER(ConvGeom), C.POINTER(_i), C.POINTER(_i)]),
    "mcn_conv_workspace_bytes": (_sz, [C.POINTER(ConvGeom), _i]),
    "mcn_conv_forward": (_i, [_vp, C.POINTER(ConvGeom), _vp, _f, _vp, _f, _vp, _vp, _vp, _sz]),
    "mcn_conv_forward_sums_groups": (_i, [C.POINTER(ConvGeom)]),
    "mcn_conv_forward_sums": (_i, [_vp, C.POINTER(ConvGeom), _vp, _vp, _vp, _vp, _sz, _vp, _sz, _vp, _sz]),
    "mcn_bnorm_forward_sums": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _d, _vp, _i]),
    "mcn_bnorm_mask_bits_supported": (_i, [_i, _i, _i, _i]),
    "mcn_bnorm_forward_sums_mask": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _d, _vp, _i]),
    "mcn_bnorm_backward_bits": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _d, _vp, _sz]),
    "mcn_conv_backward_data_masked_add_supported": (_i, [C.POINTER(ConvGeom)]),
    "mcn_conv_backward_data_masked_add": (_i, [_vp, C.POINTER(ConvGeom), _vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _sz]),
    "mcn_conv_backward_data": (_i, [_vp, C.POINTER(ConvGeom), _vp, _vp, _vp, _vp, _sz]),
    "mcn_taccum": (_i, [_vp, _vp, C.c_float, _vp, C.c_float, _vp, _sz]),
    "mcn_conv_backward_filter_partial_bytes": (_sz, [_vp]),
    "mcn_conv_backward_filter_plan": (_i, [_vp, _vp, _vp, _sz, _vp, _i, _vp]),
    "mcn_conv_backward_filter_partial": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz]),
    "mcn_conv_reduce_layout": (C.c_uint, [_vp, _i]),
    "mcn_conv_reduce_batch": (_i, [_vp, _vp, _i, C.c_uint]),
    "mcn_conv_packed_bytes": (_sz, [_vp, _i]),
    "mcn_conv_pack_filters": (_i, [_vp, _vp, _i, _vp, _vp, _sz]),
    "mcn_conv_pack_plan": (_i, [_vp, _i, _vp, _vp, _sz, _vp, _i, _vp]),
    "mcn_conv_pack_layout": (C.c_uint, [_vp, _i]),
    "mcn_conv_pack_batch": (_i, [_vp, _vp, _i, C.c_uint]),
    "mcn_conv_forward_packed": (_i, [_vp, _vp, _vp, C.c_float, _vp, C.c_float, _vp, _vp, _sz, _vp, _vp, _sz]),
    "mcn_conv_backward_data_packed": (_i, [_vp, _vp, _vp, C.c_float, _vp, _vp, _sz, _vp, _vp, _sz]),
    "mcn_sgd_momentum": (_i, [_vp, _vp, _vp, _vp, _sz, _vp, _vp] + [C.c_double] * 4 + [C.c_int]),
    "mcn_conv_backward_data_acc": (_i, [_vp, C.POINTER(ConvGeom), _vp, C.c_float, _vp, _vp, _vp, _sz]),
    "mcn_conv_backward_filter": (_i, [_vp, C.POINTER(ConvGeom), _vp, _vp, _vp, _vp, _sz]),
    "mcn_conv_backward_bias": (_i, [_vp, C.POINTER(ConvGeom), _vp, _vp, _vp, _sz]),
    "mcn_conv_backward_filter_bias": (_i, [_vp, C.POINTER(ConvGeom), _vp, _vp, _vp, _vp, _vp, _sz]),
    "mcn_subsample_output_size": (_i, [_i, _i, _i, _i, _i, _i, _i, _i, C.POINTER(_i), C.POINTER(_i)]),
    "mcn_subsample_forward": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i]),
    "mcn_subsample_backward": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i]),
    "mcn_bias_add": (_i, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "mcn_bnorm_workspace_bytes": (_sz, [_i, _i, _i, _i]),
    "mcn_bnorm_forward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _d, _i, _vp, _sz]),
    "mcn_bnorm_forward_fused": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _d, _i, _vp, _sz]),
    "mcn_bnorm_backward": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _d, _i, _vp, _sz]),
    "mcn_bnorm_backward_static": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _d, _i]),
    "mcn_bnorm_backward_masked": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _d, _vp, _sz]),
    "mcn_bnorm_backward_relu": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _d, _vp, _sz]),
    "mcn_pool_output_size": (_i, [C.POINTER(PoolGeom), C.POINTER(_i), C.POINTER(_i)]),
    "mcn_pool_forward": (_i, [_vp, C.POINTER(PoolGeom), _vp, _vp]),
    "mcn_pool_backward": (_i, [_vp, C.POINTER(PoolGeom), _vp, _vp, _vp, _i]),
    "mcn_relu_forward": (_i, [_vp, _vp, _vp, _sz]),
    "mcn_relu_backward": (_i, [_vp, _vp, _vp, _vp, _sz]),
    "mcn_relu_forward_leaky": (_i, [_vp, _vp, _vp, _sz, _d]),
    "mcn_relu_backward_leaky": (_i, [_vp, _vp, _vp, _vp, _sz, _d]),
    "mcn_add": (_i, [_vp, _vp, _vp, _vp, _sz]),
    "mcn_fill": (_i, [_vp, _vp, _f, _sz]),
    "mcn_softmax_forward": (_i, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "mcn_softmax_backward": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    "mcn_loss_workspace_bytes": (_sz, [C.POINTER(LossGeom)]),
    "mcn_loss_forward": (_i, [_vp, C.POINTER(LossGeom), _vp, _vp, _vp, _sz, _vp, _sz, _vp, _sz]),
    "mcn_loss_backward": (_i, [_vp, C.POINTER(LossGeom), _vp, _vp, _vp, _sz, _vp, _sz, _d]),
    "mcn_conv_forward_f64": (_i, [_vp, C.POINTER(ConvGeom), _vp, _d, _vp, _d, _vp, _vp]),
    "mcn_conv_backward_data_f64": (_i, [_vp, C.POINTER(ConvGeom), _vp, _vp, _vp]),
    "mcn_conv_backward_filter_f64": (_i, [_vp, C.POINTER(ConvGeom), _vp, _vp, _vp]),
    "mcn_conv_backward_bias_f64": (_i, [_vp, C.POINTER(ConvGeom), _vp, _vp]),
    "mcn_bnorm_forward_f64": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _d, _i, _vp, _sz]),
    "mcn_bnorm_backward_f64": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _d, _i, _vp, _sz]),
    "mcn_pool_forward_f64": (_i, [_vp, C.POINTER(PoolGeom), _vp, _vp]),
    "mcn_pool_backward_f64": (_i, [_vp, C.POINTER(PoolGeom), _vp, _vp, _vp, _i]),
    "mcn_subsample_forward_f64": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i]),
    "mcn_subsample_backward_f64": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i]),
    "mcn_bias_add_f64": (_i, [_vp, _vp, _vp, _i, _i, _i, _i]),
    "mcn_taccum_f64": (_i, [_vp, _vp, _d, _vp, _d, _vp, _sz]),
}

_lib = None


def lib():
    """The loaded library.  Raises if it has not been built: no fallback exists."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -m matconvnet_amd.build` (hipcc, gfx950)" % LIB_PATH)
        # torch first: it brings a HIP runtime of its own, and device tensors are shared with it only when that
        # runtime is the one already in the process when this library's dependency on libamdhip64 is resolved
        import torch  # noqa: F401
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise McnError(rc, lib().mcn_last_error_message().decode())


def set_tunable(name, value):
    check(lib().mcn_set_tunable(name.encode(), int(value)))


def get_tunable(name):
    v = C.c_int(0)
    check(lib().mcn_get_tunable(name.encode(), C.byref(v)))
    return v.value


def profile_begin(kernel_name):
    check(lib().mcn_profile_begin(kernel_name.encode()))


def profile_end():
    """(bracketed launches, sum of their durations in ms)"""
    n, ms = C.c_int(0), C.c_double(0.0)
    check(lib().mcn_profile_end(C.byref(n), C.byref(ms)))
    return n.value, ms.value


def _pair(v):
    v = np.atleast_1d(v).astype(int).ravel()
    return (int(v[0]), int(v[0])) if v.size == 1 else (int(v[0]), int(v[1]))


def _quad(v):
    v = np.atleast_1d(v).astype(int).ravel()
    return (int(v[0]),) * 4 if v.size == 1 else tuple(int(t) for t in v[:4])


def conv_geom(xshape, fshape, stride=1, pad=0, dilate=1):
    """Shapes are MATLAB-style (H, W, C, N) / (FH, FW, FC, K)."""
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
    return PoolGeom(H, W, Cc, N, ph, pw, sy, sx, pt, pb, pl, pr, POOL_MAX if method == "max" else POOL_AVERAGE)


def conv_out_shape(g):
    oh, ow = C.c_int(0), C.c_int(0)
    check(lib().mcn_conv_output_size(C.byref(g), C.byref(oh), C.byref(ow)))
    return (oh.value, ow.value, g.K, g.N)


def pool_out_shape(g):
    oh, ow = C.c_int(0), C.c_int(0)
    check(lib().mcn_pool_output_size(C.byref(g), C.byref(oh), C.byref(ow)))
    return (oh.value, ow.value, g.C, g.N)


# ---------------------------------------------------------------------------------------------------
# device-buffer helpers (torch is plumbing: allocation, host<->device copies, the stream handle)
# ---------------------------------------------------------------------------------------------------

def _torch():
    import torch
    return torch


def to_device(a, dtype=np.float32):
    """numpy (H,W,C,N) array in any order -> contiguous CUDA tensor (float32, or float64 on request) of shape
    reversed(a.shape)."""
    torch = _torch()
    f = np.asfortranarray(a, dtype=dtype)
    return torch.from_numpy(np.ascontiguousarray(f.T)).cuda()


def to_host(t, dtype=None):
    """CUDA tensor of shape (N,C,W,H) -> Fortran-ordered numpy array (H,W,C,N)."""
    a = t.detach().cpu().numpy().T
    return np.asfortranarray(a, dtype=dtype or a.dtype)


def empty(mshape, fill=None, like=None):
    """Device buffer for a MATLAB-shaped array (H,W,C,N,...), float32 or of the data type of `like`."""
    torch = _torch()
    shape = tuple(reversed([int(s) for s in mshape]))
    dtype = like.dtype if like is not None else torch.float32
    if fill is None:
        return torch.empty(shape, dtype=dtype, device="cuda")
    return torch.full(shape, float(fill), dtype=dtype, device="cuda")


def _is64(*tensors):
    """True when the tensors are double precision (all of them: mixed types are refused, as
    vl::impl::check_tensor_compatibility does, bits/data.hpp:260-266)."""
    torch = _torch()
    kinds = {t.dtype for t in tensors if t is not None}
    if len(kinds) > 1:
        raise TypeError("tensors of different data types: %s" % sorted(str(k) for k in kinds))
    return kinds == {torch.float64}


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def stream():
    return C.c_void_p(_torch().cuda.current_stream().cuda_stream)


class Workspace:
    """Grow-only device scratch buffer, the role of vl::Context::getWorkspace."""

    def __init__(self):
        self.buf = None

    def get(self, nbytes):
        torch = _torch()
        nbytes = int(nbytes)
        if nbytes == 0:
            return None, 0
        if self.buf is None or self.buf.numel() < nbytes:
            self.buf = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        return C.c_void_p(self.buf.data_ptr()), self.buf.numel()


_ws = Workspace()


# ---------------------------------------------------------------------------------------------------
# thin call wrappers (device tensors in, device tensors out)
# ---------------------------------------------------------------------------------------------------

def conv_forward(x, f, b, g, y=None, out_mult=0.0, in_mult=1.0, ws=None):
    ws = ws or _ws
    if y is None:
        y = empty(conv_out_shape(g), like=x)
    if _is64(x, f, b, y):
        check(lib().mcn_conv_forward_f64(stream(), C.byref(g), ptr(y), out_mult, ptr(x), in_mult, ptr(f), ptr(b)))
        return y
    wp, wn = ws.get(lib().mcn_conv_workspace_bytes(C.byref(g), CONV_FORWARD))
    check(lib().mcn_conv_forward(stream(), C.byref(g), ptr(y), out_mult, ptr(x), in_mult, ptr(f), ptr(b), wp, wn))
    return y


def conv_forward_sums_groups(g):
    """Partial sums per channel mcn_conv_forward_sums writes for this geometry; 0: no such form."""
    return int(lib().mcn_conv_forward_sums_groups(C.byref(g)))


def conv_forward_sums(x, f, g, packed=None, ws=None):
    """y = conv(x, f) and, from the same launch, partial sums of y and y^2 per channel: (y, sums[K][groups][2] in double)."""
    import torch
    ws = ws or _ws
    groups = conv_forward_sums_groups(g)
    y = empty(conv_out_shape(g), like=x)
    K = int(g.K)
    sums = torch.zeros(max(K * groups * 2, 1), dtype=torch.float64, device="cuda")
    wp, wn = ws.get(lib().mcn_conv_workspace_bytes(C.byref(g), CONV_FORWARD))
    pk, pkn = (ptr(packed), packed.numel() * packed.element_size()) if packed is not None else (None, 0)
    check(lib().mcn_conv_forward_sums(stream(), C.byref(g), ptr(y), ptr(x), ptr(f), pk, pkn, ptr(sums), sums.numel() * 8, wp, wn))
    return y, sums.view(K, max(groups, 1), 2)


def bnorm_forward_sums(x, g, b, sums, residual=None, relu=False, eps=1e-4):
    """Batch normalisation (with optional shortcut sum and ReLU) that takes its channel sums from `sums`."""
    H, W, Cc, N = _hwcn(x)
    y = empty((H, W, Cc, N))
    mom = empty((Cc, 2))
    check(lib().mcn_bnorm_forward_sums(stream(), ptr(y), ptr(mom), ptr(x), ptr(g), ptr(b), ptr(residual), int(relu),
                                       H, W, Cc, N, eps, ptr(sums), int(sums.shape[1])))
    return y, mom


def bnorm_forward_sums_mask(x, g, b, sums, residual=None, eps=1e-4):
    """mcn_bnorm_forward_sums with the ReLU on, which also writes one bit per element of y: (y, mask words, moments)."""
    import torch
    H, W, Cc, N = _hwcn(x)
    y = empty((H, W, Cc, N))
    mom = empty((Cc, 2))
    bits = torch.zeros((H * W * Cc * N + 31) // 32, dtype=torch.int32, device="cuda")
    check(lib().mcn_bnorm_forward_sums_mask(stream(), ptr(y), ptr(bits), ptr(mom), ptr(x), ptr(g), ptr(b), ptr(residual),
                                            H, W, Cc, N, eps, ptr(sums), int(sums.shape[1])))
    return y, bits, mom


def bnorm_backward_bits(x, g, dy, bits, moments, eps=1e-4, ws=None):
    ws = ws or _ws
    H, W, Cc, N = _hwcn(x)
    dx, dg, db = empty((H, W, Cc, N)), empty((Cc,)), empty((Cc,))
    wp, wn = ws.get(lib().mcn_bnorm_workspace_bytes(H, W, Cc, N))
    check(lib().mcn_bnorm_backward_bits(stream(), ptr(dx), ptr(dg), ptr(db), ptr(moments), ptr(x), ptr(g), ptr(dy), ptr(bits),
                                        H, W, Cc, N, eps, wp, wn))
    return dx, dg, db


def conv_backward_data_masked_add(f, dy, g, addend, bits, packed=None, ws=None):
    """dzdx = conv backward-data + (bit ? addend : addend*0)."""
    ws = ws or _ws
    dx = empty((g.H, g.W, g.C, g.N))
    wp, wn = ws.get(lib().mcn_conv_workspace_bytes(C.byref(g), CONV_BACKWARD_DATA))
    pk, pkn = (ptr(packed), packed.numel() * packed.element_size()) if packed is not None else (None, 0)
    check(lib().mcn_conv_backward_data_masked_add(stream(), C.byref(g), ptr(dx), ptr(f), pk, pkn, ptr(dy), ptr(addend), ptr(bits), wp, wn))
    return dx


def conv_backward(x, f, dy, g, want=(True, True, True), ws=None):
    ws = ws or _ws
    L = lib()
    dx = df = db = None
    if _is64(x, f, dy):
        if want[0]:
            dx = empty((g.H, g.W, g.C, g.N), like=dy)
            check(L.mcn_conv_backward_data_f64(stream(), C.byref(g), ptr(dx), ptr(f), ptr(dy)))
        if want[1]:
            df = empty((g.FH, g.FW, g.FC, g.K), like=dy)
            check(L.mcn_conv_backward_filter_f64(stream(), C.byref(g), ptr(df), ptr(x), ptr(dy)))
        if want[2]:
            db = empty((g.K,), like=dy)
            check(L.mcn_conv_backward_bias_f64(stream(), C.byref(g), ptr(db), ptr(dy)))
        return dx, df, db
    if want[0]:
        dx = empty((g.H, g.W, g.C, g.N))
        wp, wn = ws.get(L.mcn_conv_workspace_bytes(C.byref(g), CONV_BACKWARD_DATA))
        check(L.mcn_conv_backward_data(stream(), C.byref(g), ptr(dx), ptr(f), ptr(dy), wp, wn))
    if want[1]:
        df = empty((g.FH, g.FW, g.FC, g.K))
        wp, wn = ws.get(L.mcn_conv_workspace_bytes(C.byref(g), CONV_BACKWARD_FILTER))
        check(L.mcn_conv_backward_filter(stream(), C.byref(g), ptr(df), ptr(x), ptr(dy), wp, wn))
    if want[2]:
        db = empty((g.K,))
        wp, wn = ws.get(L.mcn_conv_workspace_bytes(C.byref(g), CONV_BACKWARD_BIAS))
        check(L.mcn_conv_backward_bias(stream(), C.byref(g), ptr(db), ptr(dy), wp, wn))
    return dx, df, db


def conv_backward_filter_bias(x, dy, g, ws=None):
    """(dzdf, dzdb) by one call (include/mcn_hip.h: mcn_conv_backward_filter_bias)."""
    ws = ws or _ws
    L = lib()
    df, db = empty((g.FH, g.FW, g.FC, g.K)), empty((g.K,))
    need = max(L.mcn_conv_workspace_bytes(C.byref(g), CONV_BACKWARD_FILTER), L.mcn_conv_workspace_bytes(C.byref(g), CONV_BACKWARD_BIAS))
    wp, wn = ws.get(need)
    check(L.mcn_conv_backward_filter_bias(stream(), C.byref(g), ptr(df), ptr(db), ptr(x), ptr(dy), wp, wn))
    return df, db


def conv_backward_data_acc(dx, mult, f, dy, g, ws=None):
    """dx = mult*dx + dzdx, in place (include/mcn_hip.h: mcn_conv_backward_data_acc)."""
    ws = ws or _ws
    L = lib()
    wp, wn = ws.get(L.mcn_conv_workspace_bytes(C.byref(g), CONV_BACKWARD_DATA))
    check(L.mcn_conv_backward_data_acc(stream(), C.byref(g), ptr(dx), float(mult), ptr(f), ptr(dy), wp, wn))
    return dx


class PackJob(C.Structure):
    """mcn_conv_pack_job of include/mcn_hip.h (opaque)."""
    _fields_ = [("opaque", C.c_ulonglong * 10)]


def conv_packed_bytes(g, product):
    return lib().mcn_conv_packed_bytes(C.byref(g), product)


def conv_pack_filters(f, g, product):
    """The filters packed ahead for one product (a uint8 device tensor; None when the product reads none)."""
    n = conv_packed_bytes(g, product)
    if n == 0:
        return None
    packed = _torch().empty(n, dtype=_torch().uint8, device="cuda")
    check(lib().mcn_conv_pack_filters(stream(), C.byref(g), product, ptr(f), ptr(packed), n))
    return packed


def conv_pack_many(layers):
    """layers: [(f, g, product)].  One buffer and ONE launch for all of them (mcn_conv_pack_plan / _layout / _batch);
    returns the views [(packed or None)] in the same order."""
    torch = _torch()
    L = lib()
    sizes = [conv_packed_bytes(g, product) for _, g, product in layers]
    total = sum(sizes)
    arena = torch.empty(max(total, 16), dtype=torch.uint8, device="cuda")
    jobs = (PackJob * 256)()
    n_jobs, at, views = 0, 0, []
    for (f, g, product), size in zip(layers, sizes):
        view = arena[at:at + size] if size else None
        views.append(view)
        if size:
            got = C.c_int(0)
            check(L.mcn_conv_pack_plan(C.byref(g), product, ptr(f), ptr(view), size,
                                       C.byref(jobs, n_jobs * C.sizeof(PackJob)), 256 - n_jobs, C.byref(got)))
            n_jobs += got.value
        at += size
    blocks = L.mcn_conv_pack_layout(jobs, n_jobs)
    host = np.frombuffer(jobs, dtype=np.uint8, count=n_jobs * C.sizeof(PackJob)).copy()
    device_jobs = torch.from_numpy(host).cuda() if n_jobs else None
    check(L.mcn_conv_pack_batch(stream(), ptr(device_jobs), n_jobs, blocks))
    torch.cuda.synchronize()   # (device_jobs must outlive the launch)
    return views


class ReduceJob(C.Structure):
    """mcn_conv_reduce_job of include/mcn_hip.h (opaque)."""
    _fields_ = [("opaque", C.c_ulonglong * 6)]


def conv_backward_filter_deferred(layers):
    """layers: [(x, dy, g)].  The filter gradients of all of them with ONE launch for the sums over reduction splits
    (mcn_conv_backward_filter_partial + mcn_conv_reduce_layout / _batch); layers whose geometry has no deferred form
    go through mcn_conv_backward_filter.  Returns the gradients in order."""
    torch = _torch()
    L = lib()
    jobs = (ReduceJob * 256)()
    n_jobs, outs, keep = 0, [], []
    for x, dy, g in layers:
        df = empty((g.FH, g.FW, g.FC, g.K))
        outs.append(df)
        size = L.mcn_conv_backward_filter_partial_bytes(C.byref(g))
        if size == 0:
            wp, wn = _ws.get(L.mcn_conv_workspace_bytes(C.byref(g), CONV_BACKWARD_FILTER))
            check(L.mcn_conv_backward_filter(stream(), C.byref(g), ptr(df), ptr(x), ptr(dy), wp, wn))
            continue
        partials = torch.empty(size, dtype=torch.uint8, device="cuda")
        keep.append(partials)
        got = C.c_int(0)
        check(L.mcn_conv_backward_filter_plan(C.byref(g), ptr(df), ptr(partials), size,
                                              C.byref(jobs, n_jobs * C.sizeof(ReduceJob)), 256 - n_jobs, C.byref(got)))
        n_jobs += got.value
        check(L.mcn_conv_backward_filter_partial(stream(), C.byref(g), ptr(df), ptr(x), ptr(dy), ptr(partials), size))
    blocks = L.mcn_conv_reduce_layout(jobs, n_jobs)
    host = np.frombuffer(jobs, dtype=np.uint8, count=n_jobs * C.sizeof(ReduceJob)).copy()
    device_jobs = torch.from_numpy(host).cuda() if n_jobs else None
    check(L.mcn_conv_reduce_batch(stream(), ptr(device_jobs), n_jobs, blocks))
    torch.cuda.synchronize()   # (device_jobs and the partial banks must outlive the launch)
    return outs


def conv_forward_packed(x, f, packed, b, g, y=None, out_mult=0.0, in_mult=1.0, ws=None):
    ws = ws or _ws
    if y is None:
        y = empty(conv_out_shape(g))
    wp, wn = ws.get(lib().mcn_conv_workspace_bytes(C.byref(g), CONV_FORWARD))
    check(lib().mcn_conv_forward_packed(stream(), C.byref(g), ptr(y), out_mult, ptr(x), in_mult, ptr(f), ptr(packed),
                                        packed.numel() if packed is not None else 0, ptr(b), wp, wn))
    return y


def conv_backward_data_packed(dx, mult, f, packed, dy, g, ws=None):
    ws = ws or _ws
    L = lib()
    wp, wn = ws.get(L.mcn_conv_workspace_bytes(C.byref(g), CONV_BACKWARD_DATA))
    check(L.mcn_conv_backward_data_packed(stream(), C.byref(g), ptr(dx), float(mult), ptr(f), ptr(packed),
                                          packed.numel() if packed is not None else 0, ptr(dy), wp, wn))
    return dx


def _hwcn(t):
    s = list(reversed(t.shape))
    return (s + [1, 1, 1])[:4]


def bnorm_forward(x, g, b, eps=1e-4, moments=None, ws=None):
    ws = ws or _ws
    H, W, Cc, N = _hwcn(x)
    y = empty((H, W, Cc, N), like=x)
    given = moments is not None
    mom = moments if given else empty((Cc, 2), like=x)
    if _is64(x, g, b, moments):
        check(lib().mcn_bnorm_forward_f64(stream(), ptr(y), ptr(mom), ptr(x), ptr(g), ptr(b), H, W, Cc, N, eps, int(given),
                                          None, 0))
        return y, mom
    wp, wn = ws.get(lib().mcn_bnorm_workspace_bytes(H, W, Cc, N))
    check(lib().mcn_bnorm_forward(stream(), ptr(y), ptr(mom), ptr(x), ptr(g), ptr(b), H, W, Cc, N, eps, int(given), wp, wn))
    return y, mom


def bnorm_forward_fused(x, g, b, residual=None, relu=False, eps=1e-4, ws=None):
    ws = ws or _ws
    H, W, Cc, N = _hwcn(x)
    y = empty((H, W, Cc, N))
    mom = empty((Cc, 2))
    wp, wn = ws.get(lib().mcn_bnorm_workspace_bytes(H, W, Cc, N))
    check(lib().mcn_bnorm_forward_fused(stream(), ptr(y), ptr(mom), ptr(x), ptr(g), ptr(b), ptr(residual), int(relu),
                                        H, W, Cc, N, eps, 0, wp, wn))
    return y, mom


def bnorm_backward(x, g, dy, eps=1e-4, moments=None, ws=None, want_moments=True):
    ws = ws or _ws
    H, W, Cc, N = _hwcn(x)
    dx = empty((H, W, Cc, N), like=x)
    dg = empty((Cc,), like=x)
    db = empty((Cc,), like=x)
    given = moments is not None
    mom = moments if given else (empty((Cc, 2), like=x) if want_moments else None)
    if _is64(x, g, dy, moments):
        wp, wn = (None, 0) if mom is not None else ws.get(2 * Cc * 8)
        check(lib().mcn_bnorm_backward_f64(stream(), ptr(dx), ptr(dg), ptr(db), ptr(mom), ptr(x), ptr(g), ptr(dy),
                                           H, W, Cc, N, eps, int(given), wp, wn))
        return dx, dg, db, mom
    wp, wn = ws.get(lib().mcn_bnorm_workspace_bytes(H, W, Cc, N))
    check(lib().mcn_bnorm_backward(stream(), ptr(dx), ptr(dg), ptr(db), ptr(mom), ptr(x), ptr(g), ptr(dy),
                                   H, W, Cc, N, eps, int(given), wp, wn))
    return dx, dg, db, mom


def bnorm_backward_static(x, g, dy, eps=1e-4, moments=None, out=None):
    """mcn_bnorm_backward_static: the partial sums live in the library's own device array.  `out` = (dx, dg, db, mom)
    allocated by the caller beforehand, so that the call itself is made with nothing allocated around it."""
    H, W, Cc, N = _hwcn(x)
    given = moments is not None
    if out is None:
        out = (empty((H, W, Cc, N)), empty((Cc,)), empty((Cc,)), moments if given else empty((Cc, 2)))
    dx, dg, db, mom = out
    check(lib().mcn_bnorm_backward_static(stream(), ptr(dx), ptr(dg), ptr(db), ptr(mom), ptr(x), ptr(g), ptr(dy),
                                          H, W, Cc, N, eps, int(given)))
    return dx, dg, db, mom


def bnorm_backward_relu(x, g, b, dy, moments, eps=1e-4, ws=None):
    """Derivative of ReLU(bnorm(x)) given dz/d(ReLU output) and the forward pass's moments."""
    ws = ws or _ws
    H, W, Cc, N = _hwcn(x)
    dx = empty((H, W, Cc, N))
    dg = empty((Cc,))
    db = empty((Cc,))
    wp, wn = ws.get(lib().mcn_bnorm_workspace_bytes(H, W, Cc, N))
    check(lib().mcn_bnorm_backward_relu(stream(), ptr(dx), ptr(dg), ptr(db), ptr(moments), ptr(x), ptr(g), ptr(b),
                                        ptr(dy), H, W, Cc, N, eps, wp, wn))
    return dx, dg, db


def bnorm_backward_masked(x, g, dy, mask_source, moments, eps=1e-4, ws=None):
    """bnorm derivative of dy*[mask_source > 0]; also returns that masked derivative."""
    ws = ws or _ws
    H, W, Cc, N = _hwcn(x)
    dx, masked = empty((H, W, Cc, N)), empty((H, W, Cc, N))
    dg, db = empty((Cc,)), empty((Cc,))
    wp, wn = ws.get(lib().mcn_bnorm_workspace_bytes(H, W, Cc, N))
    check(lib().mcn_bnorm_backward_masked(stream(), ptr(dx), ptr(dg), ptr(db), ptr(moments), ptr(x), ptr(g), ptr(dy),
                                          ptr(mask_source), ptr(masked), H, W, Cc, N, eps, wp, wn))
    return dx, dg, db, masked


def pool_forward(x, g):
    y = empty(pool_out_shape(g), like=x)
    fn = lib().mcn_pool_forward_f64 if _is64(x) else lib().mcn_pool_forward
    check(fn(stream(), C.byref(g), ptr(y), ptr(x)))
    return y


def pool_backward(x, dy, g, dx=None):
    """dx given: accumulate into it (vl::nn::Pooling::backward contract); else a fresh write-only output."""
    acc = dx is not None
    if dx is None:
        dx = empty((g.H, g.W, g.C, g.N), like=dy)
    fn = lib().mcn_pool_backward_f64 if _is64(x, dy, dx) else lib().mcn_pool_backward
    check(fn(stream(), C.byref(g), ptr(dx), ptr(x), ptr(dy), int(acc)))
    return dx


def softmax_forward(x):
    H, W, Cc, N = _hwcn(x)
    y = _torch().empty_like(x)
    check(lib().mcn_softmax_forward(stream(), ptr(y), ptr(x), H, W, Cc, N))
    return y


def softmax_backward(x, dzdy):
    H, W, Cc, N = _hwcn(x)
    dx = _torch().empty_like(x)
    check(lib().mcn_softmax_backward(stream(), ptr(dx), ptr(x), ptr(dzdy), H, W, Cc, N))
    return dx


def loss_geom(xshape, loss="softmaxlog", top_k=5, normalise=True, threshold=0.0):
    H, W, Cc, N = (list(xshape) + [1, 1, 1])[:4]
    return LossGeom(H, W, Cc, N, LOSSES.index(loss.lower()), top_k, int(bool(normalise)), threshold)


def loss_forward(x, c, g, instance_weights=None, ws=None):
    """vl_nnloss(x, c, [], ...): the loss as a one-element device tensor."""
    ws = ws or _ws
    y = empty((1,))
    wp, wn = ws.get(lib().mcn_loss_workspace_bytes(C.byref(g)))
    check(lib().mcn_loss_forward(stream(), C.byref(g), ptr(y), ptr(x), ptr(c), c.numel(), ptr(instance_weights),
                                 0 if instance_weights is None else instance_weights.numel(), wp, wn))
    return y


def loss_backward(x, c, dzdy, g, instance_weights=None):
    """vl_nnloss(x, c, dzdy, ...): dzdx."""
    dx = empty(tuple(reversed(x.shape)))
    check(lib().mcn_loss_backward(stream(), C.byref(g), ptr(dx), ptr(x), ptr(c), c.numel(), ptr(instance_weights),
                                  0 if instance_weights is None else instance_weights.numel(), float(dzdy)))
    return dx


def relu_forward(x, leak=None):
    y = _torch().empty_like(x)
    if leak is None:
        check(lib().mcn_relu_forward(stream(), ptr(y), ptr(x), x.numel()))
    else:
        check(lib().mcn_relu_forward_leaky(stream(), ptr(y), ptr(x), x.numel(), float(leak)))
    return y


def relu_backward(x, dy, leak=None):
    dx = _torch().empty_like(x)
    if leak is None:
        check(lib().mcn_relu_backward(stream(), ptr(dx), ptr(x), ptr(dy), x.numel()))
    else:
        check(lib().mcn_relu_backward_leaky(stream(), ptr(dx), ptr(x), ptr(dy), x.numel(), float(leak)))
    return dx


SGD_CHUNK = 1024   # MCN_SGD_CHUNK of include/mcn_hip.h


def sgd_arena_layout(counts):
    """Offsets (in floats) of parameters of the given element counts inside an arena whose parameters occupy whole
    chunks, the total number of chunks, and the chunk -> parameter table (numpy int16)."""
    offsets, chunk_param, at = [], [], 0
    for p, n in enumerate(counts):
        offsets.append(at)
        k = (n + SGD_CHUNK - 1) // SGD_CHUNK
        chunk_param += [p] * k
        at += k * SGD_CHUNK
    assert len(counts) < 32768
    return offsets, len(chunk_param), np.asarray(chunk_param, dtype=np.int16)


def sgd_momentum(value, state, der, chunk_param, rates, learning_rate, weight_decay, momentum, der_scale=1.0,
                 nesterov=False):
    """In-place SGD step over parameter arenas (include/mcn_hip.h: mcn_sgd_momentum).  value, state, der: float32
    device tensors of chunks*SGD_CHUNK elements; chunk_param: int16 device tensor; rates: float64 device tensor
    [params][2] of (learningRate, weightDecay) multipliers."""
    chunks = chunk_param.numel()
    assert value.numel() == state.numel() == der.numel() == chunks * SGD_CHUNK
    check(lib().mcn_sgd_momentum(stream(), ptr(value), ptr(state), ptr(der), chunks, ptr(chunk_param), ptr(rates),
                                 float(learning_rate), float(weight_decay), float(momentum), float(der_scale),
                                 int(bool(nesterov))))


def taccum(alpha, a, beta, b, out=None):
    """alpha*a + beta*b (include/mcn_hip.h: mcn_taccum); out may be a."""
    y = _torch().empty_like(a) if out is None else out
    check(lib().mcn_taccum(stream(), ptr(y), float(alpha), ptr(a), float(beta), ptr(b), a.numel()))
    return y


def add(a, b):
    y = _torch().empty_like(a)
    check(lib().mcn_add(stream(), ptr(y), ptr(a), ptr(b), a.numel()))
    return y


def fill(t, value):
    check(lib().mcn_fill(stream(), ptr(t), float(value), t.numel()))
    return t
