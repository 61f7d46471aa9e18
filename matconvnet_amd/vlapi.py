"""ctypes binding of the C++ operator layer (libmcn_vl.so): the MATLAB-style entry points

    y                        = vl_nnconv(x, f, b, 'pad', p, 'stride', s, ...)
    dzdx, dzdf, dzdb         = vl_nnconv(x, f, b, dzdy, ...)            (f empty: subsample + bias)
    y / dzdx, dzdf, dzdb     = vl_nnconvt(x, f, b[, dzdy], 'upsample', u, 'crop', c, 'numGroups', g)
    y[, moments]             = vl_nnbnorm(x, g, b, 'epsilon', e[, 'moments', m])
    dzdx, dzdg, dzdb[, mom]  = vl_nnbnorm(x, g, b, dzdy, ...)
    y / dzdx                 = vl_nnpool(x, pool[, dzdy], 'stride', s, 'pad', p, 'method', 'max'|'avg')

Arguments follow the MEX drivers (matlab/src/vl_nnconv.cu, vl_nnbnorm.cu, vl_nnpool.cu): data arguments are
torch CUDA tensors standing for MATLAB arrays -- a MATLAB array of size H x W x C x N is a contiguous
tensor of shape (N, C, W, H) -- option names are case-insensitive strings, option values are numbers or
sequences.  Errors raise VlError carrying the reference's message text.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmcn_vl.so")


class VlError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("vl error %d: %s" % (code, message))
        self.code = code
        self.message = message


class Arg(C.Structure):
    _fields_ = [("kind", C.c_int), ("data", C.c_void_p), ("device", C.c_int), ("dtype", C.c_int),
                ("ndims", C.c_int), ("dims", C.c_size_t * 8), ("text", C.c_char_p)]


ALLOC_FN = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_int, C.c_size_t)

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `python -m matconvnet_amd.build`" % LIB_PATH)
        # torch first: it brings a HIP runtime of its own, and device tensors are shared with it only when that
        # runtime is the one already in the process when this library's dependency on libamdhip64 is resolved
        import torch  # noqa: F401
        L = C.CDLL(LIB_PATH)
        L.vlh_call.restype = C.c_int
        L.vlh_call.argtypes = [C.c_char_p, C.c_int, C.POINTER(Arg), C.c_int, C.POINTER(Arg), ALLOC_FN, C.c_void_p, C.c_void_p]
        L.vlh_last_message.restype = C.c_char_p
        L.vlh_pooling_backward.restype = C.c_int
        L.vlh_pooling_backward.argtypes = [C.c_void_p] * 4 + [C.c_int] * 14
        L.vlh_cpu_tensor_is_refused.restype = C.c_int
        L.vlh_bottleneck_create.restype = C.c_void_p
        L.vlh_bottleneck_create.argtypes = [C.c_int] * 5 + [C.c_double]
        L.vlh_unit_create.restype = C.c_void_p
        L.vlh_unit_create.argtypes = [C.c_int] * 5 + [C.c_double] + [C.c_int] * 3
        L.vlh_bottleneck_destroy.argtypes = [C.c_void_p]
        L.vlh_bottleneck_buffer.restype = C.c_void_p
        L.vlh_bottleneck_buffer.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_size_t)]
        L.vlh_bottleneck_set_stream.argtypes = [C.c_void_p, C.c_void_p]
        L.vlh_bottleneck_set_fused.argtypes = [C.c_void_p, C.c_int]
        L.vlh_bottleneck_set_fused.restype = None
        L.vlh_bottleneck_set_overlap.argtypes = [C.c_void_p, C.c_int]
        L.vlh_bottleneck_forward.argtypes = [C.c_void_p]
        L.vlh_bottleneck_backward.argtypes = [C.c_void_p]
        L.vlh_bottleneck_run.argtypes = [C.c_void_p, C.c_int, C.c_char_p, C.POINTER(C.c_float)]
        L.vlh_bottleneck_message.restype = C.c_char_p
        L.vlh_bottleneck_message.argtypes = [C.c_void_p]
        L.vlh_resnet50_create.restype = C.c_void_p
        L.vlh_resnet50_create.argtypes = [C.c_int, C.c_double, C.c_int, C.c_int]
        L.vlh_resnet50_destroy.argtypes = [C.c_void_p]
        L.vlh_resnet50_destroy.restype = None
        L.vlh_resnet50_units.argtypes = [C.c_void_p]
        L.vlh_resnet50_buffer.restype = C.c_void_p
        L.vlh_resnet50_buffer.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_size_t)]
        L.vlh_resnet50_set_stream.argtypes = [C.c_void_p, C.c_void_p]
        L.vlh_resnet50_set_fused.argtypes = [C.c_void_p, C.c_int]
        L.vlh_resnet50_set_fused.restype = None
        L.vlh_resnet50_set_test_mode.argtypes = [C.c_void_p, C.c_int]
        L.vlh_resnet50_set_test_mode.restype = None
        L.vlh_resnet50_set_deferred.argtypes = [C.c_void_p, C.c_int]
        L.vlh_resnet50_set_overlap.argtypes = [C.c_void_p, C.c_int]
        L.vlh_resnet50_set_channel_sums.argtypes = [C.c_void_p, C.c_int]
        L.vlh_bottleneck_set_deferred.argtypes = [C.c_void_p, C.c_int]
        L.vlh_resnet50_set_packed.argtypes = [C.c_void_p, C.c_int]
        L.vlh_resnet50_pack.argtypes = [C.c_void_p]
        L.vlh_bottleneck_set_packed.argtypes = [C.c_void_p, C.c_int]
        L.vlh_bottleneck_set_epilogue_sums.argtypes = [C.c_void_p, C.c_int]
        L.vlh_bottleneck_set_mask_bits.argtypes = [C.c_void_p, C.c_int]
        L.vlh_bottleneck_mask_bits_on.argtypes = [C.c_void_p]
        L.vlh_bottleneck_pack.argtypes = [C.c_void_p]
        L.vlh_resnet50_init.argtypes = [C.c_void_p, C.c_ulonglong]
        L.vlh_resnet50_forward.argtypes = [C.c_void_p]
        L.vlh_resnet50_backward.argtypes = [C.c_void_p]
        L.vlh_resnet50_sgd_step.argtypes = [C.c_void_p, C.c_double, C.c_double, C.c_double]
        L.vlh_resnet50_loss_derivative.argtypes = [C.c_void_p, C.c_double]
        L.vlh_resnet50_losses.argtypes = [C.c_void_p, C.POINTER(C.c_double)]
        L.vlh_resnet50_parameters.argtypes = [C.c_void_p]
        L.vlh_resnet50_capture.argtypes = [C.c_void_p, C.c_int, C.c_double, C.c_double, C.c_double]
        L.vlh_resnet50_replay.argtypes = [C.c_void_p]
        L.vlh_resnet50_parameters.restype = C.c_size_t
        L.vlh_resnet50_forward_flops.argtypes = [C.c_void_p]
        L.vlh_resnet50_forward_flops.restype = C.c_double
        L.vlh_resnet50_message.restype = C.c_char_p
        L.vlh_resnet50_message.argtypes = [C.c_void_p]
        _lib = L
    return _lib


def _torch():
    import torch
    return torch


def _array_arg(value, keep):
    """torch tensor (device or host), numpy array or number(s) -> Arg."""
    torch = _torch()
    a = Arg()
    a.kind = 0
    a.text = None
    if isinstance(value, torch.Tensor):
        t = value.contiguous()
        keep.append(t)
        mshape = list(reversed(t.shape))
        a.data = t.data_ptr() if t.numel() else None
        a.device = 1 if t.is_cuda else 0
        a.dtype = {torch.float32: 1, torch.float64: 2}.get(t.dtype, 0)
    else:  # host option value: MATLAB passes double row vectors
        v = np.atleast_1d(np.asarray(value, dtype=np.float64)).ravel()
        keep.append(v)
        mshape = [1, v.size] if v.size else [0, 0]
        a.data = v.ctypes.data if v.size else None
        a.device = 0
        a.dtype = 2
    a.ndims = len(mshape)
    for i, d in enumerate(mshape):
        a.dims[i] = int(d)
    return a


def _call(function, nout, args):
    torch = _torch()
    L = lib()
    keep = []
    cargs = (Arg * max(len(args), 1))()
    for i, v in enumerate(args):
        if isinstance(v, str):
            cargs[i].kind = 1
            b = v.encode()
            keep.append(b)
            cargs[i].text = b
        else:
            cargs[i] = _array_arg(v, keep)
    allocated = {}

    def alloc(user, device, nbytes):
        try:
            t = torch.empty(int(nbytes), dtype=torch.uint8, device="cuda" if device else "cpu")
        except RuntimeError:
            return None
        allocated[t.data_ptr()] = t
        return t.data_ptr()

    cb = ALLOC_FN(alloc)
    out = (Arg * 4)()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream) if torch.cuda.is_available() else None
    rc = L.vlh_call(function.encode(), nout, out, len(args), cargs, cb, None, stream)
    if rc != 0:
        raise VlError(rc, L.vlh_last_message().decode())
    results = []
    for i in range(max(nout, 1)):
        o = out[i]
        mshape = [int(o.dims[k]) for k in range(o.ndims)]
        while len(mshape) > 2 and mshape[-1] == 1:  # MATLAB drops trailing singleton dimensions
            mshape.pop()
        if not o.data:
            results.append(torch.empty(tuple(reversed(mshape)) if mshape else (0,), dtype=torch.float32))
            continue
        raw = allocated[o.data]
        dt = torch.float32 if o.dtype == 1 else torch.float64
        results.append(raw.view(dt).view(tuple(reversed(mshape))))
    return results


def vl_nnconv(*args, nout=None):
    back = len(args) > 3 and not isinstance(args[3], str)
    n = nout if nout is not None else (3 if back else 1)
    r = _call("vl_nnconv", n, list(args))
    return r[0] if n == 1 else tuple(r[:n])


def vl_nnconvt(*args, nout=None):
    back = len(args) > 3 and not isinstance(args[3], str)
    n = nout if nout is not None else (3 if back else 1)
    r = _call("vl_nnconvt", n, list(args))
    return r[0] if n == 1 else tuple(r)


def vl_nnbnorm(*args, nout=None):
    back = len(args) > 3 and not isinstance(args[3], str)
    n = nout if nout is not None else (3 if back else 1)
    r = _call("vl_nnbnorm", n, list(args))
    return r[0] if n == 1 else tuple(r[:n])


def vl_nnpool(*args):
    return _call("vl_nnpool", 1, list(args))[0]


def vl_nnrelu(*args):
    """vl_nnrelu(x [, dzdy], 'leak', value) (matlab/vl_nnrelu.m)."""
    return _call("vl_nnrelu", 1, list(args))[0]


def vl_nnsoftmax(*args):
    """vl_nnsoftmax(x [, dzdy]) (matlab/vl_nnsoftmax.m)."""
    return _call("vl_nnsoftmax", 1, list(args))[0]


def vl_nnloss(*args):
    """vl_nnloss(x, c [, dzdy], 'loss', name, 'instanceWeights', w, 'normalise', tf, 'threshold', t, 'topK', k)
    (matlab/vl_nnloss.m): the loss as a 1 x 1 device array, or dzdx when dzdy is given (a number)."""
    return _call("vl_nnloss", 1, list(args))[0]


def vl_taccum(*args):
    """vl_taccum(alpha, a, beta, b [, 'inplace']): alpha*a + beta*b (matlab/vl_taccum.m); with 'inplace', `a` itself
    is updated and returned."""
    inplace = any(isinstance(o, str) and o.lower() == "inplace" for o in args[4:])
    r = _call("vl_taccum", 0 if inplace else 1, list(args))
    return args[1] if inplace else r[0]


class _NamedBuffers:
    """Upload / download of the named device buffers a C++ harness object owns."""

    def set(self, name, array):
        """Upload a MATLAB-shaped numpy array (any order) into the named buffer."""
        torch = _torch()
        p, n = self._buf(name)
        host = np.ascontiguousarray(np.asfortranarray(array, dtype=np.float32).T).ravel()
        assert host.size == n, (name, host.size, n)
        src = torch.from_numpy(host).cuda()
        hip = C.CDLL("libamdhip64.so")
        hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        assert hip.hipMemcpy(p, src.data_ptr(), n * 4, 3) == 0  # device to device
        torch.cuda.synchronize()

    def get(self, name, mshape=None):
        """Download the named buffer as a MATLAB-shaped array (flat when no shape is given)."""
        torch = _torch()
        p, n = self._buf(name)
        dst = torch.empty(n, dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        hip = C.CDLL("libamdhip64.so")
        hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        assert hip.hipMemcpy(dst.data_ptr(), p, n * 4, 3) == 0
        torch.cuda.synchronize()
        if mshape is None:
            return dst.cpu().numpy()
        return np.asfortranarray(dst.cpu().numpy().reshape(tuple(reversed(mshape))).T)


class ResNet50(_NamedBuffers):
    """ResNet-50 forward + backward of the C++ harness (examples/imagenet/cnn_imagenet_init_resnet.m:52-134 without
    the loss layers); buffers are owned by the C++ side and named "input", "prediction", "dprediction",
    "stem.f", "fc.f", "unit<i>.<name>", ..."""

    def __init__(self, N=32, eps=1e-5, image_size=224, classes=1000, fused=True, seed=None, packed=True, deferred=False,
                 channel_sums=False, overlap=False):
        """packed: the convolutions read filter banks packed ahead, refreshed in one launch after every update (and by
        `set` of a parameter here); False: every call packs its own, as the plain operator calls do.
        deferred: the sums that finish the filter gradients run in one launch at the end of backward (off by
        default: for a whole network the partial banks, about 33 MB per layer, have left the caches by then, and
        reading them back from memory costs what the 54 saved launches gain)."""
        self.L = lib()
        self.packed = False
        self.N, self.image_size, self.classes = N, image_size, classes
        self.h = self.L.vlh_resnet50_create(N, eps, image_size, classes)
        msg = self.L.vlh_resnet50_message(self.h).decode()
        if msg:
            self.close()
            raise VlError(2, msg)
        torch = _torch()
        self._check(self.L.vlh_resnet50_set_stream(self.h, C.c_void_p(torch.cuda.current_stream().cuda_stream)))
        self.L.vlh_resnet50_set_fused(self.h, int(fused))
        if packed:
            self._check(self.L.vlh_resnet50_set_packed(self.h, 1))
            self.packed = True
        if deferred:
            self._check(self.L.vlh_resnet50_set_deferred(self.h, 1))
        if channel_sums:
            # (folded mode: the convolutions sum their output per channel for batch normalisation, identity units keep
            # their last ReLU's mask as bits, wherever the shapes allow; moments equal to rounding, not bit for bit)
            self._check(self.L.vlh_resnet50_set_channel_sums(self.h, 1))
        if overlap:
            # (backward: the units' filter gradients on a second stream beside the kernels that follow them; same bits)
            self._check(self.L.vlh_resnet50_set_overlap(self.h, 1))
        if seed is not None:
            self._check(self.L.vlh_resnet50_init(self.h, seed))

    def set(self, name, array):
        super().set(name, array)
        if self.packed and name.rsplit(".", 1)[-1] in ("f", "f1", "f2", "f3", "fs"):
            self.pack()

    def pack(self):
        """Refresh the packed filter banks (one launch); needed after writing filters by other means than `set`."""
        self._check(self.L.vlh_resnet50_pack(self.h))

    def close(self):
        if self.h:
            self.L.vlh_resnet50_destroy(self.h)
            self.h = None

    @property
    def units(self):
        return self.L.vlh_resnet50_units(self.h)

    @property
    def forward_flops_per_image(self):
        return self.L.vlh_resnet50_forward_flops(self.h)

    def set_fused(self, on):
        self.L.vlh_resnet50_set_fused(self.h, int(on))

    def set_test_mode(self, on):
        """Batch normalisation with the moving averages ("running.*") instead of the batch's moments; forward only."""
        self.L.vlh_resnet50_set_test_mode(self.h, int(on))

    def set_overlap(self, on):
        """backward: the units' filter gradients on a second stream beside the kernels that follow them (same bits)."""
        self._check(self.L.vlh_resnet50_set_overlap(self.h, int(on)))

    def _buf(self, name):
        n = C.c_size_t(0)
        p = self.L.vlh_resnet50_buffer(self.h, name.encode(), C.byref(n))
        if not p:
            raise KeyError(name)
        return p, n.value

    def _check(self, rc):
        if rc != 0:
            raise VlError(rc, self.L.vlh_resnet50_message(self.h).decode())

    def forward(self):
        self._check(self.L.vlh_resnet50_forward(self.h))

    def backward(self):
        self._check(self.L.vlh_resnet50_backward(self.h))

    def sgd_step(self, learning_rate, momentum=0.9, weight_decay=1e-4):
        self._check(self.L.vlh_resnet50_sgd_step(self.h, learning_rate, momentum, weight_decay))

    def loss_derivative(self, der_output=1.0):
        """"dprediction" from "prediction" and "labels" (softmax log-loss normalised by the batch size)."""
        self._check(self.L.vlh_resnet50_loss_derivative(self.h, der_output))

    def losses(self):
        """(softmax log-loss, top-1 error, top-5 error) of the batch, each normalised by the batch size."""
        v = (C.c_double * 3)()
        self._check(self.L.vlh_resnet50_losses(self.h, v))
        return tuple(v)

    @property
    def parameters(self):
        return self.L.vlh_resnet50_parameters(self.h)

    def set_stream(self, torch_stream):
        self._check(self.L.vlh_resnet50_set_stream(self.h, C.c_void_p(torch_stream.cuda_stream)))

    def capture(self, training, learning_rate=0.0, momentum=0.0, weight_decay=0.0):
        """Record forward (or the whole training step) on the network's stream into a HIP graph; `replay` launches it.
        Needs a stream other than the default one (`set_stream`) and one eager run of the same work beforehand."""
        self._check(self.L.vlh_resnet50_capture(self.h, int(training), learning_rate, momentum, weight_decay))

    def replay(self):
        self._check(self.L.vlh_resnet50_replay(self.h))


class Bottleneck(_NamedBuffers):
    """The ResNet-50 bottleneck block of the C++ harness (buffers owned by the C++ side)."""

    def __init__(self, H=56, W=56, Cc=256, M=64, N=32, eps=1e-5, fused=False, overlap=False, Cout=0, stride=1,
                 adapter=False, packed=False, deferred=False, epilogue_sums=False, mask_bits=False):
        """packed: the convolutions read filter banks packed ahead; `set` of a filter and every step of `run` refresh
        them with one launch (`pack`).  deferred: one launch at the end of backward sums the reduction splits of all
        the unit's filter gradients."""
        self.L = lib()
        self.packed = False
        self.shape = (H, W, Cc, M, N)
        self.h = self.L.vlh_unit_create(H, W, Cc, M, N, eps, Cout, stride, int(adapter))
        torch = _torch()
        self.L.vlh_bottleneck_set_stream(self.h, C.c_void_p(torch.cuda.current_stream().cuda_stream))
        self.L.vlh_bottleneck_set_fused(self.h, int(fused))
        if overlap and self.L.vlh_bottleneck_set_overlap(self.h, 1) != 0:
            raise VlError(2, self.L.vlh_bottleneck_message(self.h).decode())
        if packed:
            self._check(self.L.vlh_bottleneck_set_packed(self.h, 1))
            self.packed = True
        if deferred:
            self._check(self.L.vlh_bottleneck_set_deferred(self.h, 1))
        if epilogue_sums:
            # (fused mode: the forward convolutions sum their output per channel, batch normalisation takes the sums)
            self._check(self.L.vlh_bottleneck_set_epilogue_sums(self.h, 1))
        self.mask_bits = False
        if mask_bits:
            # (with epilogue_sums, identity shortcut: the last ReLU's mask kept as one bit per element for backward;
            # stays off where the shapes have no such form)
            self._check(self.L.vlh_bottleneck_set_mask_bits(self.h, 1))
            self.mask_bits = bool(self.L.vlh_bottleneck_mask_bits_on(self.h))

    def set(self, name, array):
        super().set(name, array)
        if self.packed and name in ("f1", "f2", "f3", "fs"):
            self.pack()

    def pack(self):
        self._check(self.L.vlh_bottleneck_pack(self.h))

    def close(self):
        if self.h:
            self.L.vlh_bottleneck_destroy(self.h)
            self.h = None

    def _buf(self, name):
        n = C.c_size_t(0)
        p = self.L.vlh_bottleneck_buffer(self.h, name.encode(), C.byref(n))
        if not p:
            raise KeyError(name)
        return p, n.value

    def _check(self, rc):
        if rc != 0:
            raise VlError(rc, self.L.vlh_bottleneck_message(self.h).decode())

    def forward(self):
        self._check(self.L.vlh_bottleneck_forward(self.h))

    def backward(self):
        self._check(self.L.vlh_bottleneck_backward(self.h))

    def run(self, steps, stage=None):
        ms = C.c_float(0.0)
        self._check(self.L.vlh_bottleneck_run(self.h, steps, stage.encode() if stage else None, C.byref(ms)))
        return ms.value
