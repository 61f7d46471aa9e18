"""Seeded synthetic inputs for the benchmark configurations (fp32, MATLAB layout H x W x C x N, returned
as Fortran-ordered numpy arrays).  One generator per configuration; the same bytes feed the GPU kernels
and whatever CPU code they are compared with."""
import numpy as np


def _f(a):
    return np.asfortranarray(a, dtype=np.float32)


def conv_single(seed=1, N=100):
    """Single vl_nnconv layer: x 32x32x3xN U[-1,1), f 5x5x3x32 N(0,0.01^2), b = 0, stride 1, pad 2."""
    r = np.random.default_rng(seed)
    x = _f(r.uniform(-1.0, 1.0, size=(32, 32, 3, N)))
    f = _f(0.01 * r.standard_normal((5, 5, 3, 32)))
    b = np.zeros((32,), np.float32)
    dy = _f(r.standard_normal((32, 32, 32, N)))
    return dict(x=x, f=f, b=b, dy=dy, stride=1, pad=2, dilate=1)


def bnorm_case(seed=2, H=56, W=56, C=256, N=32, eps=1e-4):
    """vl_nnbnorm backward: per-channel mean N(0,1), std U(0.5,2); g U(0.5,1.5); b N(0,0.1)."""
    r = np.random.default_rng(seed)
    mu = r.standard_normal(C).astype(np.float32)
    sd = r.uniform(0.5, 2.0, C).astype(np.float32)
    x = r.standard_normal((H, W, C, N), dtype=np.float32)
    x = _f(x * sd[None, None, :, None] + mu[None, None, :, None])
    g = r.uniform(0.5, 1.5, C).astype(np.float32)
    b = (0.1 * r.standard_normal(C)).astype(np.float32)
    dy = _f(r.standard_normal((H, W, C, N), dtype=np.float32))
    return dict(x=x, g=g, b=b, dy=dy, eps=eps)


def pool_max_case(seed=3, H=112, W=112, C=64, N=32, ties=False):
    """vl_nnpool max 3x3 stride 2 pad 1; `ties` quantises x to 8 levels to stress first-max routing."""
    r = np.random.default_rng(seed)
    x = r.standard_normal((H, W, C, N), dtype=np.float32)
    if ties:
        x = np.floor(np.clip((x + 2.0) * 2.0, 0.0, 7.0)).astype(np.float32)
    oh, ow = (H + 2 - 3) // 2 + 1, (W + 2 - 3) // 2 + 1
    dy = r.standard_normal((oh, ow, C, N), dtype=np.float32)
    return dict(x=_f(x), dy=_f(dy), pool=3, stride=2, pad=1, method="max")


def pool_avg_case(seed=4, H=56, W=56, C=256, N=32):
    """vl_nnpool avg 2x2 stride 2."""
    r = np.random.default_rng(seed)
    x = r.standard_normal((H, W, C, N), dtype=np.float32)
    dy = r.standard_normal((H // 2, W // 2, C, N), dtype=np.float32)
    return dict(x=_f(x), dy=_f(dy), pool=2, stride=2, pad=0, method="avg")


def he_normal(r, shape):
    fh, fw, fc, _ = shape
    return _f(r.standard_normal(shape, dtype=np.float32) * np.float32(np.sqrt(2.0 / (fh * fw * fc))))


def bottleneck_case(seed=5, H=56, W=56, C=256, M=64, N=32, eps=1e-5, Cout=None, stride=1, adapter=False):
    """ResNet-50 bottleneck unit: conv1x1 C->M, bn, relu, conv3x3 M->M pad 1 (stride), bn, relu, conv1x1 M->Cout,
    bn, + shortcut, relu; shortcut = identity, or (adapter) conv1x1 C->Cout (stride) + bn.  He-normal weights, no
    conv bias, bnorm gain 1 / bias 0 (gains and biases of the adapter unit are randomised a little so that they
    matter)."""
    r = np.random.default_rng(seed)
    Cout = C if Cout is None else Cout
    Ho, Wo = (H - 1) // stride + 1, (W - 1) // stride + 1
    x = _f(r.standard_normal((H, W, C, N), dtype=np.float32))
    dy = _f(r.standard_normal((Ho, Wo, Cout, N), dtype=np.float32))
    f1 = he_normal(r, (1, 1, C, M))
    f2 = he_normal(r, (3, 3, M, M))
    f3 = he_normal(r, (1, 1, M, Cout))
    ones = lambda n: np.ones((n,), np.float32)
    zeros = lambda n: np.zeros((n,), np.float32)
    w = dict(x=x, dy=dy, f1=f1, f2=f2, f3=f3, g1=ones(M), b1=zeros(M), g2=ones(M), b2=zeros(M),
             g3=ones(Cout), b3=zeros(Cout), eps=eps, stride=stride, adapter=adapter)
    if adapter:
        w.update(fs=he_normal(r, (1, 1, C, Cout)), gs=(1 + 0.1 * r.standard_normal(Cout)).astype(np.float32),
                 bs=(0.1 * r.standard_normal(Cout)).astype(np.float32))
    return w


def resnet50_case(seed=9, image_size=64, N=4, classes=10, eps=1e-5):
    """Parameters and inputs of ResNet-50 (examples/imagenet/cnn_imagenet_init_resnet.m:52-134): He-normal filters,
    gains and biases a little away from 1 and 0 so that they matter, N(0,1) images and prediction derivative."""
    r = np.random.default_rng(seed)
    gain = lambda n: (1 + 0.1 * r.standard_normal(n)).astype(np.float32)
    bias = lambda n: (0.1 * r.standard_normal(n)).astype(np.float32)
    w = dict(eps=eps, input=_f(r.standard_normal((image_size, image_size, 3, N), dtype=np.float32)),
             dprediction=_f(r.standard_normal((1, 1, classes, N), dtype=np.float32)),
             stem=dict(f=he_normal(r, (7, 7, 3, 64)), g=gain(64), b=bias(64)), units=[])
    C = 64
    for s, length in enumerate((3, 4, 6, 3)):
        M, Cout = 64 << s, 256 << s
        for l in range(length):
            first = l == 0
            u = dict(f1=he_normal(r, (1, 1, C, M)), f2=he_normal(r, (3, 3, M, M)), f3=he_normal(r, (1, 1, M, Cout)),
                     g1=gain(M), b1=bias(M), g2=gain(M), b2=bias(M), g3=gain(Cout), b3=bias(Cout), eps=eps,
                     stride=2 if first and s >= 1 else 1, adapter=first)
            if first:
                u.update(fs=he_normal(r, (1, 1, C, Cout)), gs=gain(Cout), bs=bias(Cout))
            w["units"].append(u)
            C = Cout
    w["fc"] = dict(f=he_normal(r, (1, 1, C, classes)), b=bias(classes))
    return w


def conv_vgg(seed=6, H=56, W=56, C=256, K=256, N=64):
    """VGG-style wide 3x3 conv backward: x N(0,1), f He-normal 3x3xCxK, stride 1, pad 1."""
    r = np.random.default_rng(seed)
    x = _f(r.standard_normal((H, W, C, N), dtype=np.float32))
    f = he_normal(r, (3, 3, C, K))
    dy = _f(r.standard_normal((H, W, K, N), dtype=np.float32))
    return dict(x=x, f=f, b=None, dy=dy, stride=1, pad=1, dilate=1)
