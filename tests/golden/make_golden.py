"""Writes the golden vectors under tests/golden/ from the REAL MatConvNet CPU objects.

Run here (needs /root/reference to build oracle/_ref):   python tests/golden/make_golden.py
The vectors are data only: seeded inputs and the outputs vl::nn::Pooling, vl::nn::BatchNorm and
vl::impl::im2row produced for them.  They pin the oracle (and through it the GPU kernels) on machines
where the reference sources are absent.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import binding as ob  # noqa: E402


def F(a, dtype=np.float32):
    return np.asfortranarray(a, dtype=dtype)


def pool_vectors():
    r = np.random.default_rng(2024)
    out = {}
    cases = [
        # H, W, C, N, pool, stride, pad, method, input mode
        (12, 12, 2, 2, 3, 2, 1, "max", "ties"),
        (12, 12, 2, 2, 3, 2, 1, "max", "special"),
        (12, 12, 2, 2, 3, 2, 1, "avg", "normal"),
        (8, 8, 2, 2, 2, 2, 0, "avg", "normal"),
        (8, 8, 2, 2, 2, 2, 0, "max", "ties"),
        (9, 7, 2, 1, (3, 2), (2, 1), (0, 1, 1, 0), "max", "ties"),
        (9, 7, 2, 1, (3, 2), (2, 1), (0, 1, 1, 0), "avg", "normal"),
        (7, 9, 1, 2, (2, 3), (1, 2), (1, 0, 2, 1), "max", "normal"),
        (16, 16, 3, 1, 3, 1, 1, "max", "ties"),
        (16, 16, 3, 1, 3, 1, 1, "avg", "normal"),
    ]
    for i, (H, W, C, N, pool, stride, pad, method, mode) in enumerate(cases):
        g = ob.pool_geom((H, W, C, N), pool, stride, pad, method)
        if mode == "ties":
            x = r.integers(0, 4, size=(H, W, C, N)).astype(np.float32)
        elif mode == "special":
            x = r.integers(0, 3, size=(H, W, C, N)).astype(np.float32)
            flat = x.reshape(-1)
            flat[r.random(flat.size) < 0.2] = np.nan
            flat[r.random(flat.size) < 0.2] = -np.inf
        else:
            x = r.standard_normal((H, W, C, N)).astype(np.float32)
        x = F(x)
        dy = F(r.standard_normal(ob.pool_out_shape(g)))
        out["geom_%d" % i] = np.array([getattr(g, f) for f, _ in g._fields_], np.int32)
        out["x_%d" % i] = x
        out["dy_%d" % i] = dy
        out["y_%d" % i] = ob.ref_pool_forward(x, g)
        out["dx_%d" % i] = ob.ref_pool_backward(x, dy, g)
    out["count"] = np.int32(len(cases))
    np.savez_compressed(os.path.join(HERE, "pool_golden.npz"), **out)


def bnorm_vectors():
    r = np.random.default_rng(2025)
    out = {}
    cases = [(8, 8, 3, 2, 1e-4), (13, 17, 2, 3, 1e-4), (2, 2, 1, 2, 1e-4), (5, 3, 6, 3, 1e-5), (4, 4, 2, 3, 10.0)]
    k = 0
    for (H, W, C, N, eps) in cases:
        mu = r.standard_normal(C)
        sd = r.uniform(0.5, 2.0, C)
        x64 = r.standard_normal((H, W, C, N)) * sd[None, None, :, None] + mu[None, None, :, None]
        g64 = r.uniform(0.5, 1.5, C)
        b64 = 0.1 * r.standard_normal(C)
        dy64 = r.standard_normal((H, W, C, N))
        for dtype in (np.float32, np.float64):
            x, g, b, dy = F(x64.astype(np.float32), dtype), g64.astype(np.float32).astype(dtype), \
                b64.astype(np.float32).astype(dtype), F(dy64.astype(np.float32), dtype)
            y, mom = ob.ref_bnorm_forward(x, g, b, eps)
            dx, dg, db, mom2 = ob.ref_bnorm_backward(x, g, b, dy, eps)
            given = F(np.stack([mu, sd + 0.1], axis=1), dtype)
            yg, _ = ob.ref_bnorm_forward(x, g, b, eps, moments=given)
            dxg, dgg, dbg, _ = ob.ref_bnorm_backward(x, g, b, dy, eps, moments=given)
            for name, val in dict(x=x, g=g, b=b, dy=dy, y=y, mom=mom, dx=dx, dg=dg, db=db, mom2=mom2,
                                  given=given, yg=yg, dxg=dxg, dgg=dgg, dbg=dbg).items():
                out["%s_%d" % (name, k)] = val
            out["eps_%d" % k] = np.float64(eps)
            k += 1
    out["count"] = np.int32(k)
    np.savez_compressed(os.path.join(HERE, "bnorm_golden.npz"), **out)


def bnorm_edge_vectors():
    """The corners of the one-pass variance (bits/nnbnorm.cu:64-70,118-132): a constant channel (variance 0 or, in
    float, a rounding residue of either sign that max(0, .) clamps: sigma = sqrt(epsilon) or next to it), a channel with
    mean 1e3 and standard deviation 1e-2 (E[x^2] - mean^2 cancels ten digits: the float instantiation keeps none of
    the variance, the double one six digits), the same with mean 30 (seven digits cancel: float keeps a digit or two, double nine) and one element per channel (H = W = N = 1).  Float and double."""
    r = np.random.default_rng(2027)
    out = {}
    k = 0
    for kind, (H, W, C, N, eps) in (("constant", (6, 5, 3, 4, 1e-4)), ("constant", (8, 8, 2, 3, 1e-5)),
                                    ("cancel", (8, 8, 3, 4, 1e-4)), ("cancel", (14, 14, 2, 6, 1e-5)),
                                    ("cancel_mild", (8, 8, 3, 4, 1e-4)), ("cancel_mild", (14, 14, 2, 6, 1e-5)),
                                    ("single", (1, 1, 4, 1, 1e-4))):
        x64 = r.standard_normal((H, W, C, N)) * 1.5 + 0.25
        if kind == "constant":
            x64[:, :, 1, :] = 0.7          # (not representable in binary: sums and squares round)
        if kind == "cancel":       # condition number mean^2/var = 1e10: float keeps nothing, double about six digits
            x64[:, :, 0, :] = 1e3 + 1e-2 * r.standard_normal((H, W, N))
        if kind == "cancel_mild":  # 1e7: float still keeps nothing, double nine digits
            x64[:, :, 0, :] = 30.0 + 1e-2 * r.standard_normal((H, W, N))
        g64 = r.uniform(0.5, 1.5, C)
        b64 = 0.1 * r.standard_normal(C)
        dy64 = r.standard_normal((H, W, C, N))
        for dtype in (np.float32, np.float64):
            x, g, b, dy = F(x64.astype(np.float32), dtype), g64.astype(np.float32).astype(dtype), \
                b64.astype(np.float32).astype(dtype), F(dy64.astype(np.float32), dtype)
            y, mom = ob.ref_bnorm_forward(x, g, b, eps)
            dx, dg, db, mom2 = ob.ref_bnorm_backward(x, g, b, dy, eps)
            for name, val in dict(x=x, g=g, b=b, dy=dy, y=y, mom=mom, dx=dx, dg=dg, db=db, mom2=mom2).items():
                out["%s_%d" % (name, k)] = val
            out["eps_%d" % k] = np.float64(eps)
            out["kind_%d" % k] = np.array(kind)
            k += 1
    out["count"] = np.int32(k)
    np.savez_compressed(os.path.join(HERE, "bnorm_edge_golden.npz"), **out)


def im2row_vectors():
    r = np.random.default_rng(2026)
    out = {}
    cases = [
        # H, W, C, FH, FW, stride, pad, dilate
        (6, 7, 2, 3, 3, 1, 1, 1),
        (9, 8, 2, 3, 2, (2, 3), (1, 0, 2, 1), 1),
        (11, 10, 1, 3, 3, (3, 2), (2, 2, 3, 3), (2, 1)),
        (5, 5, 3, 1, 1, 1, 0, 1),
        (8, 8, 2, 5, 5, 1, 2, 1),
        (10, 9, 2, 2, 3, 2, (3, 0, 0, 2), (3, 2)),
    ]
    for i, (H, W, C, FH, FW, stride, pad, dilate) in enumerate(cases):
        g = ob.conv_geom((H, W, C, 1), (FH, FW, C, 1), stride, pad, dilate)
        x = F(r.standard_normal((H, W, C)))
        st = ob.ref_im2row_forward(x, g)
        t = F(r.standard_normal(st.shape))
        back = ob.ref_im2row_backward(t, g)
        out["geom_%d" % i] = np.array([getattr(g, f) for f, _ in g._fields_], np.int32)
        out["x_%d" % i] = x
        out["stacked_%d" % i] = st
        out["t_%d" % i] = t
        out["back_%d" % i] = back
    out["count"] = np.int32(len(cases))
    np.savez_compressed(os.path.join(HERE, "im2row_golden.npz"), **out)


if __name__ == "__main__":
    ob.build()
    assert ob.ref() is not None, "oracle/_ref did not build: is /root/reference present?"
    pool_vectors()
    bnorm_vectors()
    bnorm_edge_vectors()
    im2row_vectors()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
