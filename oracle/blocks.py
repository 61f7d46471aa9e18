"""Networks composed from oracle operators.  TEST INFRASTRUCTURE ONLY (tests, smoke check, CPU-baseline leg
of the benchmark)."""
import numpy as np

from . import binding as ob


def bottleneck(w, dtype=np.float32, keep=False):
    """ResNet-50 bottleneck unit forward + backward, in the order the reference's DagNN evaluates it
    (matlab/+dagnn/@DagNN/eval.m:88-119) for one segment of examples/imagenet/cnn_imagenet_init_resnet.m:86-118:
    conv1x1, bnorm, relu, conv3x3 pad 1 (stride s), bnorm, relu, conv1x1, bnorm, + shortcut, relu, with the
    shortcut the input itself or (first segment of a section) conv1x1 stride s + bnorm; no conv bias; bnorm
    backward with the moments cached by the forward pass (matlab/+dagnn/BatchNorm.m:27-34); the derivatives of a
    variable with two consumers are added (matlab/+dagnn/Layer.m:127-135).
    `w` is a dict from matconvnet_amd.workloads.bottleneck_case."""
    c = lambda a: np.asfortranarray(a, dtype=dtype) if a.ndim > 1 else a.astype(dtype)
    x, dy = c(w["x"]), c(w["dy"])
    f1, f2, f3 = c(w["f1"]), c(w["f2"]), c(w["f3"])
    eps, stride, adapter = w["eps"], w.get("stride", 1), w.get("adapter", False)
    g1 = ob.conv_geom(x.shape, f1.shape, 1, 0, 1)
    a1 = ob.conv_forward(x, f1, None, g1)
    n1, m1 = ob.bnorm_forward(a1, c(w["g1"]), c(w["b1"]), eps)
    r1 = ob.relu_forward(n1)
    g2 = ob.conv_geom(r1.shape, f2.shape, stride, 1, 1)
    a2 = ob.conv_forward(r1, f2, None, g2)
    n2, m2 = ob.bnorm_forward(a2, c(w["g2"]), c(w["b2"]), eps)
    r2 = ob.relu_forward(n2)
    g3 = ob.conv_geom(r2.shape, f3.shape, 1, 0, 1)
    a3 = ob.conv_forward(r2, f3, None, g3)
    n3, m3 = ob.bnorm_forward(a3, c(w["g3"]), c(w["b3"]), eps)
    if adapter:
        fs = c(w["fs"])
        gs = ob.conv_geom(x.shape, fs.shape, stride, 0, 1)
        as_ = ob.conv_forward(x, fs, None, gs)
        ns, ms = ob.bnorm_forward(as_, c(w["gs"]), c(w["bs"]), eps)
        shortcut = ns
    else:
        shortcut = x
    s = ob.add(n3, shortcut)
    y = ob.relu_forward(s)
    ds = ob.relu_backward(s, dy)
    da3, dg3, db3, _ = ob.bnorm_backward(a3, c(w["g3"]), ds, eps, moments=m3)
    dr2, df3, _ = ob.conv_backward(r2, f3, da3, g3, want=(True, True, False))
    dn2 = ob.relu_backward(n2, dr2)
    da2, dg2, db2, _ = ob.bnorm_backward(a2, c(w["g2"]), dn2, eps, moments=m2)
    dr1, df2, _ = ob.conv_backward(r1, f2, da2, g2, want=(True, True, False))
    dn1 = ob.relu_backward(n1, dr1)
    da1, dg1, db1, _ = ob.bnorm_backward(a1, c(w["g1"]), dn1, eps, moments=m1)
    dxm, df1, _ = ob.conv_backward(x, f1, da1, g1, want=(True, True, False))
    out = dict(y=y, df1=df1, df2=df2, df3=df3, dg1=dg1, db1=db1, dg2=dg2, db2=db2, dg3=dg3, db3=db3)
    if adapter:
        das, dgs, dbs, _ = ob.bnorm_backward(as_, c(w["gs"]), ds, eps, moments=ms)
        dxs, dfs, _ = ob.conv_backward(x, fs, das, gs, want=(True, True, False))
        out.update(dzdx=ob.add(dxm, dxs), dfs=dfs, dgs=dgs, dbs=dbs)
    else:
        out.update(dzdx=ob.add(dxm, ds))
    if keep:
        out.update(a1=a1, n1=n1, r1=r1, a2=a2, n2=n2, r2=r2, a3=a3, n3=n3, s=s, m1=m1, m2=m2, m3=m3)
    return out
