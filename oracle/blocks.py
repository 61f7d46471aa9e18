"""Networks composed from oracle operators.  TEST INFRASTRUCTURE ONLY (tests, smoke check, CPU-baseline leg
of the benchmark)."""
import numpy as np

from . import binding as ob


def _c(dtype):
    return lambda a: np.asfortranarray(a, dtype=dtype) if a.ndim > 1 else a.astype(dtype)


def unit_forward(w, x, dtype=np.float32):
    """Forward half of `bottleneck`; returns the state its backward half needs."""
    c = _c(dtype)
    f1, f2, f3 = c(w["f1"]), c(w["f2"]), c(w["f3"])
    eps, stride, adapter = w["eps"], w.get("stride", 1), w.get("adapter", False)
    t = dict(x=x, f1=f1, f2=f2, f3=f3)
    t["g1"] = ob.conv_geom(x.shape, f1.shape, 1, 0, 1)
    t["a1"] = ob.conv_forward(x, f1, None, t["g1"])
    t["n1"], t["m1"] = ob.bnorm_forward(t["a1"], c(w["g1"]), c(w["b1"]), eps)
    t["r1"] = ob.relu_forward(t["n1"])
    t["g2"] = ob.conv_geom(t["r1"].shape, f2.shape, stride, 1, 1)
    t["a2"] = ob.conv_forward(t["r1"], f2, None, t["g2"])
    t["n2"], t["m2"] = ob.bnorm_forward(t["a2"], c(w["g2"]), c(w["b2"]), eps)
    t["r2"] = ob.relu_forward(t["n2"])
    t["g3"] = ob.conv_geom(t["r2"].shape, f3.shape, 1, 0, 1)
    t["a3"] = ob.conv_forward(t["r2"], f3, None, t["g3"])
    t["n3"], t["m3"] = ob.bnorm_forward(t["a3"], c(w["g3"]), c(w["b3"]), eps)
    if adapter:
        t["fs"] = c(w["fs"])
        t["gs"] = ob.conv_geom(x.shape, t["fs"].shape, stride, 0, 1)
        t["as"] = ob.conv_forward(x, t["fs"], None, t["gs"])
        t["ns"], t["ms"] = ob.bnorm_forward(t["as"], c(w["gs"]), c(w["bs"]), eps)
        shortcut = t["ns"]
    else:
        shortcut = x
    t["s"] = ob.add(t["n3"], shortcut)
    t["y"] = ob.relu_forward(t["s"])
    return t


def unit_backward(w, t, dy, dtype=np.float32):
    """Backward half of `bottleneck` from the state `unit_forward` returned."""
    c = _c(dtype)
    eps, adapter = w["eps"], w.get("adapter", False)
    ds = ob.relu_backward(t["s"], dy)
    da3, dg3, db3, _ = ob.bnorm_backward(t["a3"], c(w["g3"]), ds, eps, moments=t["m3"])
    dr2, df3, _ = ob.conv_backward(t["r2"], t["f3"], da3, t["g3"], want=(True, True, False))
    dn2 = ob.relu_backward(t["n2"], dr2)
    da2, dg2, db2, _ = ob.bnorm_backward(t["a2"], c(w["g2"]), dn2, eps, moments=t["m2"])
    dr1, df2, _ = ob.conv_backward(t["r1"], t["f2"], da2, t["g2"], want=(True, True, False))
    dn1 = ob.relu_backward(t["n1"], dr1)
    da1, dg1, db1, _ = ob.bnorm_backward(t["a1"], c(w["g1"]), dn1, eps, moments=t["m1"])
    dxm, df1, _ = ob.conv_backward(t["x"], t["f1"], da1, t["g1"], want=(True, True, False))
    out = dict(df1=df1, df2=df2, df3=df3, dg1=dg1, db1=db1, dg2=dg2, db2=db2, dg3=dg3, db3=db3)
    if adapter:
        das, dgs, dbs, _ = ob.bnorm_backward(t["as"], c(w["gs"]), ds, eps, moments=t["ms"])
        dxs, dfs, _ = ob.conv_backward(t["x"], t["fs"], das, t["gs"], want=(True, True, False))
        out.update(dzdx=ob.add(dxm, dxs), dfs=dfs, dgs=dgs, dbs=dbs)
    else:
        out.update(dzdx=ob.add(dxm, ds))
    return out


def bottleneck(w, dtype=np.float32, keep=False):
    """ResNet-50 bottleneck unit forward + backward, in the order the reference's DagNN evaluates it
    (matlab/+dagnn/@DagNN/eval.m:88-119) for one segment of examples/imagenet/cnn_imagenet_init_resnet.m:86-118:
    conv1x1, bnorm, relu, conv3x3 pad 1 (stride s), bnorm, relu, conv1x1, bnorm, + shortcut, relu, with the
    shortcut the input itself or (first segment of a section) conv1x1 stride s + bnorm; no conv bias; bnorm
    backward with the moments cached by the forward pass (matlab/+dagnn/BatchNorm.m:27-34); the derivatives of a
    variable with two consumers are added (matlab/+dagnn/Layer.m:127-135).
    `w` is a dict from matconvnet_amd.workloads.bottleneck_case."""
    c = _c(dtype)
    t = unit_forward(w, c(w["x"]), dtype)
    out = unit_backward(w, t, c(w["dy"]), dtype)
    out["y"] = t["y"]
    if keep:
        out.update({k: t[k] for k in ("a1", "n1", "r1", "a2", "n2", "r2", "a3", "n3", "s", "m1", "m2", "m3")})
    return out


def resnet50(w, dtype=np.float32):
    """ResNet-50 forward + backward as examples/imagenet/cnn_imagenet_init_resnet.m:52-134 wires it, without the
    loss layers (the derivative with respect to the prediction is given): conv 7x7 stride 2 pad 3 without bias (:53-56),
    bnorm, relu, max pool 3x3 stride 2 pad 1 (:58-66), the bottleneck units (:73-115), average pool over the whole
    remaining map (:117-120), 1x1 convolution with bias (:122-126).  `w` comes from
    matconvnet_amd.workloads.resnet50_case: `stem`, `units` (list of unit dicts), `fc`, `input`, `dprediction`."""
    c = _c(dtype)
    eps = w["eps"]
    x = c(w["input"])
    st = w["stem"]
    f0 = c(st["f"])
    g0 = ob.conv_geom(x.shape, f0.shape, 2, 3, 1)
    a0 = ob.conv_forward(x, f0, None, g0)
    n0, m0 = ob.bnorm_forward(a0, c(st["g"]), c(st["b"]), eps)
    r0 = ob.relu_forward(n0)
    gp = ob.pool_geom(r0.shape, 3, 2, 1, "max")
    p0 = ob.pool_forward(r0, gp)
    states, h = [], p0
    for u in w["units"]:
        t = unit_forward(u, h, dtype)
        states.append(t)
        h = t["y"]
    ga = ob.pool_geom(h.shape, (h.shape[0], h.shape[1]), 1, 0, "avg")
    avg = ob.pool_forward(h, ga)
    ff, fb = c(w["fc"]["f"]), c(w["fc"]["b"])
    gf = ob.conv_geom(avg.shape, ff.shape, 1, 0, 1)
    pred = ob.conv_forward(avg, ff, fb, gf)
    out = dict(prediction=pred)
    davg, out["fc.df"], out["fc.db"] = ob.conv_backward(avg, ff, c(w["dprediction"]), gf)
    d = ob.pool_backward(h, davg, ga)
    for i in range(len(states) - 1, -1, -1):
        g = unit_backward(w["units"][i], states[i], d, dtype)
        d = g.pop("dzdx")
        for k, v in g.items():
            out["unit%d.%s" % (i, k)] = v
    dr0 = ob.pool_backward(r0, d, gp)
    dn0 = ob.relu_backward(n0, dr0)
    da0, out["stem.dg"], out["stem.db"], _ = ob.bnorm_backward(a0, c(st["g"]), dn0, eps, moments=m0)
    _, out["stem.df"], _ = ob.conv_backward(x, f0, da0, g0, want=(False, True, False))
    return out
