"""The C++ operator layer (vl::nn classes + MEX-convention front-end) on the GPU, driven the way the
reference's own tests drive vl_nnconv / vl_nnbnorm / vl_nnpool (matlab/xtest/suite/nnconv.m, nnbnorm.m,
nnpool.m), checked against the CPU oracle."""
import numpy as np
import pytest
import torch

from matconvnet_amd import workloads
from util import F, bits_equal, rel_max

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(np.asfortranarray(a, dtype=np.float32).T)).cuda()


def host(t):
    return np.asfortranarray(t.detach().cpu().numpy().T)


def test_vl_nnconv_forward_backward(vl, ob):
    r = np.random.default_rng(1)
    x = F(r.standard_normal((14, 12, 6, 3)))
    f = F(r.standard_normal((3, 3, 6, 8)) * 0.2)
    b = r.standard_normal(8).astype(np.float32)
    g = ob.conv_geom(x.shape, f.shape, (1, 1), (1, 0, 2, 1), 1)
    y = vl.vl_nnconv(dev(x), dev(f), dev(b), "pad", [1, 0, 2, 1])
    want = ob.conv_forward(x, f, b, g)
    assert tuple(reversed(y.shape)) == want.shape
    assert rel_max(host(y), want) < 2e-4
    dy = F(r.standard_normal(want.shape))
    dx, df, db = vl.vl_nnconv(dev(x), dev(f), dev(b), dev(dy), "Pad", [1, 0, 2, 1], "STRIDE", 1)
    wdx, wdf, wdb = ob.conv_backward(x, f, dy, g)
    assert rel_max(host(dx), wdx) < 2e-4 and rel_max(host(df), wdf) < 2e-4 and rel_max(host(db).ravel(), wdb) < 2e-4
    assert tuple(reversed(df.shape)) == f.shape


def test_vl_nnconv_skipped_outputs_and_empty_bias(vl, ob):
    r = np.random.default_rng(2)
    x = F(r.standard_normal((9, 9, 4, 2)))
    f = F(r.standard_normal((3, 3, 4, 5)))
    dy = F(r.standard_normal((7, 7, 5, 2)))
    empty = torch.empty((0,), dtype=torch.float32, device="cuda")
    dx, df, db = vl.vl_nnconv(dev(x), dev(f), empty, dev(dy), "NoDerData")
    assert dx.numel() == 0 and db.numel() == 0 and df.numel() == f.size
    g = ob.conv_geom(x.shape, f.shape, 1, 0, 1)
    assert rel_max(host(df), ob.conv_backward(x, f, dy, g)[1]) < 2e-4


def test_vl_nnconv_validation_messages(vl):
    x = torch.zeros((2, 4, 8, 8), device="cuda")   # MATLAB 8x8x4x2
    f = torch.zeros((5, 4, 3, 3), device="cuda")   # 3x3x4x5
    b = torch.zeros((5,), device="cuda")
    cases = [
        (("stride", 0), "At least one element of STRIDE is smaller than one."),
        (("pad", -1), "An element of PAD is negative."),
        (("pad", [1, 2, 3]), "PAD has neither one nor four elements."),
        (("dilate", 0), "An element of DILATE is less than one."),
        (("bogus", 1), "Unknown option 'bogus'."),
        (("stride",), "Option 'Stride' requires an argument."),
    ]
    for opts, message in cases:
        with pytest.raises(vl.VlError) as e:
            vl.vl_nnconv(x, f, b, *opts)
        assert e.value.message == message, e.value.message
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnconv(x, torch.zeros((5, 3, 3, 3), device="cuda"), b)
    assert e.value.message == "The FILTERS depth does not divide the DATA depth."
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnconv(x, torch.zeros((5, 4, 9, 9), device="cuda"), b)
    assert e.value.message == "FILTERS are larger than the DATA (including padding)."
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnconv(x, f, b, torch.zeros((2, 5, 5, 5), device="cuda"))
    assert e.value.message == "DEROUTPUT dimensions are incompatible with X and FILTERS."
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnconv(x, f, torch.zeros((4,), device="cuda"))
    assert e.value.message == "The number of elements of BIASES is not the same as the number of filters."
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnconv(x, f)
    assert e.value.message == "There are less than three arguments."


def test_cpu_tensors_are_refused_not_silently_computed(vl):
    assert vl.lib().vlh_cpu_tensor_is_refused() == 1
    assert b"HIP" in vl.lib().vlh_last_message()
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnpool(torch.zeros((1, 1, 4, 4)), 2)
    assert e.value.code == 1  # VLE_Unsupported


def test_vl_nnbnorm_modes(vl, ob):
    w = workloads.bnorm_case(seed=3, H=13, W=17, C=4, N=7)
    x, g, b, dy = w["x"], w["g"], w["b"], w["dy"]
    d = lambda a: F(a, np.float64) if a.ndim > 1 else a.astype(np.float64)
    y, mom = vl.vl_nnbnorm(dev(x), dev(g), dev(b), nout=2)
    wy, wmom = ob.bnorm_forward(d(x), d(g), d(b), 1e-4)
    assert tuple(reversed(mom.shape)) == (4, 2)
    assert rel_max(host(y), wy) < 1e-5 and rel_max(host(mom), wmom) < 1e-5
    dx, dg, db, mom2 = vl.vl_nnbnorm(dev(x), dev(g), dev(b), dev(dy), "epsilon", 1e-3, nout=4)
    wdx, wdg, wdb, wmom2 = ob.bnorm_backward(d(x), d(g), d(dy), 1e-3)
    assert rel_max(host(dx), wdx) < 1e-5 and rel_max(host(dg).ravel(), wdg) < 1e-5
    assert rel_max(host(db).ravel(), wdb) < 1e-5 and rel_max(host(mom2), wmom2) < 1e-5
    # 'moments' given = batch moments reproduces the batch mode (nnbnorm.m:53-79)
    dx2, dg2, db2 = vl.vl_nnbnorm(dev(x), dev(g), dev(b), dev(dy), "epsilon", 1e-3, "moments", mom2)
    assert rel_max(host(dx2), wdx) < 1e-5 and rel_max(host(dg2).ravel(), wdg) < 1e-5
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnbnorm(dev(x), dev(g[:3]), dev(b))
    assert e.value.message == "The MULTIPLIERS size does not match the DATA depth."
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnbnorm(dev(x), dev(g), dev(b), dev(dy[:, :, :, :3]))
    assert e.value.message == "DATA and DEROUTPUT do not have the same size."


@pytest.mark.parametrize("method", ["max", "avg"])
def test_vl_nnpool(vl, ob, method):
    r = np.random.default_rng(4)
    x = F(r.integers(0, 4, size=(12, 14, 3, 2)).astype(np.float32))
    g = ob.pool_geom(x.shape, (3, 2), (2, 1), (1, 0, 0, 1), method)
    y = vl.vl_nnpool(dev(x), [3, 2], "stride", [2, 1], "pad", [1, 0, 0, 1], "method", method)
    assert bits_equal(host(y), ob.pool_forward(x, g))
    dy = F(r.standard_normal(ob.pool_out_shape(g)))
    dx = vl.vl_nnpool(dev(x), [3, 2], dev(dy), "stride", [2, 1], "pad", [1, 0, 0, 1], "METHOD", method.upper())
    assert bits_equal(host(dx), ob.pool_backward(x, dy, g))


def test_vl_nnpool_validation_messages(vl):
    x = torch.zeros((1, 1, 8, 8), device="cuda")
    for args, message in [
        ((3, "pad", 3), "A padding value is larger or equal to the size of the pooling window."),
        ((0,), "A dimension of the pooling SIZE is void."),
        ((9,), "The pooling window is larger than the DATA (including padding)."),
        ((2, "method", "median"), "METHOD is not a supported method."),
        ((2, "stride", [1, 0]), "At least one element of STRIDE is smaller than one."),
        (([1, 2, 3],), "SIZE has neither one nor two elements."),
    ]:
        with pytest.raises(vl.VlError) as e:
            vl.vl_nnpool(x, *args)
        assert e.value.message == message, e.value.message


def test_pooling_class_accumulates_like_the_reference(vl, ob):
    """vl::nn::Pooling::backward adds into derInput (callers zero it); backwardOverwrite does not read it."""
    import ctypes as C
    r = np.random.default_rng(5)
    x = F(r.integers(0, 3, size=(10, 10, 2, 2)).astype(np.float32))
    g = ob.pool_geom(x.shape, 3, 2, 1, "max")
    dy = F(r.standard_normal(ob.pool_out_shape(g)))
    base = F(r.standard_normal(x.shape))
    xd, dyd = dev(x), dev(dy)
    for overwrite in (0, 1):
        dx = dev(base)
        rc = vl.lib().vlh_pooling_backward(C.c_void_p(torch.cuda.current_stream().cuda_stream), C.c_void_p(dx.data_ptr()),
                                           C.c_void_p(xd.data_ptr()), C.c_void_p(dyd.data_ptr()), 10, 10, 2, 2, 3, 3, 2, 2, 1, 1, 1, 1, 0, overwrite)
        assert rc == 0
        want = ob.pool_backward(x, dy, g) if overwrite else ob.pool_backward(x, dy, g, dx=base.copy(order="F"))
        assert bits_equal(host(dx), want)


def _oracle_bottleneck(ob, w, dtype):
    from oracle import blocks
    return blocks.bottleneck(w, dtype)


def _load(blk, w):
    for k in ("x", "f1", "f2", "f3", "g1", "b1", "g2", "b2", "g3", "b3"):
        blk.set(k, w[k])
    blk.set("dzdy", w["dy"])


def test_bottleneck_block_end_to_end_small_batch(vl, ob):
    """ResNet-50 bottleneck fwd+bwd at N = 2 against the block composed from oracle operators (double).
    Block-level gate 5e-4 on every output (three stacked layers of 2e-4 / 1e-5 operators)."""
    w = workloads.bottleneck_case(N=2)
    blk = vl.Bottleneck(N=2, eps=w["eps"])
    try:
        _load(blk, w)
        blk.forward()
        blk.backward()
        want = _oracle_bottleneck(ob, w, np.float64)
        shapes = dict(y=w["x"].shape, dzdx=w["x"].shape, df1=w["f1"].shape, df2=w["f2"].shape, df3=w["f3"].shape,
                      dg1=(64,), db1=(64,), dg2=(64,), db2=(64,), dg3=(256,), db3=(256,))
        errs = {k: rel_max(blk.get(k, shapes[k]), want[k]) for k in shapes}
        print("bottleneck N=2:", {k: "%.1e" % v for k, v in errs.items()})
        assert max(errs.values()) < 5e-4, errs
    finally:
        blk.close()


def test_bottleneck_block_full_config_stage_by_stage(vl, ob):
    """benchmark configuration 4 at its full size (N = 32, 56x56, 256/64 channels).  ReLU's derivative is
    discontinuous, so an end-to-end comparison of gradients at this size flips a handful of masks between any
    two float implementations and says nothing about either.  Instead every stage of the GPU block is
    checked against the oracle applied to the SAME inputs (the GPU's own intermediate buffers): wiring,
    shapes and each operator at its real size.  Gates: conv 2e-4 (float oracle), bnorm 1e-5 (double oracle on
    the float inputs), relu / sum bit-exact.  The forward output y, which is continuous in everything, is
    also compared end to end."""
    N = 32
    w = workloads.bottleneck_case(N=N)
    blk = vl.Bottleneck(N=N, eps=w["eps"])
    try:
        _load(blk, w)
        blk.forward()
        blk.backward()
        big, small = (56, 56, 256, N), (56, 56, 64, N)
        shp = dict(a1=small, n1=small, r1=small, a2=small, n2=small, r2=small, a3=big, n3=big, s=big, y=big,
                   m1=(64, 2), m2=(64, 2), m3=(256, 2), ds=big, da3=big, dr2=small, dn2=small, da2=small,
                   dr1=small, dn1=small, da1=small, dxm=big, dzdx=big, df1=w["f1"].shape, df2=w["f2"].shape,
                   df3=w["f3"].shape, dg1=(64,), db1=(64,), dg2=(64,), db2=(64,), dg3=(256,), db3=(256,))
        G = {k: blk.get(k, v) for k, v in shp.items()}
        x, dy, eps = w["x"], w["dy"], w["eps"]
        d = lambda a: F(a, np.float64) if a.ndim > 1 else a.astype(np.float64)
        g1 = ob.conv_geom(x.shape, w["f1"].shape, 1, 0, 1)
        g2 = ob.conv_geom(small, w["f2"].shape, 1, 1, 1)
        g3 = ob.conv_geom(small, w["f3"].shape, 1, 0, 1)
        errs = {}
        # forward
        errs["a1"] = rel_max(G["a1"], ob.conv_forward(x, w["f1"], None, g1))
        errs["a2"] = rel_max(G["a2"], ob.conv_forward(G["r1"], w["f2"], None, g2))
        errs["a3"] = rel_max(G["a3"], ob.conv_forward(G["r2"], w["f3"], None, g3))
        for i, (a, n, m, gk, bk) in enumerate([("a1", "n1", "m1", "g1", "b1"), ("a2", "n2", "m2", "g2", "b2"), ("a3", "n3", "m3", "g3", "b3")]):
            wy, wm = ob.bnorm_forward(d(G[a]), d(w[gk]), d(w[bk]), eps)
            errs[n] = rel_max(G[n], wy)
            errs[m] = rel_max(G[m], wm)
        assert bits_equal(G["r1"], ob.relu_forward(G["n1"])) and bits_equal(G["r2"], ob.relu_forward(G["n2"]))
        assert bits_equal(G["s"], ob.add(G["n3"], x)) and bits_equal(G["y"], ob.relu_forward(G["s"]))
        # backward
        assert bits_equal(G["ds"], ob.relu_backward(G["s"], dy))
        for (da, dg, db, a, m, gk, dyk) in [("da3", "dg3", "db3", "a3", "m3", "g3", "ds"), ("da2", "dg2", "db2", "a2", "m2", "g2", "dn2"),
                                            ("da1", "dg1", "db1", "a1", "m1", "g1", "dn1")]:
            wdx, wdg, wdb, _ = ob.bnorm_backward(d(G[a]), d(w[gk]), d(G[dyk]), eps, moments=d(G[m]))
            errs[da], errs[dg], errs[db] = rel_max(G[da], wdx), rel_max(G[dg], wdg), rel_max(G[db], wdb)
        wdx, wdf, _ = ob.conv_backward(G["r2"], w["f3"], G["da3"], g3, want=(True, True, False))
        errs["dr2"], errs["df3"] = rel_max(G["dr2"], wdx), rel_max(G["df3"], wdf)
        assert bits_equal(G["dn2"], ob.relu_backward(G["n2"], G["dr2"]))
        wdx, wdf, _ = ob.conv_backward(G["r1"], w["f2"], G["da2"], g2, want=(True, True, False))
        errs["dr1"], errs["df2"] = rel_max(G["dr1"], wdx), rel_max(G["df2"], wdf)
        assert bits_equal(G["dn1"], ob.relu_backward(G["n1"], G["dr1"]))
        wdx, wdf, _ = ob.conv_backward(x, w["f1"], G["da1"], g1, want=(True, True, False))
        errs["dxm"], errs["df1"] = rel_max(G["dxm"], wdx), rel_max(G["df1"], wdf)
        assert bits_equal(G["dzdx"], ob.add(G["dxm"], G["ds"]))
        print("bottleneck N=32 stage errors:", {k: "%.1e" % v for k, v in errs.items()})
        for k, v in errs.items():
            gate = 1e-5 if k[0] in "nm" or k[:2] in ("da", "dg", "db") else 2e-4
            assert v <= gate, (k, v, gate)
        # end to end, forward only
        want_y = _oracle_bottleneck(ob, w, np.float32)["y"]
        assert rel_max(G["y"], want_y) < 2e-4
    finally:
        blk.close()


def test_bottleneck_fused_mode_is_bit_identical(vl, ob):
    """Folding ReLU and the shortcut sum into the batch-norm output pass changes no bit of any output."""
    w = workloads.bottleneck_case(N=4)
    outs = {}
    shapes = dict(y=w["x"].shape, dzdx=w["x"].shape, df1=w["f1"].shape, df2=w["f2"].shape, df3=w["f3"].shape,
                  dg1=(64,), db1=(64,), dg2=(64,), db2=(64,), dg3=(256,), db3=(256,), m1=(64, 2), m3=(256, 2))
    for fused in (False, True, "overlap"):
        blk = vl.Bottleneck(N=4, eps=w["eps"], fused=bool(fused), overlap=(fused == "overlap"))
        try:
            _load(blk, w)
            for _ in range(3 if fused == "overlap" else 1):  # (several steps: the second stream must be joined each time)
                blk.forward()
                blk.backward()
            outs[fused] = {k: blk.get(k, v) for k, v in shapes.items()}
        finally:
            blk.close()
    for k in shapes:
        assert bits_equal(outs[False][k], outs[True][k]), k
        assert bits_equal(outs[False][k], outs["overlap"][k]), k  # filter gradients on a second stream: same bits


def test_bnorm_forward_fused_matches_separate_calls(capi, ob):
    w = workloads.bnorm_case(seed=5, H=14, W=14, C=8, N=3)
    res = F(np.random.default_rng(6).standard_normal(w["x"].shape))
    xd, gd, bd, rd = capi.to_device(w["x"]), capi.to_device(w["g"]), capi.to_device(w["b"]), capi.to_device(res)
    y0, m0 = capi.bnorm_forward(xd, gd, bd, 1e-4)
    want = capi.relu_forward(capi.add(y0, rd))
    got, m1 = capi.bnorm_forward_fused(xd, gd, bd, residual=rd, relu=True, eps=1e-4)
    assert bits_equal(capi.to_host(got), capi.to_host(want)) and bits_equal(capi.to_host(m1), capi.to_host(m0))
    got, _ = capi.bnorm_forward_fused(xd, gd, bd, relu=True, eps=1e-4)
    assert bits_equal(capi.to_host(got), capi.to_host(capi.relu_forward(y0)))
    got, _ = capi.bnorm_forward_fused(xd, gd, bd, residual=rd, eps=1e-4)
    assert bits_equal(capi.to_host(got), capi.to_host(capi.add(y0, rd)))


def test_bnorm_backward_relu_matches_separate_calls(capi, ob):
    """ReLU's derivative folded into batch-norm's: bit-identical to the two calls, and right against the oracle."""
    w = workloads.bnorm_case(seed=9, H=14, W=18, C=8, N=5)
    d = lambda a: F(a, np.float64) if a.ndim > 1 else a.astype(np.float64)
    xd, gd, bd, dyd = (capi.to_device(w[k]) for k in ("x", "g", "b", "dy"))
    r, mom = capi.bnorm_forward_fused(xd, gd, bd, relu=True, eps=1e-4)
    masked = capi.relu_backward(r, dyd)
    want = capi.bnorm_backward(xd, gd, masked, 1e-4, moments=mom)
    got = capi.bnorm_backward_relu(xd, gd, bd, dyd, mom, 1e-4)
    for a, b_ in zip(got, want[:3]):
        assert bits_equal(capi.to_host(a), capi.to_host(b_))
    # against the oracle in double: forward, mask, backward
    y64, _ = ob.bnorm_forward(d(w["x"]), d(w["g"]), d(w["b"]), 1e-4)
    dy64 = d(w["dy"]) * (y64 > 0)
    odx, odg, odb, _ = ob.bnorm_backward(d(w["x"]), d(w["g"]), dy64, 1e-4)
    # (an element whose pre-activation is within rounding of 0 may be masked differently in float and double)
    flips = np.sum((capi.to_host(r) > 0) != (y64 > 0))
    if flips == 0:
        assert rel_max(capi.to_host(got[0]), odx) < 1e-5
        assert rel_max(capi.to_host(got[1]).ravel(), odg) < 1e-5 and rel_max(capi.to_host(got[2]).ravel(), odb) < 1e-5


def test_bnorm_backward_masked_matches_separate_calls(capi, ob):
    """A later ReLU's derivative taken (and written out) inside batch-norm's summing pass: same bits as the two calls."""
    w = workloads.bnorm_case(seed=12, H=14, W=18, C=8, N=5)
    r = np.random.default_rng(13)
    later = F(r.standard_normal(w["x"].shape))   # output of the later ReLU's layer: zeros, negatives, positives
    later[::3] = 0.0
    xd, gd, bd, dyd, ld = (capi.to_device(v) for v in (w["x"], w["g"], w["b"], w["dy"], later))
    _, mom = capi.bnorm_forward(xd, gd, bd, 1e-4)
    masked = capi.relu_backward(ld, dyd)
    want = capi.bnorm_backward(xd, gd, masked, 1e-4, moments=mom)
    got = capi.bnorm_backward_masked(xd, gd, dyd, ld, mom, 1e-4)
    for a, b_ in zip(got[:3], want[:3]):
        assert bits_equal(capi.to_host(a), capi.to_host(b_))
    assert bits_equal(capi.to_host(got[3]), capi.to_host(masked))


UNITS = [  # (H, W, C, M, Cout, stride, adapter): the kinds of segment ResNet-50 is made of, at reduced size
    (14, 14, 64, 16, 64, 1, False),     # plain segment, identity shortcut
    (14, 14, 32, 16, 64, 1, True),      # first segment of section 2: adapter, no downsampling
    (14, 14, 64, 32, 128, 2, True),     # first segment of sections 3-5: adapter and 3x3 layer with stride 2
    (13, 11, 64, 32, 128, 2, True),     # odd extents: the stride classes differ in size
]


@pytest.mark.parametrize("H,W,Cc,M,Cout,stride,adapter", UNITS)
def test_residual_unit_against_oracle_and_across_modes(vl, ob, H, W, Cc, M, Cout, stride, adapter):
    """Each kind of ResNet-50 segment, N = 3: against the unit composed from oracle operators (double), and the fused,
    two-stream and packed-ahead / deferred-sum schedules bit for bit against the layer-by-layer one."""
    w = workloads.bottleneck_case(seed=9, H=H, W=W, C=Cc, M=M, N=3, Cout=Cout, stride=stride, adapter=adapter)
    Ho, Wo = (H - 1) // stride + 1, (W - 1) // stride + 1
    shapes = dict(y=(Ho, Wo, Cout, 3), dzdx=w["x"].shape, df1=w["f1"].shape, df2=w["f2"].shape, df3=w["f3"].shape,
                  dg1=(M,), db1=(M,), dg2=(M,), db2=(M,), dg3=(Cout,), db3=(Cout,))
    names = ["x", "f1", "f2", "f3", "g1", "b1", "g2", "b2", "g3", "b3"]
    if adapter:
        shapes.update(dfs=w["fs"].shape, dgs=(Cout,), dbs=(Cout,))
        names += ["fs", "gs", "bs"]
    outs = {}
    for mode in ("plain", "fused", "overlap", "packed"):
        blk = vl.Bottleneck(H=H, W=W, Cc=Cc, M=M, N=3, eps=w["eps"], fused=mode != "plain", overlap=mode == "overlap",
                            Cout=Cout, stride=stride, adapter=adapter, packed=mode == "packed", deferred=mode == "packed")
        try:
            for k in names:
                blk.set(k, w[k])
            blk.set("dzdy", w["dy"])
            for _ in range(2):
                blk.forward()
                blk.backward()
            outs[mode] = {k: blk.get(k, v) for k, v in shapes.items()}
        finally:
            blk.close()
    want = _oracle_bottleneck(ob, w, np.float64)
    errs = {k: rel_max(outs["plain"][k], want[k]) for k in shapes}
    assert max(errs.values()) < 5e-4, errs
    for k in shapes:
        assert bits_equal(outs["plain"][k], outs["fused"][k]), k
        assert bits_equal(outs["plain"][k], outs["overlap"][k]), k
        assert bits_equal(outs["plain"][k], outs["packed"][k]), k


def test_timed_schedule_at_full_size_is_bit_identical_to_the_layer_by_layer_block(vl, ob):
    """The schedule bench.py times -- N = 32 at 56x56, batch-norm folding (fused), filter banks packed ahead
    (packed), one summing launch for the three filter gradients (deferred), stepped through `run` exactly as the
    bench steps it -- against the layer-by-layer block on the same inputs, every output bit for bit.  The
    layer-by-layer block is the one test_bottleneck_block_full_config_stage_by_stage checks against the oracle at
    this size; at this size the planner picks other unit widths, split counts and summing job tables than at the
    small batches of the tests above."""
    N = 32
    w = workloads.bottleneck_case()
    assert w["x"].shape == (56, 56, 256, N)
    shapes = dict(y=w["x"].shape, dzdx=w["x"].shape, df1=w["f1"].shape, df2=w["f2"].shape, df3=w["f3"].shape,
                  dg1=(64,), db1=(64,), dg2=(64,), db2=(64,), dg3=(256,), db3=(256,), m1=(64, 2), m2=(64, 2), m3=(256, 2))
    outs = {}
    for mode in ("plain", "timed"):
        timed = mode == "timed"
        blk = vl.Bottleneck(N=N, eps=w["eps"], fused=timed, packed=timed, deferred=timed)
        try:
            _load(blk, w)
            if timed:
                blk.run(2)          # two whole steps, as bench.py's warm-up and timed region run them
            else:
                for _ in range(2):
                    blk.forward()
                    blk.backward()
            torch.cuda.synchronize()
            outs[mode] = {k: blk.get(k, v) for k, v in shapes.items()}
        finally:
            blk.close()
    for k in shapes:
        assert np.isfinite(outs["plain"][k]).all(), k
        assert bits_equal(outs["plain"][k], outs["timed"][k]), k


def test_block_with_channel_sums_taken_by_the_convolutions(vl, ob):
    """The schedule in which the forward convolutions sum their own output per channel and the batch normalisations
    take those sums (no summing pass over a1, a2, a3), at the benchmarked size: moments within 1e-6 of the
    layer-by-layer block's (another summation order, both in double), every other output within 1e-4 of it (the
    moments' last bits move every normalised value a little), and the same bits on a second run."""
    N = 32
    w = workloads.bottleneck_case()
    shapes = dict(y=w["x"].shape, dzdx=w["x"].shape, df1=w["f1"].shape, df2=w["f2"].shape, df3=w["f3"].shape,
                  dg1=(64,), db1=(64,), dg2=(64,), db2=(64,), dg3=(256,), db3=(256,), m1=(64, 2), m2=(64, 2), m3=(256, 2))
    outs = {}
    for mode in ("plain", "sums", "sums again"):
        on = mode != "plain"
        blk = vl.Bottleneck(N=N, eps=w["eps"], fused=on, packed=on, deferred=on, epilogue_sums=on)
        try:
            _load(blk, w)
            if on:
                blk.run(2)
            else:
                blk.forward()
                blk.backward()
            torch.cuda.synchronize()
            outs[mode] = {k: blk.get(k, v) for k, v in shapes.items()}
        finally:
            blk.close()
    for k in shapes:
        assert bits_equal(outs["sums"][k], outs["sums again"][k]), k
        err = rel_max(outs["sums"][k], outs["plain"][k])
        assert err <= (1e-6 if k[0] == "m" else 1e-4), (k, err)


def test_block_with_channel_sums_against_the_oracle(vl, ob):
    """The same schedule on a small batch against the oracle in double (gate as for the other block tests: 5e-4 end to
    end).  Seed 6: with 1.2 million values entering each ReLU, about every other seed puts one of them within float
    rounding of zero, where single precision (the layer-by-layer block included) and the oracle in double pick
    different sides and one derivative moves by a whole element; this seed has none."""
    w = workloads.bottleneck_case(N=6, seed=6)
    shapes = dict(y=w["x"].shape, dzdx=w["x"].shape, df1=w["f1"].shape, df2=w["f2"].shape, df3=w["f3"].shape,
                  dg1=(64,), db1=(64,), dg2=(64,), db2=(64,), dg3=(256,), db3=(256,))
    blk = vl.Bottleneck(N=6, eps=w["eps"], fused=True, packed=True, deferred=True, epilogue_sums=True)
    try:
        _load(blk, w)
        blk.run(1)
        torch.cuda.synchronize()
        got = {k: blk.get(k, v) for k, v in shapes.items()}
    finally:
        blk.close()
    want = _oracle_bottleneck(ob, w, np.float64)
    errs = {k: rel_max(got[k], want[k]) for k in shapes}
    assert max(errs.values()) < 5e-4, errs


def test_block_with_the_last_relu_mask_kept_as_bits(vl, ob):
    """The benchmarked schedule with the unit's last ReLU mask kept as one bit per element (backward reads 3 MB of bits
    instead of the 103 MB output; the shortcut's share of the derivative is added in the epilogue of the first
    convolution's input gradient) against the same schedule without: every output bit for bit, at the benchmarked
    size, two steps."""
    N = 32
    w = workloads.bottleneck_case()
    shapes = dict(y=w["x"].shape, dzdx=w["x"].shape, df1=w["f1"].shape, df2=w["f2"].shape, df3=w["f3"].shape,
                  dg1=(64,), db1=(64,), dg2=(64,), db2=(64,), dg3=(256,), db3=(256,), m1=(64, 2), m2=(64, 2), m3=(256, 2))
    outs = {}
    for bits in (False, True):
        blk = vl.Bottleneck(N=N, eps=w["eps"], fused=True, packed=True, deferred=True, epilogue_sums=True, mask_bits=bits)
        try:
            assert blk.mask_bits == bits          # (this shape has the form: 56x56 planes are whole mask words)
            _load(blk, w)
            blk.run(2)
            torch.cuda.synchronize()
            outs[bits] = {k: blk.get(k, v) for k, v in shapes.items()}
        finally:
            blk.close()
    for k in shapes:
        assert np.isfinite(outs[True][k]).all(), k
        assert bits_equal(outs[False][k], outs[True][k]), k
    # a unit whose planes are not whole mask words keeps the float mask, silently
    blk = vl.Bottleneck(H=14, W=14, Cc=256, M=64, N=4, eps=1e-5, fused=True, packed=True, deferred=True, epilogue_sums=True, mask_bits=True)
    try:
        assert blk.mask_bits is False
    finally:
        blk.close()


def test_timed_schedule_batch_norm_stages_against_the_double_oracle_at_full_size(vl, ob):
    """The batch-norm stages of the benchmarked schedule (moments from the convolutions' own channel sums, ReLU and the
    shortcut sum folded into the output pass, the last mask as bits) at N = 32, each against the oracle in double on
    the stage's OWN inputs -- the block's buffers -- at 1e-5: the moments, what the output pass writes, and the three
    derivatives of every stage.  (A mask is what the forward pass wrote: r > 0.)"""
    N = 32
    w = workloads.bottleneck_case()
    blk = vl.Bottleneck(N=N, eps=w["eps"], fused=True, packed=True, deferred=True, epilogue_sums=True, mask_bits=True)
    try:
        _load(blk, w)
        blk.run(1)
        torch.cuda.synchronize()
        big, small = (56, 56, 256, N), (56, 56, 64, N)
        shp = dict(a1=small, r1=small, a2=small, r2=small, a3=big, y=big, m1=(64, 2), m2=(64, 2), m3=(256, 2),
                   da3=big, dr2=small, da2=small, dr1=small, da1=small,
                   dg1=(64,), db1=(64,), dg2=(64,), db2=(64,), dg3=(256,), db3=(256,))
        G = {k: blk.get(k, v) for k, v in shp.items()}
    finally:
        blk.close()
    x, dy, eps = w["x"], w["dy"], w["eps"]
    d = lambda a: F(a, np.float64) if a.ndim > 1 else a.astype(np.float64)
    errs = {}
    # forward: moments and the written output (ReLU, and for the last stage the shortcut sum, included)
    for a, r, m, gk, bk, add in [("a1", "r1", "m1", "g1", "b1", None), ("a2", "r2", "m2", "g2", "b2", None),
                                 ("a3", "y", "m3", "g3", "b3", x)]:
        wy, wm = ob.bnorm_forward(d(G[a]), d(w[gk]), d(w[bk]), eps)
        if add is not None:
            wy = wy + d(add)
        errs[m] = rel_max(G[m], wm)
        errs[r] = rel_max(G[r], np.maximum(wy, 0))
    # backward: the derivative that enters each stage, masked by what the forward pass wrote
    for da, dg, db, a, m, gk, dz, r in [("da3", "dg3", "db3", "a3", "m3", "g3", dy, "y"),
                                        ("da2", "dg2", "db2", "a2", "m2", "g2", G["dr2"], "r2"),
                                        ("da1", "dg1", "db1", "a1", "m1", "g1", G["dr1"], "r1")]:
        dn = d(dz) * (G[r] > 0)
        wdx, wdg, wdb, _ = ob.bnorm_backward(d(G[a]), d(w[gk]), dn, eps, moments=d(G[m]))
        errs[da], errs[dg], errs[db] = rel_max(G[da], wdx), rel_max(G[dg], wdg), rel_max(G[db], wdb)
    print("timed schedule, batch-norm stages at N=32:", {k: "%.1e" % v for k, v in errs.items()})
    for k, v in errs.items():
        assert v <= 1e-5, (k, v)


def test_timed_schedule_with_filter_gradients_on_a_second_stream(vl, ob):
    """The benchmarked schedule with the three filter-gradient matrix kernels on a second stream (they run beside the
    batch-norm derivatives of the layer below; the sums over their reduction splits follow the join, in one launch)
    against the same schedule on one stream: every output bit for bit, at the benchmarked size, three steps (the
    second stream is joined at the end of each)."""
    N = 32
    w = workloads.bottleneck_case()
    shapes = dict(y=w["x"].shape, dzdx=w["x"].shape, df1=w["f1"].shape, df2=w["f2"].shape, df3=w["f3"].shape,
                  dg1=(64,), db1=(64,), dg2=(64,), db2=(64,), dg3=(256,), db3=(256,), m1=(64, 2), m2=(64, 2), m3=(256, 2))
    outs = {}
    for two in (False, True):
        blk = vl.Bottleneck(N=N, eps=w["eps"], fused=True, overlap=two, packed=True, deferred=True, epilogue_sums=True,
                            mask_bits=True)
        try:
            _load(blk, w)
            blk.run(3)
            torch.cuda.synchronize()
            outs[two] = {k: blk.get(k, v) for k, v in shapes.items()}
        finally:
            blk.close()
    for k in shapes:
        assert np.isfinite(outs[True][k]).all(), k
        assert bits_equal(outs[False][k], outs[True][k]), k
