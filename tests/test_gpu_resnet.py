"""ResNet-50 forward + backward driven through the C++ operator classes (examples/imagenet/cnn_imagenet_init_resnet.m:
52-134), at reduced image size, against the network composed from oracle operators."""
import numpy as np
import pytest

from matconvnet_amd import workloads
from util import bits_equal, rel_max

pytestmark = pytest.mark.gpu

S, N, CLASSES = 64, 4, 10
UNIT_PARAMS = ("f1", "f2", "f3", "g1", "b1", "g2", "b2", "g3", "b3")
ADAPTER_PARAMS = ("fs", "gs", "bs")


def _load(net, w):
    net.set("input", w["input"])
    net.set("dprediction", w["dprediction"])
    for k in "fgb":
        net.set("stem." + k, w["stem"][k])
    for i, u in enumerate(w["units"]):
        for k in UNIT_PARAMS + (ADAPTER_PARAMS if u["adapter"] else ()):
            net.set("unit%d.%s" % (i, k), u[k])
    net.set("fc.f", w["fc"]["f"])
    net.set("fc.b", w["fc"]["b"])


def _gradient_names(w):
    names = ["prediction", "fc.df", "fc.db", "stem.df", "stem.dg", "stem.db"]
    for i, u in enumerate(w["units"]):
        names += ["unit%d.d%s" % (i, k) for k in UNIT_PARAMS + (ADAPTER_PARAMS if u["adapter"] else ())]
        names += ["unit%d.y" % i, "unit%d.dzdx" % i]
    return names


@pytest.fixture(scope="module")
def case():
    return workloads.resnet50_case(seed=9, image_size=S, N=N, classes=CLASSES)


@pytest.fixture(scope="module")
def runs(vl, case):
    """Every output buffer of the network after two forward + backward passes, layer by layer and fused."""
    out = {}
    for mode in ("plain", "fused"):
        net = vl.ResNet50(N=N, eps=case["eps"], image_size=S, classes=CLASSES, fused=mode == "fused")
        try:
            assert net.units == 16
            _load(net, case)
            for _ in range(2):
                net.forward()
                net.backward()
            got = {k: net.get(k) for k in _gradient_names(case)}
            got["stem.p"] = net.get("stem.p")
            got["stem.dp"] = net.get("stem.dp")
            got["unit15.dzdy"] = net.get("unit15.dzdy")
            if mode == "plain":   # the tensors ReLU and max pooling take their masks from
                got["stem.n"], got["stem.r"] = net.get("stem.n"), net.get("stem.r")
                for i in range(net.units):
                    for k in ("n1", "n2", "s"):
                        got["unit%d.%s" % (i, k)] = net.get("unit%d.%s" % (i, k))
            out[mode] = got
        finally:
            net.close()
    return out


def test_fused_schedule_is_bit_identical(runs, case):
    for k in _gradient_names(case):
        assert bits_equal(runs["plain"][k], runs["fused"][k]), k


def test_prediction_end_to_end(runs, case, ob):
    """Forward pass of the whole network against the oracle network (float and double)."""
    from oracle import blocks
    want = blocks.resnet50(case, np.float64)
    got = runs["plain"]["prediction"].reshape(want["prediction"].shape, order="F")
    assert np.isfinite(got).all()
    assert rel_max(got, want["prediction"]) < 1e-3


def test_stage_by_stage_against_oracle(runs, case, ob):
    """ReLU's derivative is discontinuous and the deepest sections normalise over few samples, so the gradients of
    the whole network are not a continuous function of rounding error (the oracle in float and in double differ by
    several percent there).  Each stage is therefore checked on the inputs the device network actually gave it: the
    stage's input and incoming derivative are read back from the device, the oracle stage runs on them in double, and
    every output of the device's stage is compared.  A stage's input buffer is its predecessor's output buffer, so the
    chain of checks covers the wiring as well.  Inside a stage the tensors that ReLU and max pooling derive their masks
    from are compared with the oracle's and then taken from the device, so that a value within rounding of zero (or
    of its neighbour in a pooling window) selects the same elements on both sides."""
    from oracle import binding
    from oracle import blocks
    G = runs["plain"]
    f64 = lambda a: np.asfortranarray(a, dtype=np.float64) if a.ndim > 1 else a.astype(np.float64)
    shaped = lambda name, like: G[name].reshape(like.shape, order="F")
    errs = {}

    # stem: input -> pooled map; pooled derivative -> parameter derivatives
    st, eps = case["stem"], case["eps"]
    x = f64(case["input"])
    g0 = binding.conv_geom(x.shape, st["f"].shape, 2, 3, 1)
    a0 = binding.conv_forward(x, f64(st["f"]), None, g0)
    n0, m0 = binding.bnorm_forward(a0, f64(st["g"]), f64(st["b"]), eps)
    r0 = binding.relu_forward(n0)
    gp = binding.pool_geom(r0.shape, 3, 2, 1, "max")
    p0 = binding.pool_forward(r0, gp)
    assert p0.shape == (S // 4, S // 4, 64, N)
    errs["stem.p"] = rel_max(shaped("stem.p", p0), p0)
    errs["stem.n"] = rel_max(shaped("stem.n", n0), n0)
    errs["stem.r"] = rel_max(shaped("stem.r", r0), r0)
    n0, r0 = f64(shaped("stem.n", n0)), f64(shaped("stem.r", r0))
    dp = f64(shaped("stem.dp", p0))
    dr0 = binding.pool_backward(r0, dp, gp)
    dn0 = binding.relu_backward(n0, dr0)
    da0, dg0, db0, _ = binding.bnorm_backward(a0, f64(st["g"]), dn0, eps, moments=m0)
    _, df0, _ = binding.conv_backward(x, f64(st["f"]), da0, g0, want=(False, True, False))
    errs["stem.df"] = rel_max(shaped("stem.df", df0), df0)
    errs["stem.dg"] = rel_max(G["stem.dg"], dg0)
    errs["stem.db"] = rel_max(G["stem.db"], db0)

    # units: input = the device's previous output, incoming derivative = the device's next dzdx
    h = f64(shaped("stem.p", p0))
    states = []
    for i, u in enumerate(case["units"]):
        t = blocks.unit_forward(u, h, np.float64)
        states.append(t)
        errs["unit%d.y" % i] = rel_max(shaped("unit%d.y" % i, t["y"]), t["y"])
        for k in ("n1", "n2", "s"):
            name = "unit%d.%s" % (i, k)
            errs[name] = rel_max(shaped(name, t[k]), t[k])
            t[k] = f64(shaped(name, t[k]))
        h = f64(shaped("unit%d.y" % i, t["y"]))
    last = states[-1]["y"]
    assert last.shape == (S // 32, S // 32, 2048, N)
    for i, u in enumerate(case["units"]):
        nxt = "unit%d.dzdx" % (i + 1) if i + 1 < len(case["units"]) else "unit15.dzdy"
        dy = f64(G[nxt].reshape(states[i]["y"].shape, order="F"))
        g = blocks.unit_backward(u, states[i], dy, np.float64)
        for k, v in g.items():
            name = "unit%d.%s" % (i, k)
            errs[name] = rel_max(G[name].reshape(v.shape, order="F"), v)
    # the first unit's dzdx is the buffer the stem reads
    assert bits_equal(G["unit0.dzdx"], G["stem.dp"])

    # head: average pooling over the whole map, 1x1 convolution with bias
    ga = binding.pool_geom(h.shape, (h.shape[0], h.shape[1]), 1, 0, "avg")
    avg = binding.pool_forward(h, ga)
    ff, fb = f64(case["fc"]["f"]), f64(case["fc"]["b"])
    gf = binding.conv_geom(avg.shape, ff.shape, 1, 0, 1)
    pred = binding.conv_forward(avg, ff, fb, gf)
    errs["prediction"] = rel_max(shaped("prediction", pred), pred)
    davg, dff, dfb = binding.conv_backward(avg, ff, f64(case["dprediction"]), gf)
    dlast = binding.pool_backward(h, davg, ga)
    errs["fc.df"] = rel_max(shaped("fc.df", dff), dff)
    errs["fc.db"] = rel_max(G["fc.db"], dfb)
    errs["unit15.dzdy"] = rel_max(shaped("unit15.dzdy", dlast), dlast)

    worst = sorted(errs.items(), key=lambda kv: -kv[1])[:6]
    print("ResNet-50 %dx%d N=%d, worst stage errors:" % (S, S, N), {k: "%.1e" % v for k, v in worst})
    assert all(np.isfinite(v) for v in errs.values())
    assert max(errs.values()) < 1e-4, worst


def test_seeded_initialisation_runs_at_full_image_size(vl):
    """224 x 224 images, 1000 classes, N = 2: the reference geometry end to end (7 x 7 average pooling, finite outputs,
    gradients that are not identically zero)."""
    net = vl.ResNet50(N=2, eps=1e-5, image_size=224, classes=1000, fused=True, seed=3)
    try:
        r = np.random.default_rng(4)
        net.set("input", np.asfortranarray(r.standard_normal((224, 224, 3, 2), dtype=np.float32)))
        net.set("dprediction", np.asfortranarray(r.standard_normal((1, 1, 1000, 2), dtype=np.float32)))
        net.forward()
        net.backward()
        assert abs(net.forward_flops_per_image / 1e9 - 8.178) < 0.001   # 4.09 G multiply-adds
        for name in ("prediction", "stem.df", "unit0.dfs", "unit7.df2", "unit15.dg3", "fc.df", "fc.db"):
            v = net.get(name)
            assert np.isfinite(v).all() and np.abs(v).max() > 0, name
    finally:
        net.close()


def test_sgd_step_follows_the_reference_solver(vl, ob, case):
    """Two training steps (forward, backward, update).  After each, every parameter, its momentum and the moving
    averages of the moments equal, bit for bit, what the three vl_taccum calls per parameter of
    examples/cnn_train_dag.m:335-364 (oracle, float) give from the state before the step and the derivatives the
    device computed; rates as examples/imagenet/cnn_imagenet_init_resnet.m:178-195 sets them."""
    lr, mom, wd = 0.1, 0.9, 1e-4
    net = vl.ResNet50(N=N, eps=case["eps"], image_size=S, classes=CLASSES, fused=True)
    try:
        _load(net, case)
        names = [("stem." + k, "stem.d" + k) for k in "fgb"]
        moments = ["stem.m"]
        for i, u in enumerate(case["units"]):
            names += [("unit%d.%s" % (i, k), "unit%d.d%s" % (i, k)) for k in UNIT_PARAMS + (ADAPTER_PARAMS if u["adapter"] else ())]
            moments += ["unit%d.m%s" % (i, k) for k in ("1", "2", "3") + (("s",) if u["adapter"] else ())]
        names += [("fc.f", "fc.df"), ("fc.b", "fc.db")]
        assert net.parameters == sum(net.get(v).size for v, _ in names)
        f32 = np.float32
        for step in range(2):
            before = {v: (net.get(v), net.get("momentum." + v)) for v, _ in names}
            running = {m: net.get("running." + m) for m in moments}
            net.forward()
            net.backward()
            net.sgd_step(lr, mom, wd)
            for v, d in names:
                value, state = before[v]
                der = net.get(d)
                this_lr = lr / 100.0 ** 2 if v == "stem.f" else lr
                g = ob.taccum(1.0, der, wd, value)
                s_new = ob.taccum(mom, state, -1.0, g)
                v_new = ob.taccum(1.0, value, this_lr, s_new)
                assert bits_equal(net.get("momentum." + v), s_new), (step, v)
                assert bits_equal(net.get(v), v_new), (step, v)
                assert np.abs(v_new - value).max() > 0, v
            for m in moments:
                want = ob.taccum(1.0 - 0.3, running[m], 0.3, net.get(m))
                assert bits_equal(net.get("running." + m), want), (step, m)
    finally:
        net.close()


def test_test_mode_uses_the_stored_moments(vl, case):
    """Evaluation mode (matlab/+dagnn/BatchNorm.m:12-17): with the moving averages set to the batch's own moments the
    prediction is the training-mode one; with other moments it is not; fused and layer-by-layer agree bit for bit;
    backward is refused."""
    from matconvnet_amd.vlapi import VlError
    outs = {}
    for fused in (False, True):
        net = vl.ResNet50(N=N, eps=case["eps"], image_size=S, classes=CLASSES, fused=fused)
        try:
            _load(net, case)
            net.forward()
            train = net.get("prediction")
            moments = ["stem.m"]
            for i, u in enumerate(case["units"]):
                moments += ["unit%d.m%s" % (i, k) for k in ("1", "2", "3") + (("s",) if u["adapter"] else ())]
            net.set_test_mode(True)
            net.forward()
            zero_moments = net.get("prediction")          # running moments still zero: mean 0, sigma 0
            assert not np.allclose(zero_moments, train, rtol=1e-3, atol=1e-3)
            for m in moments:
                net.set("running." + m, net.get(m))
            net.forward()
            outs[fused] = net.get("prediction")
            assert rel_max(outs[fused], train) < 1e-6
            with pytest.raises(VlError, match="training-mode"):
                net.backward()
            net.set_test_mode(False)
            net.forward()
            net.backward()
        finally:
            net.close()
    assert bits_equal(outs[False], outs[True])


def test_filters_packed_ahead_and_deferred_sums_change_no_bit(vl, case):
    """All convolutions reading banks packed ahead by one launch (after uploads, and after every update), and all
    filter gradients finished by one summing launch at the end of backward, against every call packing and summing
    for itself: predictions, gradients, and the parameters after two training steps."""
    lr, mom, wd = 0.05, 0.9, 1e-4
    watch = _gradient_names(case) + ["stem.f", "unit0.f1", "unit3.f2", "unit3.fs", "unit15.f3", "fc.f", "momentum.unit7.f2"]
    seen = {}
    for packed in (False, True):
        net = vl.ResNet50(N=N, eps=case["eps"], image_size=S, classes=CLASSES, fused=True, packed=packed, deferred=packed)  # (deferred is off by default)
        try:
            _load(net, case)
            for _ in range(2):
                net.forward()
                net.backward()
                net.sgd_step(lr, mom, wd)
            net.forward()
            net.backward()
            seen[packed] = {k: net.get(k) for k in watch}
        finally:
            net.close()
    for k in watch:
        assert bits_equal(seen[False][k], seen[True][k]), k
    assert not bits_equal(seen[True]["unit3.f2"], np.asfortranarray(case["units"][3]["f2"]).ravel(order="F"))


def test_graph_replays_match_eager_steps(vl, case):
    """A training step and an evaluation pass recorded into HIP graphs: every replay -- with uploads, downloads and
    device synchronisations of the program between them, and the input changed from one to the next -- leaves the same
    bits in the parameters, the momentum, the moving averages and the prediction as the same calls made eagerly."""
    import torch
    from matconvnet_amd.vlapi import VlError
    lr, mom, wd = 0.002, 0.9, 1e-4   # (small: at 0.05 four steps on random data already blow the evaluation pass up to 1e34)
    r = np.random.default_rng(77)
    inputs = [np.asfortranarray(r.standard_normal((S, S, 3, N), dtype=np.float32)) for _ in range(3)]
    watch = ["prediction", "stem.f", "momentum.stem.f", "running.stem.m", "unit0.fs", "unit7.g2", "momentum.unit7.f2",
             "running.unit15.m3", "unit15.f3", "fc.f", "fc.b", "momentum.fc.b"]
    stream = torch.cuda.Stream()
    history = {}
    with torch.cuda.stream(stream):
        for mode in ("eager", "graph"):
            net = vl.ResNet50(N=N, eps=case["eps"], image_size=S, classes=CLASSES, fused=True)
            try:
                _load(net, case)
                if mode == "graph":
                    with pytest.raises(VlError, match="nothing has been captured"):
                        net.replay()
                net.forward(); net.backward(); net.sgd_step(lr, mom, wd)     # (also sizes the workspace)
                if mode == "graph":
                    net.capture(True, lr, mom, wd)
                seen = []
                for x in inputs:
                    net.set("input", x)
                    if mode == "graph":
                        net.replay()
                    else:
                        net.forward(); net.backward(); net.sgd_step(lr, mom, wd)
                    seen.append({k: net.get(k) for k in watch})
                # evaluation with the moving averages the steps above left
                net.set_test_mode(True)
                net.forward()
                if mode == "graph":
                    net.capture(False)
                for x in inputs:
                    net.set("input", x)
                    if mode == "graph":
                        net.replay()
                    else:
                        net.forward()
                    seen.append({"prediction": net.get("prediction")})
                history[mode] = seen
            finally:
                net.close()
    for i, (a, b) in enumerate(zip(history["eager"], history["graph"])):
        for k in a:
            assert np.isfinite(a[k]).all(), (i, k)
            assert bits_equal(a[k], b[k]), (i, k)
    assert not bits_equal(history["eager"][0]["fc.f"], history["eager"][2]["fc.f"])
    assert not bits_equal(history["eager"][3]["prediction"], history["eager"][4]["prediction"])


def test_capture_needs_a_stream_of_its_own(vl):
    from matconvnet_amd.vlapi import VlError
    net = vl.ResNet50(N=1, image_size=32, classes=4, seed=1)
    try:
        net.forward()
        with pytest.raises(VlError, match="default stream"):
            net.capture(False)
    finally:
        net.close()


def test_image_size_must_be_a_multiple_of_32(vl):
    from matconvnet_amd.vlapi import VlError
    with pytest.raises(VlError, match="multiple of 32"):
        vl.ResNet50(N=1, image_size=100)


def test_loss_layers_and_a_few_training_steps(vl, case):
    """The network's last layers (softmax log-loss, top-1 / top-5 error; cnn_imagenet_init_resnet.m:128-139) on the
    device: their values and the derivative the backward pass starts from against the numpy restatement of
    vl_nnloss.m; then whole training steps (forward, loss derivative, backward, SGD) on one fixed batch lower that
    batch's loss."""
    from oracle import loss as ol
    r = np.random.default_rng(31)
    net = vl.ResNet50(N=N, eps=case["eps"], image_size=S, classes=CLASSES, fused=True)
    try:
        _load(net, case)
        labels = r.integers(1, CLASSES + 1, N).astype(np.float32)
        labels[-1] = 0.0   # (a skipped image)
        net.set("labels", np.asfortranarray(labels.reshape(1, 1, 1, N)))
        net.forward()
        net.loss_derivative()
        pred = np.asfortranarray(net.get("prediction").reshape(1, 1, CLASSES, N, order="F"))
        objective, top1, top5 = net.losses()
        assert abs(objective - float(ol.vl_nnloss(pred, labels, None, loss="softmaxlog"))) < 1e-5 * max(1.0, abs(objective))
        assert top1 == pytest.approx(float(ol.vl_nnloss(pred, labels, None, loss="classerror")), abs=1e-6)
        assert top5 == pytest.approx(float(ol.vl_nnloss(pred, labels, None, loss="topkerror", top_k=5)), abs=1e-6)
        want = ol.vl_nnloss(pred, labels, 1.0, loss="softmaxlog")
        got = net.get("dprediction").reshape(1, 1, CLASSES, N, order="F")
        assert rel_max(got, want) < 1e-5 and not got[..., -1].any()
        first = objective
        for _ in range(12):   # (a rate at which the trajectory is stable: at 0.05 the loss of this batch bounces)
            net.forward()
            net.loss_derivative()
            net.backward()
            net.sgd_step(0.01, 0.9, 1e-4)
        net.forward()
        last = net.losses()[0]
        assert np.isfinite(last) and last < 0.3 * first, (first, last)
    finally:
        net.close()


def test_channel_sums_schedule_of_the_whole_network(vl):
    """The network with the forward convolutions summing their own output per channel and the identity units keeping
    their last ReLU's mask as bits (ResNet50(channel_sums=True); engaged by the 56x56 units at this size).  Forward:
    against the folded schedule without, to rounding (the moments come from another summation order).  Backward: the
    whole network's gradients are not continuous in rounding error (see test_stage_by_stage_against_oracle), so the
    second unit -- identity shortcut, 56x56: both forms engaged -- is checked on the tensors the network actually gave
    it: a stand-alone layer-by-layer unit run on the network's input and incoming derivative of that unit must give
    the network's outputs of that unit.  And two runs give the same bits."""
    B = 8
    w = workloads.resnet50_case(seed=4, image_size=224, N=B, classes=10)
    names = ("prediction", "unit0.y", "unit1.y", "unit2.dzdx", "unit1.dzdx") + tuple("unit1.d" + k for k in UNIT_PARAMS)
    outs = []
    for kw in (dict(), dict(channel_sums=True), dict(channel_sums=True)):
        net = vl.ResNet50(N=B, eps=w["eps"], image_size=224, classes=10, fused=True, **kw)
        try:
            _load(net, w)
            net.forward()
            net.backward()
            outs.append({k: net.get(k) for k in names})
        finally:
            net.close()
    plain, sums, again = outs
    for k in names:
        assert np.isfinite(sums[k]).all(), k
        assert bits_equal(sums[k], again[k]), k
    for k, gate in (("unit0.y", 1e-5), ("unit1.y", 1e-5), ("prediction", 1e-4)):   # (fifty layers later: 1e-5 measured)
        assert rel_max(sums[k], plain[k]) < gate, (k, rel_max(sums[k], plain[k]))
    u = w["units"][1]
    assert not u["adapter"]
    shape = (56, 56, 256, B)
    blk = vl.Bottleneck(H=56, W=56, Cc=256, M=64, N=B, eps=w["eps"])
    try:
        blk.set("x", sums["unit0.y"].reshape(shape, order="F"))
        blk.set("dzdy", sums["unit2.dzdx"].reshape(shape, order="F"))
        for k in UNIT_PARAMS:
            blk.set(k, u[k])
        blk.forward()
        blk.backward()
        assert rel_max(blk.get("y", shape).ravel(order="F"), sums["unit1.y"].ravel(order="F")) < 1e-5
        errs = {"dzdx": rel_max(blk.get("dzdx", shape).ravel(order="F"), sums["unit1.dzdx"].ravel(order="F"))}
        for k in UNIT_PARAMS:
            errs["d" + k] = rel_max(blk.get("d" + k, np.shape(u[k])).ravel(order="F"), sums["unit1.d" + k].ravel(order="F"))
        assert max(errs.values()) < 2e-4, errs
    finally:
        blk.close()


@pytest.mark.parametrize("deferred", [False, True])
def test_filter_gradients_on_a_second_stream_change_no_bit(vl, case, deferred):
    """backward() with every unit's filter gradients on a second stream of the network's (joined once, at the end)
    against the one-stream schedule: gradients after two passes, parameters after two training steps, and the same
    training step replayed three times from a HIP graph (the fork and the join are recorded with it)."""
    import torch
    lr, mom, wd = 0.002, 0.9, 1e-4
    watch = _gradient_names(case) + ["stem.f", "unit0.f1", "unit3.f2", "unit3.fs", "unit15.f3", "fc.f", "momentum.unit7.f2"]
    seen = {}
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for two in (False, True):
            net = vl.ResNet50(N=N, eps=case["eps"], image_size=S, classes=CLASSES, fused=True, deferred=deferred, overlap=two)
            try:
                _load(net, case)
                for _ in range(2):
                    net.forward()
                    net.backward()
                    net.sgd_step(lr, mom, wd)
                net.forward()
                net.backward()
                got = {k: net.get(k) for k in watch}
                net.capture(True, lr, mom, wd)
                for i in range(3):
                    net.replay()
                    torch.cuda.synchronize()
                    got["replay%d" % i] = np.concatenate([net.get(k).ravel() for k in ("stem.f", "unit7.f2", "unit15.f3", "fc.f")])
                seen[two] = got
            finally:
                net.close()
    for k in seen[False]:
        assert np.isfinite(seen[True][k]).all(), k
        assert bits_equal(seen[False][k], seen[True][k]), k
    assert not bits_equal(seen[True]["replay0"], seen[True]["replay2"])
