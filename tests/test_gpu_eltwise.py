"""GPU parity of the element-wise companions (ReLU, sum, scaled sum, fill): bit-exact against the oracle."""
import numpy as np
import pytest

from util import F, bits_equal

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 3, 4, 5, 255, 1024, 100003])
def test_relu_add_fill(capi, ob, n):
    r = np.random.default_rng(n)
    x = r.standard_normal(n).astype(np.float32)
    x[::7] = 0.0
    if n > 4:
        x[3] = np.nan
        x[4] = -0.0
    dy = r.standard_normal(n).astype(np.float32)
    xd, dyd = capi.to_device(x), capi.to_device(dy)
    assert bits_equal(capi.to_host(capi.relu_forward(xd)), ob.relu_forward(x))
    assert bits_equal(capi.to_host(capi.relu_backward(xd, dyd)), ob.relu_backward(x, dy))
    assert bits_equal(capi.to_host(capi.add(xd, dyd)), ob.add(x, dy))
    t = capi.empty((n,))
    capi.fill(t, 1.5)
    assert np.array_equal(capi.to_host(t), np.full(n, 1.5, np.float32))


def test_unaligned_views(capi, ob):
    """Pointers that are only 4-byte aligned take the scalar path."""
    import torch
    base = torch.randn(1001, device="cuda")
    x = base[1:]
    y = torch.empty(1001, device="cuda")[1:]
    capi.check(capi.lib().mcn_relu_forward(capi.stream(), capi.ptr(y), capi.ptr(x), x.numel()))
    assert torch.equal(y, torch.clamp_min(x, 0))


@pytest.mark.parametrize("n", [1, 5, 1024, 100003])
def test_taccum(capi, ob, n):
    """alpha*a + beta*b, out of place and in place, bit for bit the scal + axpy pair of the oracle."""
    r = np.random.default_rng(n + 1)
    a = r.standard_normal(n).astype(np.float32)
    b = r.standard_normal(n).astype(np.float32)
    want = ob.taccum(0.9, a, -0.0123, b)
    ad, bd = capi.to_device(a), capi.to_device(b)
    assert bits_equal(capi.to_host(capi.taccum(0.9, ad, -0.0123, bd)), want)
    capi.taccum(0.9, ad, -0.0123, bd, out=ad)
    assert bits_equal(capi.to_host(ad), want)


def test_vl_taccum_driver(ob):
    """The MEX conventions: a new array without options, the first array updated with 'InPlace'."""
    import torch
    from matconvnet_amd import vlapi as vl
    r = np.random.default_rng(4)
    a = F(r.standard_normal((6, 5, 4, 3)))
    b = F(r.standard_normal((6, 5, 4, 3)))
    dev = lambda v: torch.from_numpy(np.ascontiguousarray(v.transpose(3, 2, 1, 0))).cuda()
    host = lambda t: np.asfortranarray(t.cpu().numpy().transpose(3, 2, 1, 0))
    want = ob.taccum(0.5, a, 2.0, b)
    ad, bd = dev(a), dev(b)
    y = vl.vl_taccum(0.5, ad, 2.0, bd)
    assert bits_equal(host(y), want) and bits_equal(host(ad), a)
    same = vl.vl_taccum(0.5, ad, 2.0, bd, "inplace")
    assert same is ad and bits_equal(host(ad), want)


@pytest.mark.parametrize("nesterov", [False, True])
def test_sgd_momentum_arena_matches_the_reference_call_sequence(capi, ob, nesterov):
    """One launch over all parameters against the three vl_taccum calls per parameter of
    examples/cnn_train_dag.m:335-364 (oracle, float): same bits, for parameters with their own learning-rate and
    weight-decay multipliers, one of them frozen (both rates 0), sizes that are not multiples of the chunk."""
    import torch
    counts = [7 * 7 * 3 * 64, 64, 64, 1024, 3 * 3 * 16 * 16, 1, 5000]
    mults = [(0.0001, 1.0), (1.0, 1.0), (1.0, 0.0), (0.0, 0.0), (1.0, 1.0), (2.0, 0.5), (1.0, 1.0)]
    lr, wd, mom, workers = 0.1, 1e-4, 0.9, 4
    offsets, chunks, chunk_param = capi.sgd_arena_layout(counts)
    r = np.random.default_rng(21)
    n = chunks * capi.SGD_CHUNK
    value, state, der = (np.zeros(n, np.float32) for _ in range(3))
    for off, c in zip(offsets, counts):
        value[off:off + c] = r.standard_normal(c)
        state[off:off + c] = 0.1 * r.standard_normal(c)
        der[off:off + c] = r.standard_normal(c)
    vd, sd, dd = (torch.from_numpy(a.copy()).cuda() for a in (value, state, der))
    capi.sgd_momentum(vd, sd, dd, torch.from_numpy(chunk_param).cuda(),
                      torch.tensor(mults, dtype=torch.float64).cuda(), lr, wd, mom, der_scale=1.0 / workers,
                      nesterov=nesterov)
    got_v, got_s = vd.cpu().numpy(), sd.cpu().numpy()
    assert bits_equal(dd.cpu().numpy(), der)
    f32 = np.float32
    for off, c, (lm, dm) in zip(offsets, counts, mults):
        v, s_, d = value[off:off + c], state[off:off + c], der[off:off + c]
        this_lr, this_decay = lr * lm, wd * dm
        if this_lr > 0 or this_decay > 0:
            g = ob.taccum(1.0 / workers, d, this_decay, v)
            s_new = ob.taccum(mom, s_, -1.0, g)
            delta = (f32(mom) * s_new - g).astype(f32) if nesterov else s_new
            v_new = ob.taccum(1.0, v, this_lr, delta)
        else:
            s_new, v_new = s_, v
        assert bits_equal(got_s[off:off + c], s_new), (off, c)
        assert bits_equal(got_v[off:off + c], v_new), (off, c)
    # padding stays zero
    pad = np.ones(n, bool)
    for off, c in zip(offsets, counts):
        pad[off:off + c] = False
    assert not got_v[pad].any() and not got_s[pad].any()


@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
def test_leaky_relu(capi, ob, vl, n):
    """vl_nnrelu with a leak (matlab/vl_nnrelu.m:49-55): y = x .* (leak + (1 - leak)*(x > 0)).  Pinned by what the
    definition fixes: leak 0 is the plain ReLU bit for bit (the oracle's), leak 1 the identity, positive inputs pass
    unchanged, negative ones come out as single(leak)*x exactly, and the derivative multiplies by the same factor."""
    import torch
    r = np.random.default_rng(n)
    x = r.standard_normal(n).astype(np.float32)
    x[::5] = 0.0
    dy = r.standard_normal(n).astype(np.float32)
    xd, dyd = capi.to_device(x), capi.to_device(dy)
    assert bits_equal(capi.to_host(capi.relu_forward(xd, leak=0.0)), ob.relu_forward(x))
    assert bits_equal(capi.to_host(capi.relu_backward(xd, dyd, leak=0.0)), ob.relu_backward(x, dy))
    assert bits_equal(capi.to_host(capi.relu_forward(xd, leak=1.0)), x * np.float32(1))
    for leak in (0.1, 0.01, 0.3):
        y = capi.to_host(capi.relu_forward(xd, leak=leak))
        dx = capi.to_host(capi.relu_backward(xd, dyd, leak=leak))
        pos = x > 0
        one = np.float32(leak + (1.0 - leak))
        assert bits_equal(y[pos], x[pos] * one) and bits_equal(y[~pos], x[~pos] * np.float32(leak))
        assert bits_equal(dx[pos], dy[pos] * one) and bits_equal(dx[~pos], dy[~pos] * np.float32(leak))
        # through the front-end, options by name
        yt = vl.vl_nnrelu(xd.reshape(1, 1, 1, n), "Leak", leak)
        assert bits_equal(yt.cpu().numpy().ravel(), y)
        dt = vl.vl_nnrelu(xd.reshape(1, 1, 1, n), dyd.reshape(1, 1, 1, n), "leak", leak)
        assert bits_equal(dt.cpu().numpy().ravel(), dx)
    assert bits_equal(vl.vl_nnrelu(xd.reshape(1, 1, 1, n)).cpu().numpy().ravel(), ob.relu_forward(x))
    with pytest.raises(vl.VlError) as e:
        vl.vl_nnrelu(xd, "leek", 0.1)
    assert e.value.message == "Unknown option 'leek'."


def test_yardsticks_run_and_report_their_work(capi):
    """The measurement helpers of the bench line: the streaming copy moves what it says (the copy is checked), the
    matrix-pipe stream reports its floating-point operations and rejects a senseless iteration count."""
    import ctypes as C
    import torch
    L = capi.lib()
    src = torch.arange(1 << 16, device="cuda", dtype=torch.float32)
    dst = torch.zeros_like(src)
    capi.check(L.mcn_hbm_yardstick(capi.stream(), capi.ptr(dst), capi.ptr(src), src.numel() * 4, 2, 16, 2, 0, 0))
    torch.cuda.synchronize()
    assert torch.equal(dst, src)
    sink = torch.zeros(4, device="cuda")
    flop = C.c_double(0.0)
    cus = int(L.mcn_device_compute_units())
    for is_double, per_wave in ((0, 8 * 4096.0), (1, 16 * 2048.0)):
        capi.check(L.mcn_mfma_yardstick(capi.stream(), capi.ptr(sink), 3, is_double, C.byref(flop)))
        torch.cuda.synchronize()
        assert flop.value == cus * 16 * 3 * per_wave
    assert float(sink.abs().sum()) == 0.0   # (the sink is never written)
    assert L.mcn_mfma_yardstick(capi.stream(), capi.ptr(sink), 0, 0, C.byref(flop)) != 0
