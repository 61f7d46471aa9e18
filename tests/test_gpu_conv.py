"""GPU parity, convolution (forward, backward-data, backward-filter, backward-bias) through the C ABI.
Gate from the task: max|diff|/max|ref| <= 2e-4 in fp32 against the CPU restatement of the reference
(im2row + sgemm per image) on the same seeded inputs."""
import numpy as np
import pytest

from matconvnet_amd import workloads
from util import F, rel_max

pytestmark = pytest.mark.gpu

TOL = 2e-4

# H, W, C, N, FH, FW, FC, K, stride, pad, dilate
CASES = [
    (8, 9, 3, 2, 3, 3, 3, 4, 1, 1, 1),
    (9, 8, 4, 3, 3, 2, 4, 6, (2, 1), (1, 0, 2, 1), 1),
    (12, 11, 2, 2, 3, 3, 2, 3, (2, 3), (2, 2, 1, 1), (2, 1)),
    (7, 7, 6, 2, 1, 1, 6, 5, 1, 0, 1),
    (10, 10, 6, 2, 3, 3, 2, 9, 1, 1, 1),                    # 3 filter groups
    (10, 9, 4, 2, 5, 3, 2, 4, (1, 2), (2, 1, 1, 3), 1),     # 2 groups, rectangular, asymmetric pad
    (16, 16, 8, 3, 3, 3, 8, 8, 1, (0, 2, 1, 0), 1),         # asymmetric pad, stride 1
    (14, 14, 16, 2, 3, 3, 16, 32, 1, 1, (2, 2)),            # dilation
    (64, 64, 8, 2, 11, 11, 8, 10, (3, 2), (5, 5, 8, 8), 1), # nnconv.m:163-202 geometry (reduced N)
    (28, 28, 32, 4, 3, 3, 32, 48, 1, 1, 1),
    (28, 28, 48, 3, 1, 1, 48, 24, 1, 0, 1),
    (17, 13, 5, 3, 5, 5, 5, 7, 1, 2, 1),                    # odd everything
    (6, 6, 3, 2, 6, 6, 3, 4, 1, 0, 1),                      # 1x1 output (the reference's FC special case)
    (20, 18, 32, 2, 3, 3, 32, 40, (2, 1), (1, 0, 2, 1), (1, 2)),  # 32 channels: tap-major kernels with stride + dilation
    (13, 11, 64, 3, 2, 3, 64, 130, 1, (0, 1, 1, 1), 1),      # even-sized filter, 130 filters (partial channel tile)
    (9, 9, 16, 2, 3, 3, 16, 16, (3, 3), 1, 1),               # 16 channels: tap-major forward only
    (14, 14, 64, 2, 3, 3, 32, 64, 1, 1, 1),                  # 2 groups of 32 channels: tap-major kernels per group
    (15, 14, 64, 2, 3, 3, 16, 96, (2, 2), 1, 1),             # 4 groups, strided: stride classes inside every group
    (12, 12, 96, 2, 1, 1, 32, 48, 2, 0, 1),                  # 3 groups, 1x1 stride 2
    (6, 6, 32, 8, 6, 6, 32, 200, 1, 0, 1),                   # fully connected, 1152 rows: forward splits the reduction
    (4, 4, 16, 4, 4, 4, 16, 640, 1, 0, 1),                   # fully connected, 640 filters: backward-data splits it
    (13, 13, 2, 3, 13, 13, 2, 5, 1, 0, 1),                   # fully connected with 169 taps: only the 1x1 view fits the MFMA kernels
    (20, 22, 64, 3, 3, 3, 64, 64, 1, 1, 1),                  # 576-row filter volume, 64 filters: 192-row filter-gradient tiles
    (12, 12, 64, 2, 3, 3, 64, 40, (2, 1), (1, 0, 1, 1), 1),  # the same volume with a partial filter tile, strided
]


# first layers: few input channels, 32 or 64 filters (the filter gradient takes a kernel of its own, which also gives
# the bias gradient): H, W, C, N, FH, FW, FC, K, stride, pad, dilate
FIRST_LAYERS = [
    (32, 32, 3, 5, 5, 5, 3, 32, 1, 2, 1),                     # BASELINE configs[0] at a smaller batch
    (64, 64, 3, 3, 7, 7, 3, 64, 2, 3, 1),                     # the ResNet stem's geometry on a smaller image
    (30, 31, 1, 3, 3, 3, 1, 32, (1, 2), (1, 0, 2, 1), 1),     # one channel, rectangular stride, asymmetric padding
    (17, 16, 4, 2, 5, 3, 4, 64, 1, (0, 1, 1, 0), 1),          # four channels, odd output height
    (150, 20, 2, 2, 3, 3, 2, 32, (3, 1), 1, 1),               # tall planes: more than one tile per column
    (9, 40, 3, 2, 2, 2, 3, 64, 1, 0, 1),                      # short planes, even filter
    (21, 19, 1, 3, 3, 3, 1, 32, 1, 1, 1),                     # stride 1, one channel, odd height: the input gradient's own kernel
    (40, 12, 3, 2, 7, 7, 3, 64, 1, (3, 3, 2, 4), 1),          # stride 1, 7x7, asymmetric padding
    (150, 9, 2, 2, 5, 5, 2, 32, 1, (2, 2, 0, 1), 1),          # stride 1, tall planes: more than one tile per column
    (6, 70, 4, 2, 3, 3, 4, 12, 1, 1, 1),                      # stride 1, 12 filters (no filter-gradient kernel of its own), short and wide
]


@pytest.mark.parametrize("case", FIRST_LAYERS)
def test_first_layer_filter_and_bias_gradients(capi, ob, case):
    """Filter gradient of first layers against the oracle, alone and together with the bias gradient
    (mcn_conv_backward_filter_bias: one pass gives both), and the same call on a layer that is no first layer."""
    x, f, b = _tensors(case)
    og = ob.conv_geom(x.shape, f.shape, *case[8:])
    dy = F(np.random.default_rng(6).standard_normal(ob.conv_out_shape(og)))
    _check(capi, ob, x, f, b, dy, *case[8:])
    g = capi.conv_geom(x.shape, f.shape, *case[8:])
    _, wdf, wdb = ob.conv_backward(x, f, dy, og)
    df, db = capi.conv_backward_filter_bias(capi.to_device(x), capi.to_device(dy), g)
    assert rel_max(capi.to_host(df), wdf) <= TOL and rel_max(capi.to_host(db), wdb) <= TOL
    # three workgroups walk all the tiles, each staging its next tile during the product
    capi.set_tunable("conv_first_max_wg", 3)
    try:
        df, db = capi.conv_backward_filter_bias(capi.to_device(x), capi.to_device(dy), g)
    finally:
        capi.set_tunable("conv_first_max_wg", 0)
    assert rel_max(capi.to_host(df), wdf) <= TOL and rel_max(capi.to_host(db), wdb) <= TOL


def test_filter_and_bias_gradients_by_one_call_on_any_layer(capi, ob):
    case = CASES[9]
    x, f, b = _tensors(case)
    og = ob.conv_geom(x.shape, f.shape, *case[8:])
    dy = F(np.random.default_rng(6).standard_normal(ob.conv_out_shape(og)))
    g = capi.conv_geom(x.shape, f.shape, *case[8:])
    _, wdf, wdb = ob.conv_backward(x, f, dy, og)
    df, db = capi.conv_backward_filter_bias(capi.to_device(x), capi.to_device(dy), g)
    assert rel_max(capi.to_host(df), wdf) <= TOL and rel_max(capi.to_host(db), wdb) <= TOL


def _tensors(case, seed=5):
    H, W, C, N, FH, FW, FC, K, stride, pad, dilate = case
    r = np.random.default_rng(seed)
    x = F(r.standard_normal((H, W, C, N)))
    f = F(r.standard_normal((FH, FW, FC, K)) / np.sqrt(FH * FW * FC))
    b = r.standard_normal(K).astype(np.float32)
    return x, f, b


def _check(capi, ob, x, f, b, dy, stride, pad, dilate, tol=TOL):
    g = capi.conv_geom(x.shape, f.shape, stride, pad, dilate)
    og = ob.conv_geom(x.shape, f.shape, stride, pad, dilate)
    xd, fd, dyd = capi.to_device(x), capi.to_device(f), capi.to_device(dy)
    dx, df, db = [capi.to_host(t) for t in capi.conv_backward(xd, fd, dyd, g)]
    wdx, wdf, wdb = ob.conv_backward(x, f, dy, og)
    errs = dict(dzdx=rel_max(dx, wdx), dzdf=rel_max(df, wdf), dzdb=rel_max(db, wdb))
    assert max(errs.values()) <= tol, errs
    return errs


@pytest.mark.parametrize("case", CASES)
def test_backward_vs_oracle(capi, ob, case):
    x, f, b = _tensors(case)
    og = ob.conv_geom(x.shape, f.shape, *case[8:])
    dy = F(np.random.default_rng(6).standard_normal(ob.conv_out_shape(og)))
    _check(capi, ob, x, f, b, dy, *case[8:])


@pytest.mark.parametrize("case", CASES)
def test_forward_vs_oracle(capi, ob, case):
    x, f, b = _tensors(case)
    g = capi.conv_geom(x.shape, f.shape, *case[8:])
    og = ob.conv_geom(x.shape, f.shape, *case[8:])
    y = capi.to_host(capi.conv_forward(capi.to_device(x), capi.to_device(f), capi.to_device(b), g))
    assert rel_max(y, ob.conv_forward(x, f, b, og)) <= TOL
    # no bias, and y = outMult*y + inMult*conv
    base = F(np.random.default_rng(7).standard_normal(y.shape))
    y2 = capi.to_host(capi.conv_forward(capi.to_device(x), capi.to_device(f), None, g, y=capi.to_device(base), out_mult=0.5, in_mult=2.0))
    assert rel_max(y2, ob.conv_forward(x, f, None, og, y=base.copy(order="F"), out_mult=0.5, in_mult=2.0)) <= TOL


def test_out_mult_zero_ignores_previous_output(capi, ob):
    case = CASES[0]
    x, f, b = _tensors(case)
    g = capi.conv_geom(x.shape, f.shape, *case[8:])
    y = capi.empty(capi.conv_out_shape(g), fill=float("nan"))
    capi.conv_forward(capi.to_device(x), capi.to_device(f), capi.to_device(b), g, y=y, out_mult=0.0)
    assert np.isfinite(capi.to_host(y)).all()


def test_direct_and_mfma_paths_agree(capi, ob):
    """The general direct kernels and the MFMA implicit-GEMM kernels compute the same thing."""
    case = (28, 28, 32, 4, 3, 3, 32, 48, 1, 1, 1)
    x, f, b = _tensors(case)
    g = capi.conv_geom(x.shape, f.shape, *case[8:])
    dy = F(np.random.default_rng(6).standard_normal(capi.conv_out_shape(g)))
    xd, fd, dyd = capi.to_device(x), capi.to_device(f), capi.to_device(dy)
    fast = [capi.to_host(t) for t in capi.conv_backward(xd, fd, dyd, g)]
    try:
        capi.set_tunable("conv_force_direct", 1)
        slow = [capi.to_host(t) for t in capi.conv_backward(xd, fd, dyd, g)]
    finally:
        capi.set_tunable("conv_force_direct", 0)
    for a, w in zip(fast, slow):
        assert rel_max(a, w) <= TOL


@pytest.mark.parametrize("case", [(28, 28, 32, 4, 3, 3, 32, 48, 1, 1, 1), (20, 18, 32, 2, 3, 3, 32, 40, (2, 1), (1, 0, 2, 1), (1, 2)),
                                  (14, 14, 64, 2, 1, 1, 64, 256, 1, 0, 1)])
def test_tap_major_and_channel_major_kernels_agree(capi, ob, case):
    """The uniform-tap (tap-major) MFMA kernels and the general channel-major ones are two orderings of the same
    sums: both within the gate of the oracle and of each other."""
    x, f, b = _tensors(case)
    g = capi.conv_geom(x.shape, f.shape, *case[8:])
    dy = F(np.random.default_rng(6).standard_normal(capi.conv_out_shape(g)))
    xd, fd, dyd, bd = capi.to_device(x), capi.to_device(f), capi.to_device(dy), capi.to_device(b)
    fast = [capi.to_host(t) for t in capi.conv_backward(xd, fd, dyd, g)] + [capi.to_host(capi.conv_forward(xd, fd, bd, g))]
    try:
        capi.set_tunable("conv_no_uniform_tap", 1)
        slow = [capi.to_host(t) for t in capi.conv_backward(xd, fd, dyd, g)] + [capi.to_host(capi.conv_forward(xd, fd, bd, g))]
    finally:
        capi.set_tunable("conv_no_uniform_tap", 0)
    for a, w in zip(fast, slow):
        assert rel_max(a, w) <= TOL
    og = ob.conv_geom(x.shape, f.shape, *case[8:])
    for a, w in zip(slow[:3], ob.conv_backward(x, f, dy, og)):
        assert rel_max(a, w) <= TOL


def test_baseline_config1_full(capi, ob):
    """benchmark configuration 1: x 32x32x3x100, f 5x5x3x32, stride 1, pad 2 (the reference's CPU-runnable case)."""
    w = workloads.conv_single()
    errs = _check(capi, ob, w["x"], w["f"], w["b"], w["dy"], w["stride"], w["pad"], w["dilate"])
    print("conv cfg1:", errs)
    g = capi.conv_geom(w["x"].shape, w["f"].shape, w["stride"], w["pad"], w["dilate"])
    y = capi.to_host(capi.conv_forward(capi.to_device(w["x"]), capi.to_device(w["f"]), capi.to_device(w["b"]), g))
    assert rel_max(y, ob.conv_forward(w["x"], w["f"], w["b"], ob.conv_geom(w["x"].shape, w["f"].shape, 1, 2, 1))) <= TOL


@pytest.mark.parametrize("which", ["1x1_256_64", "3x3_64_64", "1x1_64_256"])
def test_baseline_config4_conv_shapes_full(capi, ob, which):
    """The three convolutions of the ResNet-50 bottleneck at N = 32, 56x56 (benchmark configuration 4)."""
    r = np.random.default_rng(40)
    C, K, fs, pad = {"1x1_256_64": (256, 64, 1, 0), "3x3_64_64": (64, 64, 3, 1), "1x1_64_256": (64, 256, 1, 0)}[which]
    x = F(r.standard_normal((56, 56, C, 32), dtype=np.float32))
    f = workloads.he_normal(r, (fs, fs, C, K))
    dy = F(r.standard_normal((56, 56, K, 32), dtype=np.float32))
    print(which, _check(capi, ob, x, f, None, dy, 1, pad, 1))


def test_baseline_config5_reduced_batch(capi, ob):
    """benchmark configuration 5 geometry (56x56x256, 3x3x256x256, pad 1) at N = 2 against the oracle."""
    w = workloads.conv_vgg(N=2)
    print("conv cfg5 (N=2):", _check(capi, ob, w["x"], w["f"], None, w["dy"], 1, 1, 1))


def test_baseline_config5_full_size_properties(capi, ob):
    """benchmark configuration 5 at full size (N = 64): too big for the CPU oracle in a test, so
    (1) dzdx of single images is compared with the oracle run on those images alone (images are
        independent in backward-data),
    (2) dzdf / dzdb are linear in the batch: the full-batch result must equal the sum of the results on the
        two half batches, and the first half's dzdf is checked against the oracle on a 2-image slice via
        the same linearity (full = slice + rest)."""
    w = workloads.conv_vgg()
    x, f, dy = w["x"], w["f"], w["dy"]
    N = x.shape[3]
    g = capi.conv_geom(x.shape, f.shape, 1, 1, 1)
    xd, fd, dyd = capi.to_device(x), capi.to_device(f), capi.to_device(dy)
    dx, df, db = capi.conv_backward(xd, fd, dyd, g)
    dxh = capi.to_host(dx)
    for n in (0, N - 1):
        og = ob.conv_geom((56, 56, 256, 1), f.shape, 1, 1, 1)
        wdx, _, _ = ob.conv_backward(None, f, F(dy[:, :, :, n:n + 1]), og, want=(True, False, False))
        assert rel_max(dxh[:, :, :, n:n + 1], wdx) <= TOL
    # linearity over the batch, and an oracle anchor on a 2-image slice
    def part(lo, hi):
        gp = capi.conv_geom((56, 56, 256, hi - lo), f.shape, 1, 1, 1)
        _, dfp, dbp = capi.conv_backward(capi.to_device(x[:, :, :, lo:hi]), fd, capi.to_device(dy[:, :, :, lo:hi]), gp, want=(False, True, True))
        return capi.to_host(dfp).astype(np.float64), capi.to_host(dbp).astype(np.float64)
    dfa, dba = part(0, 2)
    dfb, dbb = part(2, N)
    assert rel_max(capi.to_host(df), dfa + dfb) <= TOL and rel_max(capi.to_host(db), dba + dbb) <= TOL
    og2 = ob.conv_geom((56, 56, 256, 2), f.shape, 1, 1, 1)
    _, wdf, wdb = ob.conv_backward(F(x[:, :, :, 0:2]), f, F(dy[:, :, :, 0:2]), og2, want=(False, True, True))
    assert rel_max(dfa, wdf) <= TOL and rel_max(dba, wdb) <= TOL


def test_errors(capi):
    with pytest.raises(capi.McnError) as e:
        capi.conv_out_shape(capi.conv_geom((8, 8, 3, 1), (3, 3, 2, 4)))
    assert e.value.code == capi.ILLEGAL_ARGUMENT
    with pytest.raises(capi.McnError):
        capi.conv_out_shape(capi.conv_geom((2, 2, 3, 1), (3, 3, 3, 4)))
    with pytest.raises(capi.McnError):
        capi.conv_out_shape(capi.conv_geom((8, 8, 4, 1), (3, 3, 2, 3)))  # 2 groups do not divide 3 filters


WS_CASES = [  # (xshape, fshape, stride, pad, dilate): reduction rows a multiple of 64, bank small enough for LDS
    ((20, 18, 64, 3), (1, 1, 64, 64), 1, 0, 1),
    ((20, 18, 64, 2), (1, 1, 64, 40), 1, 0, 1),          # output channels not a multiple of 32
    ((13, 11, 64, 5), (3, 3, 64, 32), 1, 1, 1),          # pixels not a multiple of 32
    ((17, 15, 64, 2), (3, 3, 64, 64), 1, (2, 0, 1, 3), 1),
    ((19, 19, 64, 2), (3, 2, 64, 96), (2, 3), 1, 1),     # strided: backward-data runs once per stride class
    ((22, 21, 64, 2), (1, 1, 64, 64), 2, 0, 1),          # 1x1, stride 2: three of four classes are zeros
    ((23, 20, 64, 2), (5, 3, 64, 64), (2, 2), (2, 1, 1, 0), (2, 1)),  # stride and dilation together
    ((21, 20, 64, 2), (3, 3, 64, 64), 1, 2, 2),          # dilated
    ((12, 12, 64, 4), (2, 2, 64, 16), 1, (1, 0, 0, 1), 1),
    ((10, 9, 64, 3), (1, 1, 64, 128), 1, 0, 1),          # wide enough for the 128-channel units
    ((56, 56, 64, 3), (1, 1, 64, 64), 1, 0, 1),          # several units per wavefront: the load stream crosses units
    # banks larger than LDS, cut into slices of output channels (one slice per workgroup)
    ((28, 28, 128, 2), (1, 1, 128, 512), 1, 0, 1),       # 2 slices forward; backward-data (512 -> 128) 2 slices too
    ((14, 14, 256, 3), (1, 1, 256, 1000), 1, 0, 1),      # 8 slices, output channels not a multiple of the slice
    ((14, 13, 128, 3), (3, 3, 128, 128), 1, 1, 1),       # 3x3: 4 slices of 32 channels
    ((15, 14, 64, 2), (3, 3, 64, 192), 2, 1, 1),         # strided, sliced
]


@pytest.mark.parametrize("wa", [0, 1, 2, 4])
@pytest.mark.parametrize("xs,fs,stride,pad,dilate", WS_CASES)
def test_weights_stationary_kernel(capi, ob, xs, fs, stride, pad, dilate, wa):
    """Forward and backward-data through the weights-stationary MFMA kernel (forced onto small problems),
    every width of its units, against the oracle."""
    r = np.random.default_rng(sum(xs) + sum(fs) + wa)
    x = F(r.standard_normal(xs))
    f = F(r.standard_normal(fs) * 0.2)
    b = r.standard_normal(fs[3]).astype(np.float32)
    g = ob.conv_geom(xs, fs, stride, pad, dilate)
    cg = capi.conv_geom(xs, fs, stride, pad, dilate)
    capi.set_tunable("conv_ws_min_units", 1)
    capi.set_tunable("conv_ws_wa", wa)
    capi.set_tunable("conv_ws_sliced_strided", 1)   # (by default a sliced bank is not used for a strided gather)
    try:
        capi.profile_begin("conv_ws_mfma")
        y = capi.conv_forward(capi.to_device(x), capi.to_device(f), capi.to_device(b), cg)
        want = ob.conv_forward(x, f, b, g)
        dy = F(r.standard_normal(want.shape))
        dx, _, _ = capi.conv_backward(capi.to_device(x), capi.to_device(f), capi.to_device(dy), cg, want=(True, False, False))
        launches, _ = capi.profile_end()
    finally:
        capi.set_tunable("conv_ws_min_units", 0)
        capi.set_tunable("conv_ws_wa", 0)
        capi.set_tunable("conv_ws_sliced_strided", 0)
    strided = np.any(np.atleast_1d(stride) != 1)

    def eligible(cin, cout):
        """The kernel's own admission rule: reduction channels a multiple of 16 and rows a multiple of 64, the
        packed bank (padded to the channel tile) -- or one of 2, 4 or 8 equal slices of its output channels, each a
        multiple of 32 -- within 150 KB of LDS, a slice a whole number of units."""
        taps = fs[0] * fs[1]
        tile = 128 if cout > 64 else (64 if cout > 32 else 32)
        padded = -(-cout // tile) * tile
        if cin % 16 != 0 or (taps * cin) % 64 != 0:
            return False
        for slices in (1, 2, 4, 8):
            if padded % (32 * slices) != 0:
                return False
            if taps * cin * (padded // slices) * 4 <= 150 * 1024:
                return wa == 0 or (padded // slices) % (32 * wa) == 0
        return False

    # the kernel under test really ran (a strided layer's backward-data product is one launch per stride class
    # whose tap subset is eligible, so only a lower bound is fixed there)
    if strided:
        assert launches >= int(eligible(xs[2], fs[3]))
    else:
        assert launches == int(eligible(xs[2], fs[3])) + int(eligible(fs[3], xs[2]))
    assert rel_max(capi.to_host(y), want) < 2e-4
    assert rel_max(capi.to_host(dx), ob.conv_backward(x, f, dy, g, want=(True, False, False))[0]) < 2e-4


def test_sliced_bank_not_used_for_strided_gather(capi, ob):
    """A bank cut into slices makes every slice gather the pixels again; for a strided forward gather the tiled
    kernel is chosen instead (same result either way)."""
    xs, fs = (15, 14, 64, 2), (3, 3, 64, 192)
    r = np.random.default_rng(5)
    x, f = F(r.standard_normal(xs)), F(r.standard_normal(fs) * 0.2)
    cg = capi.conv_geom(xs, fs, 2, 1, 1)
    capi.set_tunable("conv_ws_min_units", 1)
    try:
        capi.profile_begin("conv_ws_mfma")
        y = capi.conv_forward(capi.to_device(x), capi.to_device(f), None, cg)
        launches, _ = capi.profile_end()
    finally:
        capi.set_tunable("conv_ws_min_units", 0)
    assert launches == 0
    assert rel_max(capi.to_host(y), ob.conv_forward(x, f, None, ob.conv_geom(xs, fs, 2, 1, 1))) < 2e-4


@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("tiled", [False, True])
def test_fast_epilogue_out_mult(capi, ob, with_bias, tiled):
    """y = outMult*y + inMult*conv (+ bias) through the straight-line store path of both MFMA kernels."""
    r = np.random.default_rng(11 + with_bias)
    xs, fs = (20, 18, 64, 3), (3, 3, 64, 64)
    x = F(r.standard_normal(xs))
    f = F(r.standard_normal(fs) * 0.2)
    b = r.standard_normal(fs[3]).astype(np.float32) if with_bias else None
    g = ob.conv_geom(xs, fs, 1, 1, 1)
    cg = capi.conv_geom(xs, fs, 1, 1, 1)
    base = F(r.standard_normal(capi.conv_out_shape(cg)))
    capi.set_tunable("conv_ws_min_units", 1)
    capi.set_tunable("conv_no_ws", int(tiled))
    try:
        capi.profile_begin("conv_ws_mfma")
        y = capi.conv_forward(capi.to_device(x), capi.to_device(f), None if b is None else capi.to_device(b), cg,
                              y=capi.to_device(base), out_mult=0.5, in_mult=2.0)
        launches, _ = capi.profile_end()
    finally:
        capi.set_tunable("conv_ws_min_units", 0)
        capi.set_tunable("conv_no_ws", 0)
    assert launches == (0 if tiled else 1)
    want = ob.conv_forward(x, f, b, g, y=base.copy(order="F"), out_mult=0.5, in_mult=2.0)
    assert rel_max(capi.to_host(y), want) < 2e-4


@pytest.mark.parametrize("path", ["ws", "tiled", "direct"])
def test_backward_data_accumulate(capi, ob, path):
    """derInput = mult*derInput + dzdx through each kernel family (and mult = 0 ignores what was there)."""
    r = np.random.default_rng(23)
    xs, fs = (20, 18, 64, 3), (3, 3, 64, 64)
    x = F(r.standard_normal(xs))
    f = F(r.standard_normal(fs) * 0.2)
    g = ob.conv_geom(xs, fs, 1, 1, 1)
    cg = capi.conv_geom(xs, fs, 1, 1, 1)
    dy = F(r.standard_normal(capi.conv_out_shape(cg)))
    base = F(r.standard_normal(xs))
    want = ob.conv_backward(x, f, dy, g, want=(True, False, False))[0]
    capi.set_tunable("conv_ws_min_units", 1)
    capi.set_tunable("conv_no_ws", int(path != "ws"))
    capi.set_tunable("conv_force_direct", int(path == "direct"))
    try:
        got = capi.to_host(capi.conv_backward_data_acc(capi.to_device(base), 0.75, capi.to_device(f), capi.to_device(dy), cg))
        poisoned = capi.empty(xs, fill=float("nan"))
        plain = capi.to_host(capi.conv_backward_data_acc(poisoned, 0.0, capi.to_device(f), capi.to_device(dy), cg))
    finally:
        for k in ("conv_ws_min_units", "conv_no_ws", "conv_force_direct"):
            capi.set_tunable(k, 0)
    assert rel_max(got, 0.75 * base + want) < 2e-4
    assert rel_max(plain, want) < 2e-4


def test_groups_and_strides_run_on_the_mfma_kernels(capi, ob):
    """Filter groups and strided backward-data are served by the MFMA kernels (one launch per group and stride
    class), not by the one-thread-per-output fallback."""
    case = (15, 14, 64, 2, 3, 3, 16, 96, (2, 2), 1, 1)
    x, f, b = _tensors(case)
    cg = capi.conv_geom(x.shape, f.shape, *case[8:])
    dy = F(np.random.default_rng(3).standard_normal(capi.conv_out_shape(cg)))
    capi.profile_begin("_mfma")
    capi.conv_forward(capi.to_device(x), capi.to_device(f), capi.to_device(b), cg)
    capi.conv_backward(capi.to_device(x), capi.to_device(f), capi.to_device(dy), cg)
    launches, _ = capi.profile_end()
    # 4 groups: forward 4, backward-filter 4, backward-data 4 groups x 4 stride classes
    assert launches == 4 + 4 + 16


def test_fully_connected_split_reduction(capi, ob):
    """A filter bank that covers the whole input runs as a 1x1 layer over H*W*C channels with the reduction split
    over workgroups; y = outMult*y + inMult*conv + bias through the pass that adds the partial results."""
    r = np.random.default_rng(31)
    xs, fs = (6, 6, 32, 8), (6, 6, 32, 200)
    x = F(r.standard_normal(xs))
    f = F(r.standard_normal(fs) * 0.05)
    b = r.standard_normal(fs[3]).astype(np.float32)
    g = ob.conv_geom(xs, fs, 1, 0, 1)
    cg = capi.conv_geom(xs, fs, 1, 0, 1)
    base = F(r.standard_normal(capi.conv_out_shape(cg)))
    capi.profile_begin("conv_pix_reduce")
    y = capi.conv_forward(capi.to_device(x), capi.to_device(f), capi.to_device(b), cg, y=capi.to_device(base), out_mult=0.5, in_mult=2.0)
    launches, _ = capi.profile_end()
    assert launches == 1
    assert rel_max(capi.to_host(y), ob.conv_forward(x, f, b, g, y=base.copy(order="F"), out_mult=0.5, in_mult=2.0)) < 2e-4
    capi.set_tunable("conv_no_split", 1)
    try:
        y1 = capi.conv_forward(capi.to_device(x), capi.to_device(f), capi.to_device(b), cg)
    finally:
        capi.set_tunable("conv_no_split", 0)
    assert rel_max(capi.to_host(y1), ob.conv_forward(x, f, b, g)) < 2e-4


def _random_case(r):
    """A valid layer geometry: groups, strides, dilation, asymmetric padding, channel counts on both sides of the
    kernels' 16 / 32-channel thresholds, sometimes a filter that covers the whole input."""
    groups = int(r.choice([1, 1, 2, 4]))
    FC = int(r.choice([1, 3, 8, 16, 32]))
    Kg = int(r.choice([1, 5, 16, 32, 40]))
    FH, FW = int(r.integers(1, 6)), int(r.integers(1, 6))
    dil = (int(r.integers(1, 3)), int(r.integers(1, 3)))
    stride = (int(r.integers(1, 4)), int(r.integers(1, 4)))
    pad = tuple(int(v) for v in r.integers(0, 3, size=4))
    eh, ew = (FH - 1) * dil[0] + 1, (FW - 1) * dil[1] + 1
    H = max(1, eh - pad[0] - pad[1]) + int(r.integers(0, 12))
    W = max(1, ew - pad[2] - pad[3]) + int(r.integers(0, 12))
    if r.random() < 0.15:  # fully connected
        FH, FW, dil, pad = H, W, (1, 1), (0, 0, 0, 0)
    return (H, W, FC * groups, int(r.integers(1, 5)), FH, FW, FC, Kg * groups, stride, pad, dil)


@pytest.mark.parametrize("seed", range(48))
def test_random_geometries_vs_oracle(capi, ob, seed):
    """Forward and all three derivatives on seeded random geometries (whatever kernel the dispatch picks)."""
    r = np.random.default_rng(1000 + seed)
    case = _random_case(r)
    x, f, b = _tensors(case, seed=seed)
    og = ob.conv_geom(x.shape, f.shape, *case[8:])
    cg = capi.conv_geom(x.shape, f.shape, *case[8:])
    y = capi.to_host(capi.conv_forward(capi.to_device(x), capi.to_device(f), capi.to_device(b), cg))
    assert rel_max(y, ob.conv_forward(x, f, b, og)) <= TOL, case
    dy = F(r.standard_normal(ob.conv_out_shape(og)))
    _check(capi, ob, x, f, b, dy, *case[8:])


def test_tensors_over_2_gib_match_small_batches(capi):
    """Tensors beyond 2^31 bytes leave the 32-bit-offset fast paths (buffer descriptors, uniform-tap offsets): the
    same layer on the whole batch and on its first / last images must agree (images are independent)."""
    import torch
    H, W, Cc, N = 64, 64, 64, 2100            # 2.2 GB per tensor
    fs = (3, 3, Cc, Cc)
    torch.manual_seed(5)
    x = torch.randn((N, Cc, W, H), device="cuda")
    f = torch.randn(tuple(reversed(fs)), device="cuda") * 0.05
    g = capi.conv_geom((H, W, Cc, N), fs, 1, 1, 1)
    y = capi.conv_forward(x, f, None, g)
    dx, _, _ = capi.conv_backward(x, f, y, g, want=(True, False, False))
    for sl in (slice(0, 3), slice(N - 3, N)):
        gs = capi.conv_geom((H, W, Cc, 3), fs, 1, 1, 1)
        ys = capi.conv_forward(x[sl].contiguous(), f, None, gs)
        assert float((ys - y[sl]).abs().max()) <= 2e-4 * float(ys.abs().max())
        dxs, _, _ = capi.conv_backward(x[sl].contiguous(), f, ys, gs, want=(True, False, False))
        assert float((dxs - dx[sl]).abs().max()) <= 2e-4 * float(dxs.abs().max())


PACKED_CASES = [  # (H, W, C, N, FH, FW, K, stride, pad, dilate, groups)
    (14, 14, 64, 3, 1, 1, 128, 1, 0, 1, 1),     # 1x1: backward-data reads the bank as stored
    (14, 14, 48, 3, 1, 1, 72, 1, 0, 1, 1),      # 1x1 whose extents need padding
    (12, 10, 32, 2, 3, 3, 64, 1, 1, 1, 1),      # 3x3
    (13, 11, 32, 2, 3, 3, 64, 2, 1, 1, 1),      # stride 2: four stride classes, each its own bank
    (12, 12, 64, 2, 1, 1, 128, 2, 0, 1, 1),     # strided 1x1: one class
    (9, 9, 3, 2, 5, 5, 16, 1, 2, 1, 1),         # 3 channels: the general (not uniform-tap) order
    (10, 10, 32, 2, 3, 3, 32, 1, 1, 1, 2),      # two filter groups
    (6, 6, 16, 4, 6, 6, 40, 1, 0, 1, 1),        # fully connected
    (14, 14, 256, 4, 3, 3, 256, 1, 1, 1, 1),    # split reduction
    (13, 13, 48, 2, 3, 3, 100, 1, 1, 1, 1),     # bank tiles of the packing kernel ragged both ways (432 rows, 100 of 128 filters)
    (20, 20, 64, 2, 3, 3, 128, 2, 1, 1, 1),     # 3x3 /2: four stride classes in one launch, their banks side by side
]


@pytest.mark.parametrize("case", PACKED_CASES)
def test_filters_packed_ahead_give_the_same_bits(capi, case):
    """Forward and backward-data (overwriting and accumulating) with the banks packed ahead, one layer at a time and
    several layers in one batched launch, against the calls that pack on the fly."""
    import torch
    H, W, Cc, N, FH, FW, K, stride, pad, dilate, groups = case
    r = np.random.default_rng(5)
    xs, fs = (H, W, Cc, N), (FH, FW, Cc // groups, K)
    g = capi.conv_geom(xs, fs, stride, pad, dilate)
    x, f = capi.to_device(F(r.standard_normal(xs))), capi.to_device(F(r.standard_normal(fs)))
    b = capi.to_device(r.standard_normal(K).astype(np.float32))
    dy = capi.to_device(F(r.standard_normal(capi.conv_out_shape(g))))
    base = capi.to_device(F(r.standard_normal(xs)))
    want_y = capi.conv_forward(x, f, b, g)
    want_dx = capi.conv_backward_data_acc(capi.empty(xs), 0.0, f, dy, g)
    want_acc = capi.conv_backward_data_acc(base.clone(), 1.0, f, dy, g)
    # a second layer packed in the same batch
    g2 = capi.conv_geom((8, 8, 32, 2), (3, 3, 32, 32), 1, 1, 1)
    f2 = capi.to_device(F(r.standard_normal((3, 3, 32, 32))))
    for how in ("single", "batch"):
        if how == "single":
            pf, pb = capi.conv_pack_filters(f, g, capi.CONV_FORWARD), capi.conv_pack_filters(f, g, capi.CONV_BACKWARD_DATA)
        else:
            _, pf, pb, _ = capi.conv_pack_many([(f2, g2, capi.CONV_FORWARD), (f, g, capi.CONV_FORWARD),
                                                (f, g, capi.CONV_BACKWARD_DATA), (f2, g2, capi.CONV_BACKWARD_DATA)])
        assert (pf is None) == (capi.conv_packed_bytes(g, capi.CONV_FORWARD) == 0)
        assert torch.equal(capi.conv_forward_packed(x, f, pf, b, g), want_y), how
        assert torch.equal(capi.conv_backward_data_packed(capi.empty(xs), 0.0, f, pb, dy, g), want_dx), how
        assert torch.equal(capi.conv_backward_data_packed(base.clone(), 1.0, f, pb, dy, g), want_acc), how
    # the first case reads the 1x1 bank as stored: nothing to pack for backward-data
    if case == PACKED_CASES[0]:
        assert capi.conv_packed_bytes(g, capi.CONV_BACKWARD_DATA) == 0 and capi.conv_packed_bytes(g, capi.CONV_FORWARD) > 0


def test_packed_buffer_too_small_is_refused(capi):
    import ctypes as C
    g = capi.conv_geom((8, 8, 32, 2), (3, 3, 32, 32), 1, 1, 1)
    f = capi.to_device(F(np.ones((3, 3, 32, 32))))
    n = capi.conv_packed_bytes(g, capi.CONV_FORWARD)
    small = capi.to_device(np.zeros(n // 8, np.float32))
    rc = capi.lib().mcn_conv_pack_filters(capi.stream(), C.byref(g), capi.CONV_FORWARD, capi.ptr(f), capi.ptr(small), n // 2)
    assert rc != 0 and b"too small" in capi.lib().mcn_last_error_message()


def test_filter_gradients_with_one_deferred_sum(capi):
    """The filter gradients of several layers (1x1, 3x3, strided, grouped, 3-channel, fully connected) from the matrix
    kernels alone plus ONE launch that sums all their reduction splits, against mcn_conv_backward_filter per layer."""
    import torch
    r = np.random.default_rng(6)
    layers, want = [], []
    for H, W, Cc, N, FH, FW, K, stride, pad, dilate, groups in PACKED_CASES:
        xs, fs = (H, W, Cc, N), (FH, FW, Cc // groups, K)
        g = capi.conv_geom(xs, fs, stride, pad, dilate)
        x = capi.to_device(F(r.standard_normal(xs)))
        dy = capi.to_device(F(r.standard_normal(capi.conv_out_shape(g))))
        layers.append((x, dy, g))
        want.append(capi.conv_backward(x, None, dy, g, want=(False, True, False))[1])
    got = capi.conv_backward_filter_deferred(layers)
    assert sum(capi.lib().mcn_conv_backward_filter_partial_bytes(__import__("ctypes").byref(g)) > 0 for _, _, g in layers) >= 6
    for a, b_, case in zip(got, want, PACKED_CASES):
        assert torch.equal(a, b_), case


FEW_CASES = [
    # x, f, stride, pad, dilate        (backward-data has C output channels, forward K)
    ((32, 32, 3, 5), (5, 5, 3, 32), 1, 2, 1),                # benchmark configuration 1: dzdx has 3 channels, 32 filters reduce
    ((28, 28, 1, 4), (5, 5, 1, 20), 1, 0, 1),                # LeNet's first layer: one channel, 20 filters (not a multiple of 16)
    ((30, 29, 3, 3), (7, 7, 3, 64), 2, 3, 1),                # a ResNet stem in small: strided (four stride classes)
    ((17, 19, 4, 2), (3, 3, 4, 16), (1, 2), (1, 0, 2, 1), (2, 1)),   # four channels, dilation, one strided axis
    ((12, 13, 2, 3), (3, 2, 2, 7), 1, 1, 1),                 # two channels, seven filters
    ((14, 14, 16, 3), (3, 3, 16, 3), 1, 1, 1),               # forward with three filters (and backward-data with 16 channels)
    ((9, 9, 32, 2), (1, 1, 32, 1), 1, 0, 1),                 # forward 1x1 with one filter
    ((11, 12, 8, 2), (3, 3, 2, 8), 1, 1, 1),                 # four filter groups of two channels: dzdx per group has 2 channels
    ((64, 64, 3, 2), (11, 11, 3, 48), 4, 0, 1),              # AlexNet-like first layer: 121 taps, stride 4
]


@pytest.mark.parametrize("xs,fs,stride,pad,dilate", FEW_CASES)
def test_few_output_channels(capi, ob, xs, fs, stride, pad, dilate):
    """Products with one to four output channels run a kernel of their own (no padding to 32-channel tiles): forward,
    backward-data, accumulation into the output, bias; against the oracle, and against the tiled kernels."""
    r = np.random.default_rng(sum(xs) * 3 + sum(fs))
    x = F(r.standard_normal(xs))
    f = F(r.standard_normal(fs) * 0.2)
    b = r.standard_normal(fs[3]).astype(np.float32)
    g = ob.conv_geom(xs, fs, stride, pad, dilate)
    cg = capi.conv_geom(xs, fs, stride, pad, dilate)
    xd, fd, bd = capi.to_device(x), capi.to_device(f), capi.to_device(b)
    want = ob.conv_forward(x, f, b, g)
    dy = F(r.standard_normal(want.shape))
    base = F(r.standard_normal(want.shape))
    dbase = F(r.standard_normal(xs))
    wdx = ob.conv_backward(x, f, dy, g, want=(True, False, False))[0]
    got = {}
    for off in (0, 1):
        capi.set_tunable("conv_no_few", off)
        capi.set_tunable("conv_no_first", 1)   # (first layers at stride 1 have another kernel for the input gradient)
        try:
            capi.profile_begin("conv_few_mfma")
            y = capi.conv_forward(xd, fd, bd, cg)
            y2 = capi.conv_forward(xd, fd, bd, cg, y=capi.to_device(base), out_mult=0.5, in_mult=2.0)
            dx, _, _ = capi.conv_backward(xd, fd, capi.to_device(dy), cg, want=(True, False, False))
            dx2 = capi.conv_backward_data_acc(capi.to_device(dbase), 1.0, fd, capi.to_device(dy), cg)
            launches, _ = capi.profile_end()
        finally:
            capi.set_tunable("conv_no_few", 0)
            capi.set_tunable("conv_no_first", 0)
        got[off] = launches
        assert rel_max(capi.to_host(y), want) < 2e-4
        assert rel_max(capi.to_host(y2), 0.5 * base.astype(np.float64) + 2.0 * (want.astype(np.float64) - b.reshape(1, 1, -1, 1)) + b.reshape(1, 1, -1, 1)) < 2e-4
        assert rel_max(capi.to_host(dx), wdx) < 2e-4
        assert rel_max(capi.to_host(dx2), dbase.astype(np.float64) + wdx) < 2e-4
    assert got[0] >= 2 and got[1] == 0   # the kernel ran (at least the two products of the few-channel side)


@pytest.mark.parametrize("xs,fs,stride,pad", [((30, 29, 3, 3), (7, 7, 3, 64), 2, 3), ((14, 15, 32, 2), (1, 5, 32, 40), 1, (0, 0, 2, 2)),
                                               ((12, 12, 20, 2), (3, 3, 20, 64), 1, 1)])
def test_filter_gradient_wide_row_tile(capi, ob, xs, fs, stride, pad):
    """Filter volumes of 129...192 rows with up to 64 filters take one 192-row tile (a ResNet stem: 7x7x3 = 147 rows):
    against the oracle, with that tile and with the 128-row tiles."""
    r = np.random.default_rng(sum(xs) + sum(fs))
    x = F(r.standard_normal(xs))
    f = F(r.standard_normal(fs) * 0.1)
    g = ob.conv_geom(xs, fs, stride, pad, 1)
    cg = capi.conv_geom(xs, fs, stride, pad, 1)
    dy = F(r.standard_normal(capi.conv_out_shape(cg)))
    want = ob.conv_backward(x, f, dy, g, want=(False, True, False))[1]
    for off in (0, 1):
        capi.set_tunable("conv_wgrad_no_wide_rows", off)
        try:
            _, df, _ = capi.conv_backward(capi.to_device(x), capi.to_device(f), capi.to_device(dy), cg, want=(False, True, False))
        finally:
            capi.set_tunable("conv_wgrad_no_wide_rows", 0)
        assert rel_max(capi.to_host(df), want) < 2e-4


SUMMING = [  # x shape, filter shape, pad: the three convolutions of the bottleneck block, smaller batches
    ((56, 56, 256, 8), (1, 1, 256, 64), 0),
    ((56, 56, 64, 8), (3, 3, 64, 64), 1),
    ((56, 56, 64, 12), (1, 1, 64, 256), 0),
    ((28, 28, 256, 16), (1, 1, 256, 128), 0),     # four channel blocks side by side, one workgroup per compute unit
]


@pytest.mark.parametrize("xs,fs,pad", SUMMING)
def test_conv_forward_with_channel_sums(capi, ob, xs, fs, pad):
    """The convolution that also sums its output per channel (the first pass of a batch normalisation that
    follows): y has the bits of the plain convolution, the partial sums add up to the sums of that y taken in
    double, and batch normalisation from those sums is within 1e-5 of the reference's formula in double
    (bits/nnbnorm.cu:46-71) applied to the same y."""
    import torch
    r = np.random.default_rng(3)
    x = F(r.standard_normal(xs) + 0.3)
    f = F(r.standard_normal(fs) * np.sqrt(2.0 / (fs[0] * fs[1] * fs[2])))
    K = fs[3]
    g = capi.conv_geom(xs, fs, 1, pad, 1)
    groups = capi.conv_forward_sums_groups(g)
    assert groups > 0
    xd, fd = capi.to_device(x), capi.to_device(f)
    want = capi.conv_forward(xd, fd, None, g)
    for turn in range(2):  # (the second call finds the buffers of the first: nothing is carried over)
        y, sums = capi.conv_forward_sums(xd, fd, g)
        assert torch.equal(y, want)
        yd = y.double()
        s1, s2 = yd.sum(dim=(0, 2, 3)), (yd * yd).sum(dim=(0, 2, 3))
        tot = sums.sum(dim=1)
        assert float((tot[:, 0] - s1).abs().max() / s1.abs().max()) < 1e-6
        assert float((tot[:, 1] - s2).abs().max() / s2.abs().max()) < 1e-6
    gain = F(r.uniform(0.5, 1.5, K)).ravel()
    bias = F(r.standard_normal(K) * 0.1).ravel()
    res = F(r.standard_normal(capi.conv_out_shape(g)))
    gd, bd, rd = capi.to_device(gain), capi.to_device(bias), capi.to_device(res)
    y64 = F(capi.to_host(y), np.float64)
    ref, mom = ob.bnorm_forward(y64, gain.astype(np.float64), bias.astype(np.float64), 1e-5)
    for residual, relu in ((None, True), (rd, True), (rd, False), (None, False)):
        out, m = capi.bnorm_forward_sums(y, gd, bd, sums, residual=residual, relu=relu, eps=1e-5)
        w = ref + (res.astype(np.float64) if residual is not None else 0.0)
        if relu:
            w = np.maximum(w, 0.0)
        assert rel_max(capi.to_host(out), w) <= 1e-5
        assert rel_max(capi.to_host(m), mom) <= 1e-5
    # against the two-launch form on the same tensor: same result to rounding
    out2, m2 = capi.bnorm_forward_fused(y, gd, bd, residual=rd, relu=True, eps=1e-5)
    out1, m1 = capi.bnorm_forward_sums(y, gd, bd, sums, residual=rd, relu=True, eps=1e-5)
    assert rel_max(capi.to_host(out1), capi.to_host(out2)) <= 2e-6 and rel_max(capi.to_host(m1), capi.to_host(m2)) <= 1e-6


def test_conv_forward_with_channel_sums_refuses_what_it_cannot_do(capi):
    """Geometries the summing form does not cover report 0 groups, and the call says so instead of computing."""
    g = capi.conv_geom((9, 9, 5, 2), (3, 3, 5, 7), 1, 1, 1)
    assert capi.conv_forward_sums_groups(g) == 0
    x, f = capi.empty((9, 9, 5, 2), fill=0.0), capi.empty((3, 3, 5, 7), fill=0.0)
    with pytest.raises(capi.McnError) as e:
        capi.conv_forward_sums(x, f, g)
    assert "no such form" in str(e.value)


@pytest.mark.parametrize("K", [48, 80, 96])
def test_conv_forward_with_channel_sums_and_filter_counts_off_the_32_grid(capi, K):
    """Filter counts that leave a partial 32-channel block (48, 80) have no summing form -- the kernel sums where whole
    blocks are stored -- and say so; a count it does take (96) gives the sums of every channel, the last block included."""
    import torch
    xs, fs = (56, 56, 64, 8), (1, 1, 64, K)
    g = capi.conv_geom(xs, fs, 1, 0, 1)
    groups = capi.conv_forward_sums_groups(g)
    r = np.random.default_rng(K)
    xd = capi.to_device(F(r.standard_normal(xs) + 0.3))
    fd = capi.to_device(F(r.standard_normal(fs) * 0.2))
    if K % 32 != 0:
        assert groups == 0
        with pytest.raises(capi.McnError) as e:
            capi.conv_forward_sums(xd, fd, g)
        assert "no such form" in str(e.value)
        return
    assert groups > 0
    y, sums = capi.conv_forward_sums(xd, fd, g)
    assert torch.equal(y, capi.conv_forward(xd, fd, None, g))
    yd = y.double()
    s1, s2 = yd.sum(dim=(0, 2, 3)), (yd * yd).sum(dim=(0, 2, 3))
    tot = sums.sum(dim=1)
    assert float((tot[:, 0] - s1).abs().max() / s1.abs().max()) < 1e-6
    assert float((tot[:, 1] - s2).abs().max() / s2.abs().max()) < 1e-6
    assert float(tot[:, 1].min()) > 0.0


def test_conv_backward_data_with_masked_second_term(capi):
    """dzdx = backward-data + the shortcut's share of the derivative behind a ReLU, the mask as one bit per element:
    bit-identical to writing the masked derivative into dzdx and accumulating the convolution's onto it."""
    import torch
    from util import bits_equal
    r = np.random.default_rng(8)
    xs, fs = (56, 56, 256, 4), (1, 1, 256, 64)
    g = capi.conv_geom(xs, fs, 1, 0, 1)
    assert capi.lib().mcn_conv_backward_data_masked_add_supported(g) == 1
    f = capi.to_device(F(r.standard_normal(fs) * 0.1))
    dy = capi.to_device(F(r.standard_normal((56, 56, 64, 4))))
    addend = capi.to_device(F(r.standard_normal(xs)))
    y = capi.to_device(F(r.standard_normal(xs)))   # the ReLU's output stands in for "what it let through"
    keep = (y.reshape(-1) > 0).to(torch.int64).reshape(-1, 32)
    words = (keep * (1 << torch.arange(32, device="cuda", dtype=torch.int64))).sum(dim=1)
    bits = torch.where(words >= (1 << 31), words - (1 << 32), words).to(torch.int32)
    want = capi.relu_backward(y, addend)            # addend where y > 0, else addend*0
    want = capi.conv_backward_data_acc(want, 1.0, f, dy, g)
    got = capi.conv_backward_data_masked_add(f, dy, g, addend, bits)
    assert bits_equal(capi.to_host(got), capi.to_host(want))
    # a geometry without this form says so
    g2 = capi.conv_geom((9, 9, 5, 2), (3, 3, 5, 7), 1, 1, 1)
    assert capi.lib().mcn_conv_backward_data_masked_add_supported(g2) == 0


STREAMED = [  # H, W, C, N, FH, FW, FC, K, stride, pad, dilate: shapes the streamed-bank kernel takes when the others are off
    (28, 28, 64, 4, 3, 3, 64, 128, 1, 1, 1),                 # 128-channel tiles, taps, padding
    (20, 18, 128, 3, 1, 1, 128, 320, 1, 0, 1),               # no taps; 320 filters: a partial 128-channel tile at the end
    (14, 14, 256, 4, 3, 3, 256, 256, 1, 1, 1),               # few tiles, long reduction: split into partial tensors
    (16, 16, 64, 2, 3, 3, 64, 64, (2, 2), 1, 1),             # 64-channel tiles; strided: stride classes in backward-data
    (12, 12, 128, 3, 3, 3, 128, 96, 1, (2, 0, 1, 1), (2, 1)),  # dilation, asymmetric padding, 96 filters in a 128 tile
    (6, 6, 64, 8, 6, 6, 64, 200, 1, 0, 1),                   # fully connected: one pixel per image
]


@pytest.mark.parametrize("case", STREAMED)
def test_streamed_bank_kernel_on_its_own(capi, ob, case):
    """Forward and backward-data with the weights-stationary kernel switched off and the streamed-bank kernel's split
    reduction on, so that conv_sb_mfma runs shapes the committed configurations would send elsewhere: against the
    oracle at the convolution gate, and the launches are counted so that the test cannot pass on another kernel."""
    H, W, C, N, FH, FW, FC, K, stride, pad, dilate = case
    x, f, b = _tensors(case, seed=11)
    g = capi.conv_geom(x.shape, f.shape, stride, pad, dilate)
    og = ob.conv_geom(x.shape, f.shape, stride, pad, dilate)
    want = ob.conv_forward(x, f, b, og)
    dy = F(np.random.default_rng(12).standard_normal(want.shape))
    wdx, _, _ = ob.conv_backward(x, f, dy, og, want=(True, False, False))
    xd, fd, bd, dyd = capi.to_device(x), capi.to_device(f), capi.to_device(b), capi.to_device(dy)
    capi.set_tunable("conv_no_ws", 1)
    capi.set_tunable("conv_sb_split", 1)
    try:
        capi.profile_begin("conv_sb_mfma")
        y = capi.to_host(capi.conv_forward(xd, fd, bd, g))
        dx = capi.to_host(capi.conv_backward(xd, fd, dyd, g, want=(True, False, False))[0])
        launches, _ = capi.profile_end()
    finally:
        capi.set_tunable("conv_no_ws", 0)
        capi.set_tunable("conv_sb_split", 0)
    assert launches >= 1, launches   # (backward-data of 96 filters x 9 taps = 864 rows is not a multiple of 64: another kernel)
    errs = dict(y=rel_max(y, want), dzdx=rel_max(dx, wdx))
    assert max(errs.values()) <= TOL, errs


TAILED = [  # shapes whose tiles leave a partly filled last round when one workgroup per compute unit is assumed
    (40, 40, 64, 12, 3, 3, 64, 256, 1, 1, 1),   # forward: 300 tiles of 128 channels, 44 in the tail, three splits
    (37, 41, 64, 13, 3, 3, 64, 200, 1, 1, 1),   # a last pixel tile of 9 pixels and a channel tile of 72 of 128 in the tail
    (48, 48, 64, 16, 3, 3, 64, 64, 1, 1, 1),    # 64-channel tiles, forward and backward-data: 288 tiles, 32 in the tail
]


@pytest.mark.parametrize("case", TAILED)
def test_streamed_bank_tail_tiles_split_their_reduction(capi, ob, case):
    """The streamed-bank kernel gives the tiles of a partly filled last round a launch of their own that splits their
    reduction, and a small kernel adds the partial tiles up.  With one resident workgroup per compute unit assumed,
    shapes of a few hundred tiles take that path: forward (with bias) and backward-data against the oracle at the
    convolution gate, the tail's launches counted."""
    x, f, b = _tensors(case, seed=21)
    stride, pad, dilate = case[8:]
    g = capi.conv_geom(x.shape, f.shape, stride, pad, dilate)
    og = ob.conv_geom(x.shape, f.shape, stride, pad, dilate)
    want = ob.conv_forward(x, f, b, og)
    dy = F(np.random.default_rng(22).standard_normal(want.shape))
    wdx, _, _ = ob.conv_backward(x, f, dy, og, want=(True, False, False))
    xd, fd, bd, dyd = capi.to_device(x), capi.to_device(f), capi.to_device(b), capi.to_device(dy)
    capi.set_tunable("conv_no_ws", 1)
    capi.set_tunable("conv_sb_tail_slots", 1)
    try:
        capi.profile_begin("conv_sb_tail_reduce")
        y = capi.to_host(capi.conv_forward(xd, fd, bd, g))
        dx = capi.to_host(capi.conv_backward(xd, fd, dyd, g, want=(True, False, False))[0])
        launches, _ = capi.profile_end()
        # accumulating form through the same path: y = 2 conv(x) + bias + 0.5 y0 (the tail's summing kernel scales, adds
        # the bias and accumulates like the matrix kernel's own epilogue)
        y0 = F(np.random.default_rng(23).standard_normal(want.shape))
        yacc = capi.to_host(capi.conv_forward(xd, fd, bd, g, y=capi.to_device(y0), out_mult=0.5, in_mult=2.0))
        want_acc = 2.0 * (want - b.reshape(1, 1, -1, 1)) + b.reshape(1, 1, -1, 1) + 0.5 * y0
        # the same products with every tile by one workgroup: the tail only changes the order of a tile's partial sums
        capi.set_tunable("conv_sb_tail", 0)
        y1 = capi.to_host(capi.conv_forward(xd, fd, bd, g))
        dx1 = capi.to_host(capi.conv_backward(xd, fd, dyd, g, want=(True, False, False))[0])
    finally:
        capi.set_tunable("conv_no_ws", 0)
        capi.set_tunable("conv_sb_tail_slots", 0)
        capi.set_tunable("conv_sb_tail", 1)
    assert launches >= 1, launches
    errs = dict(y=rel_max(y, want), dzdx=rel_max(dx, wdx), y_whole=rel_max(y1, want), dzdx_whole=rel_max(dx1, wdx),
                y_modes=rel_max(y, y1), dzdx_modes=rel_max(dx, dx1), y_accumulated=rel_max(yacc, want_acc))
    assert max(errs.values()) <= TOL, errs


STRIDED_TOGETHER = [  # strided layers whose backward-data classes share one launch of the tiled kernel
    (28, 28, 128, 4, 3, 3, 128, 128, 2, 1, 1),           # 3x3 /2: four classes of 4, 2, 2 and 1 taps, 128-channel tiles
    (19, 23, 64, 3, 3, 3, 64, 64, (2, 1), (1, 0, 2, 1), 1),   # stride along one axis only: two classes, 64-channel tiles
    (21, 20, 48, 2, 5, 4, 48, 80, 2, (2, 1, 0, 3), (1, 2)),   # dilated columns, ragged tiles, 48 channels of a tile's 64
    (17, 17, 128, 5, 2, 2, 64, 96, 2, 0, 1),             # two filter groups; every class a single tap
]


@pytest.mark.parametrize("case", STRIDED_TOGETHER)
def test_stride_classes_of_backward_data_share_one_launch(capi, ob, case):
    """The backward-data product of a strided layer falls into one product per stride class (bits/nnconv.cu:246-278 does
    it as one GEMM and col2im).  Where the geometry allows, all classes run in one launch of the tiled kernel: against
    the oracle at the convolution gate, overwriting and accumulating (dzdx = dzdx0 + ...), with the banks packed on the
    fly and packed ahead, and against the one-launch-per-class path (the same products; a class may split its
    reduction there, so equal to rounding, not bit for bit; the banks packed ahead serve both paths).  The shared launch
    is counted."""
    from util import bits_equal
    H, W, C, N, FH, FW, FC, K, stride, pad, dilate = case
    r = np.random.default_rng(31)
    x = F(r.standard_normal((H, W, C, N)))
    f = F(r.standard_normal((FH, FW, FC, K)) / np.sqrt(FH * FW * FC))
    g = capi.conv_geom(x.shape, f.shape, stride, pad, dilate)
    og = ob.conv_geom(x.shape, f.shape, stride, pad, dilate)
    dy = F(r.standard_normal(capi.conv_out_shape(g)))
    wdx, _, _ = ob.conv_backward(x, f, dy, og, want=(True, False, False))
    xd, fd, dyd = capi.to_device(x), capi.to_device(f), capi.to_device(dy)
    capi.profile_begin("conv_pix_multi")
    dx = capi.to_host(capi.conv_backward(xd, fd, dyd, g, want=(True, False, False))[0])
    launches, _ = capi.profile_end()
    dx0 = F(r.standard_normal(x.shape))
    acc = capi.to_host(capi.conv_backward_data_acc(capi.to_device(dx0), 1.0, fd, dyd, g))
    packed = capi.conv_pack_filters(fd, g, capi.CONV_BACKWARD_DATA)
    ahead = capi.to_host(capi.conv_backward_data_packed(capi.empty(x.shape), 0.0, fd, packed, dyd, g))
    capi.set_tunable("conv_pix_multi", 0)
    try:
        apart = capi.to_host(capi.conv_backward(xd, fd, dyd, g, want=(True, False, False))[0])
        # (the banks packed ahead lie in one order whichever way the launches go)
        apart_ahead = capi.to_host(capi.conv_backward_data_packed(capi.empty(x.shape), 0.0, fd, packed, dyd, g))
    finally:
        capi.set_tunable("conv_pix_multi", 1)
    assert launches == (2 if FC != C else 1), launches  # (one per filter group)
    assert bits_equal(dx, ahead)
    assert bits_equal(apart, apart_ahead)
    errs = dict(dzdx=rel_max(dx, wdx), accumulated=rel_max(acc, wdx + dx0), apart=rel_max(apart, wdx), paths=rel_max(dx, apart))
    assert max(errs.values()) <= TOL, errs


def test_filter_gradient_on_a_stream_marked_as_beside_another(capi, ob):
    """mcn_stream_beside: filter-gradient launches on a marked stream ask for more local memory than they use (one
    workgroup to a compute unit).  Nothing else changes: same bits as on an unmarked stream, for a tile shape of every
    kind (128 x 128 with two and with three buffers, 192 rows, 64 x 64), and the oracle's values at the convolution gate."""
    import ctypes as C
    import torch
    from util import bits_equal
    side = torch.cuda.Stream()
    L = capi.lib()
    cases = [(14, 14, 256, 8, 1, 1, 256, 256, 1, 0, 1), (28, 28, 128, 4, 3, 3, 128, 128, 1, 1, 1),
             (28, 28, 64, 4, 1, 1, 64, 256, 1, 0, 1), (20, 20, 64, 4, 1, 1, 64, 64, 1, 0, 1)]
    capi.check(L.mcn_stream_beside(C.c_void_p(side.cuda_stream), 1))
    try:
        for case in cases:
            x, f, _ = _tensors(case, seed=41)
            stride, pad, dilate = case[8:]
            g = capi.conv_geom(x.shape, f.shape, stride, pad, dilate)
            og = ob.conv_geom(x.shape, f.shape, stride, pad, dilate)
            dy = F(np.random.default_rng(42).standard_normal(capi.conv_out_shape(g)))
            _, wdf, _ = ob.conv_backward(x, f, dy, og, want=(False, True, False))
            xd, fd, dyd = capi.to_device(x), capi.to_device(f), capi.to_device(dy)
            plain = capi.to_host(capi.conv_backward(xd, fd, dyd, g, want=(False, True, False))[1])
            torch.cuda.synchronize()
            with torch.cuda.stream(side):
                beside = capi.to_host(capi.conv_backward(xd, fd, dyd, g, want=(False, True, False))[1])
            side.synchronize()
            assert bits_equal(plain, beside), case
            assert rel_max(plain, wdf) <= TOL, case
    finally:
        capi.check(L.mcn_stream_beside(C.c_void_p(side.cuda_stream), 0))
