#!/usr/bin/env python3
"""Benchmark of the MI355X back-end on the reference's headline configurations.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one forward+backward pass of the ResNet-50 bottleneck block (BASELINE configs[3]: 56x56, 256/64
channels, N = 32, fp32) through the C++ operator layer, with every tensor resident in HBM before the timed
region.  `value` is images/s over exactly K steps.  The same line carries
  roofline      the kernel that takes most of the step, timed live with HIP events on its launch stream,
  rooflines     the graded kernels on their own configurations: conv backward (configs[4], fp32 MFMA),
                batch-norm backward (configs[1], HBM), max/avg pooling backward (configs[2], HBM).  The HBM-bound
                ones are timed COLD: four sets of tensors used in turn, so that no launch finds its inputs in the
                256 MB memory-side cache because the previous launch left them there (`achieved`); the figure a
                loop over one set of buffers shows is reported beside it as `achieved_warm`,
  resnet50      the whole ResNet-50 (224 x 224) through the same operator classes: forward and whole training steps
                (forward, backward, SGD update) at 32, 64 and 128 images,
  block_plain   the same block through the reference's operator interface only (layer by layer, no folded entry points),
  block_two_streams  the timed schedule with the filter-gradient matrix kernels on a second stream (same bits; not the
                headline, because launches that share the chip cannot be priced per kernel),
  forward_rows  forward convolution / batch normalisation / pooling on the same shapes,
  latency_rows  BASELINE configs[0] (a 7 MB layer: a launch-latency case, not a roofline one),
  double_rows   the untuned double-precision instantiation on reduced forms of the same configurations,
  hbm_ceiling   the best plain read / write / copy kernels of a small sweep, cold, timed in this run: every HBM-bound
                row is also given as a fraction of that measured copy rate,
  mfma_ceiling  the matrix pipe alone (a stream of dependent matrix instructions on every SIMD), timed in this run: every
                matrix-bound row is also given as a fraction of it,
  cpu_baseline  the CPU restatement of the reference path (oracle/) timed on this machine's host cores: the block, and
                one leg per configuration (`per_config`).
One GPU only: nothing here shards.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_FP32 = 157.3e12  # FLOP/s, MI355X dense fp32 matrix
PEAK_HBM = 8.0e12          # B/s
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same counters read for a
# 256 MiB streaming copy.  Counters are not readable from inside this process: profiles/traffic.json holds the values of
# exactly these launches, written by matconvnet_amd/profile_summary.py from the counter runs whose summaries sit
# beside it (each entry names its summary file), together with the calibration factors.
def _load_traffic():
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return {k: v.get("bytes") for k, v in json.load(f).get("kernels", {}).items()}
    except (OSError, ValueError):
        return {}


TRAFFIC = _load_traffic()
COLD_SETS = 4              # tensor sets used in turn by the HBM-bound measurements (> 256 MB between reuses)


def _sig(v, digits=4):
    """Numbers rounded to `digits` significant digits, recursively: the whole JSON line has to stay short enough for the
    driver's record, which keeps the end of it."""
    if isinstance(v, bool) or v is None:
        return v
    if isinstance(v, float):
        if v != v or v in (float("inf"), float("-inf")) or v == 0.0:
            return None if v != v else v
        return float("%.*g" % (digits, v))
    if isinstance(v, dict):
        return {k: _sig(x, digits) for k, x in v.items()}
    if isinstance(v, (list, tuple)):
        return [_sig(x, digits) for x in v]
    return v


def _two_roofs(row, flops=None, hbm_bytes=None):
    """Both roofs of a launch in the row: the time its arithmetic takes at the fp32 matrix peak and the time its HBM
    traffic takes at 8 TB/s (counter bytes where profiles/traffic.json has them, else the algorithmic bytes); `bound`
    names the larger."""
    t_mfma = flops / PEAK_MFMA_FP32 * 1e6 if flops else 0.0
    t_hbm = hbm_bytes / PEAK_HBM * 1e6 if hbm_bytes else 0.0
    row["at_mfma_peak_us"] = t_mfma
    row["at_hbm_peak_us"] = t_hbm
    row["bound"] = "mfma" if t_mfma >= t_hbm else "hbm"
    if "avg_launch_us" in row and row["avg_launch_us"]:
        row["frac_of_its_roof"] = max(t_mfma, t_hbm) / row["avg_launch_us"]
    return row


def _sync():
    import torch
    torch.cuda.synchronize()


SPIN_UP_S = 0.03  # after a pause the device needs some 20 ms of work to come back to its full clock


def spin_up(launch):
    """Untimed calls of `launch` for SPIN_UP_S of device time: the per-operator rows are steady-state figures."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < SPIN_UP_S:
        for _ in range(4):
            launch()
        _sync()


def kernel_time(capi, kernel, launch, reps):
    """Mean duration (s) of `kernel` over `reps` calls of `launch`, from HIP events bracketing each launch (after
    spin_up: see there)."""
    spin_up(launch)
    capi.profile_begin(kernel)
    for _ in range(reps):
        launch()
    n, ms = capi.profile_end()
    return (ms / n) * 1e-3 if n else float("nan"), n


def kernels_time_per_call(capi, pattern, launch, reps):
    """Summed duration (s) per call of `launch` of every kernel whose name contains `pattern` (a product that takes
    several launches), and their number per call."""
    spin_up(launch)
    capi.profile_begin(pattern)
    for _ in range(reps):
        launch()
    n, ms = capi.profile_end()
    return (ms / reps) * 1e-3 if n else float("nan"), n / reps


def _load_block(blk, w):
    for k in ("x", "f1", "f2", "f3", "g1", "b1", "g2", "b2", "g3", "b3"):
        blk.set(k, w[k])
    blk.set("dzdy", w["dy"])


def _time_block(blk, steps, warmup, layer_by_layer=False):
    def run(n):
        if layer_by_layer:
            for _ in range(n):
                blk.forward()
                blk.backward()
        else:
            blk.run(n)

    run(warmup)
    _sync()
    t0 = time.perf_counter()
    run(steps)
    _sync()
    return time.perf_counter() - t0


def bench_block(vlapi, capi, workloads, steps, warmup):
    w = workloads.bottleneck_case()
    N = w["x"].shape[3]
    # Both schedules are built and loaded first, so that no upload sits between the two measurements: after a pause the
    # device takes some 20 ms of work to come back to its full clock (steps of 820 us falling to 755 us), which is the
    # length of a measurement here.
    # The reference-interface-only schedule: every layer a call of its own on vl::nn::Convolution / BatchNorm / ReLU /
    # Sum, nothing folded, nothing packed ahead (what code written against the reference's classes gets unchanged).
    plain_blk = vlapi.Bottleneck(N=N, eps=w["eps"])
    # The timed schedule: the same operator classes for the convolutions, and the library's folded batch-norm entry
    # points, which the reference does not have:
    # fused: ReLU / shortcut sum folded into batch normalisation; packed: the filter banks are re-laid for the matrix
    # kernels by ONE launch at the start of every step (as after an update of the filters) instead of one per product;
    # deferred: the sums over reduction splits that finish the three filter gradients run in one launch at the end;
    # epilogue_sums: the forward convolutions sum their output per channel, batch normalisation takes those sums;
    # mask_bits: the unit's last ReLU leaves its mask as one bit per element for the backward pass
    blk = vlapi.Bottleneck(N=N, eps=w["eps"], fused=True, packed=True, deferred=True, epilogue_sums=True, mask_bits=True)
    # The timed schedule with the filter-gradient matrix kernels on a second stream, beside the batch-norm derivatives
    # of the layer below (same bits).  Reported beside the headline, not as it: with two kernels sharing the chip the
    # duration of a launch says nothing about the kernel, and the roofline figures below are per launch.
    two_blk = vlapi.Bottleneck(N=N, eps=w["eps"], fused=True, overlap=True, packed=True, deferred=True, epilogue_sums=True,
                               mask_bits=True)
    _load_block(plain_blk, w)
    _load_block(blk, w)
    _load_block(two_blk, w)
    dt_plain = _time_block(plain_blk, steps, warmup, layer_by_layer=True)
    dt_two = _time_block(two_blk, steps, warmup)
    dt = _time_block(blk, steps, warmup)
    plain_blk.close()
    two_blk.close()
    plain = dict(ms_per_step=dt_plain / steps * 1e3, images_per_s=N * steps / dt_plain,
                 schedule="layer by layer through vl::nn::Convolution / BatchNorm / ReLU / Sum only",
                 timed_schedule_on_two_streams=dict(
                     ms_per_step=dt_two / steps * 1e3, images_per_s=N * steps / dt_two,
                     schedule="the timed schedule with the filter-gradient matrix kernels on a second stream"))
    # which kernel family dominates the step, and its live duration
    P = 56 * 56
    # per launch family per step.  The six forward + backward-data launches go to the weights-stationary kernel
    # (conv_ws_mfma) when the bank fits in LDS, else to the tiled one (conv_pix_mfma); if a step ever mixes them,
    # they are reported as one family.
    pix_flops = 2.0 * (2.0 * P * N * (256 * 64 + 9 * 64 * 64 + 64 * 256))
    conv_flops = {"conv_wgrad_mfma": 2.0 * P * N * (256 * 64 + 9 * 64 * 64 + 64 * 256)}
    eS, eB = 4.0 * P * 64 * N, 4.0 * P * 256 * N
    hbm_bytes = {  # algorithmic bytes per step of the memory-bound families (reads + writes once each)
        # backward sums read x and dzdy (the forward sums come from the convolutions); bn3's passes also read the last
        # ReLU's mask, one bit per element
        "bnorm_sums": 2 * (eS + eS + eB) + eB / 32,
        "bnorm_forward_apply": 2 * eS + 2 * eS + 3 * eB + eB / 32,  # bn1, bn2 with ReLU; bn3 with shortcut sum, ReLU and its mask bits
        "bnorm_backward_apply": 3 * (eS + eS + eB) + eB / 32,
        "eltwise_kernel": 0.0,                                    # (nothing left: every element-wise layer is folded)
    }
    fam = {}
    for name in ["conv_ws_mfma", "conv_pix_mfma"] + list(conv_flops) + list(hbm_bytes) + ["conv_wgrad_reduce", "conv_pack_weights", "conv_pack_many"]:  # (conv_wgrad_reduce also matches conv_wgrad_reduce_many)
        capi.profile_begin(name)
        blk.run(steps)
        n, ms = capi.profile_end()
        fam[name] = (n, ms * 1e-3)
    blk.close()
    ws, pix = fam.pop("conv_ws_mfma"), fam.pop("conv_pix_mfma")
    pix_name = "conv_ws_mfma" if pix[0] == 0 else ("conv_pix_mfma" if ws[0] == 0 else "conv_ws_mfma+conv_pix_mfma")
    fam[pix_name] = (ws[0] + pix[0], ws[1] + pix[1])
    conv_flops[pix_name] = pix_flops
    top = max(fam, key=lambda k: fam[k][1])
    n, total = fam[top]
    if top in conv_flops:
        achieved = conv_flops[top] * steps / total
        roof = dict(kernel=top, bound="mfma", achieved=achieved / 1e12, peak=PEAK_MFMA_FP32 / 1e12, unit="TFLOP/s",
                    frac=achieved / PEAK_MFMA_FP32, traffic=TRAFFIC.get("block/" + top), launches_per_step=n // steps,
                    avg_launch_us=total / n * 1e6)
        # (`bound` stays the roof `achieved` and `peak` are stated on; `nearer_roof` says which one the mean launch is
        # closer to: the 1x1 layers move 25 FLOP per byte against a machine balance of 20)
        both = _two_roofs(dict(avg_launch_us=total / n * 1e6), conv_flops[top] / (n // steps), roof["traffic"])
        roof.update(at_mfma_peak_us=both["at_mfma_peak_us"], at_hbm_peak_us=both["at_hbm_peak_us"], nearer_roof=both["bound"],
                    frac_of_nearer_roof=both.get("frac_of_its_roof"))
    else:
        work = hbm_bytes.get(top, float("nan"))
        achieved = work * steps / total
        roof = dict(kernel=top, bound="hbm", achieved=achieved / 1e9, peak=PEAK_HBM / 1e9, unit="GB/s",
                    frac=achieved / PEAK_HBM, traffic=TRAFFIC.get("block/" + top), launches_per_step=n // steps, avg_launch_us=total / n * 1e6)
    breakdown = {k: round(v[1] / steps * 1e3, 4) for k, v in fam.items()}  # ms per step by kernel family
    return N * steps / dt, dt / steps * 1e3, roof, breakdown, plain


def bench_conv_bwd(capi, workloads, reps):
    """BASELINE configs[4]: 3x3x256x256 on 56x56x256x64, stride 1, pad 1: dzdx + dzdf (+ dzdb)."""
    import ctypes as C
    import torch
    L = capi.lib()
    xs, fs = (56, 56, 256, 64), (3, 3, 256, 256)
    g = capi.conv_geom(xs, fs, 1, 1, 1)
    x = torch.randn(tuple(reversed(xs)), device="cuda")
    f = torch.randn(tuple(reversed(fs)), device="cuda") * float(np.sqrt(2.0 / (9 * 256)))
    dy = torch.randn(tuple(reversed(xs)), device="cuda")
    dx, df, db = capi.empty(xs), capi.empty(fs), capi.empty((256,))
    ws = capi.Workspace()
    nbytes = max(L.mcn_conv_workspace_bytes(C.byref(g), k) for k in range(4))
    wp, wn = ws.get(nbytes)
    st = capi.stream()
    flops = 2.0 * 56 * 56 * 9 * 256 * 256 * 64
    data = lambda: capi.check(L.mcn_conv_backward_data(st, C.byref(g), capi.ptr(dx), capi.ptr(f), capi.ptr(dy), wp, wn))
    filt = lambda: capi.check(L.mcn_conv_backward_filter(st, C.byref(g), capi.ptr(df), capi.ptr(x), capi.ptr(dy), wp, wn))
    bias = lambda: capi.check(L.mcn_conv_backward_bias(st, C.byref(g), capi.ptr(db), capi.ptr(dy), wp, wn))
    for fn in (data, filt, bias):
        fn()
    _sync()
    # backward-data goes to the streamed-bank kernel when it takes the shape (conv_sb_mfma for the full rounds of
    # resident workgroups, the same kernel once more for the left-over tiles with their reduction split, and
    # conv_sb_tail_reduce: the row's time is the three together), else to the tiled one
    data_kernel = "conv_sb_mfma"
    t_data, n_data = kernels_time_per_call(capi, "conv_sb_", data, reps)
    if n_data == 0:
        data_kernel = "conv_pix_mfma"
        t_data, _ = kernel_time(capi, data_kernel, data, reps)
    elif n_data > 1:
        data_kernel = "conv_sb_mfma (%d launches: full rounds, left-over tiles split, their sum)" % round(n_data)
    t_filt, _ = kernel_time(capi, "conv_wgrad_mfma", filt, reps)
    t_red, _ = kernel_time(capi, "conv_wgrad_reduce", filt, reps)
    # whole backward call (all launches incl. weight packing, partial-sum reduction and bias), wall clock
    _sync()
    t0 = time.perf_counter()
    for _ in range(reps):
        data(); filt(); bias()
    _sync()
    t_all = (time.perf_counter() - t0) / reps
    out = []
    for name, kern, t in (("conv backward-data", data_kernel, t_data), ("conv backward-filter", "conv_wgrad_mfma", t_filt)):
        row = dict(op=name, kernel=kern, workload="configs[4] 3x3x256x256 on 56x56x256x64", bound="mfma",
                   achieved=flops / t / 1e12, peak=PEAK_MFMA_FP32 / 1e12, unit="TFLOP/s", frac=flops / t / PEAK_MFMA_FP32,
                   avg_launch_us=t * 1e6, traffic=TRAFFIC.get("cfg5/" + kern.split(" ")[0]))
        out.append(_two_roofs(row, flops, row["traffic"]))
    whole = dict(tflops=2 * flops / t_all / 1e12, frac=2 * flops / t_all / PEAK_MFMA_FP32, ms=t_all * 1e3,
                 wgrad_reduce_us=t_red * 1e6)
    return out, whole


def bench_bnorm_bwd(capi, workloads, reps):
    """BASELINE configs[1]: 56x56x256x32, moments from the batch."""
    import ctypes as C
    import torch
    L = capi.lib()
    H, W, Cc, N = 56, 56, 256, 32
    xs = [torch.randn((N, Cc, W, H), device="cuda") * 1.3 + 0.5 for _ in range(COLD_SETS)]
    dys = [torch.randn((N, Cc, W, H), device="cuda") for _ in range(COLD_SETS)]
    dxs = [capi.empty((H, W, Cc, N)) for _ in range(COLD_SETS)]
    g = torch.rand(Cc, device="cuda") + 0.5
    dg, db, mom = capi.empty((Cc,)), capi.empty((Cc,)), capi.empty((Cc, 2))
    ws = capi.Workspace()
    wp, wn = ws.get(L.mcn_bnorm_workspace_bytes(H, W, Cc, N))
    st = capi.stream()
    turn = [0]

    def make(sets):
        def call():
            i = turn[0] % sets
            turn[0] += 1
            capi.check(L.mcn_bnorm_backward(st, capi.ptr(dxs[i]), capi.ptr(dg), capi.ptr(db), capi.ptr(mom), capi.ptr(xs[i]),
                                            capi.ptr(g), capi.ptr(dys[i]), H, W, Cc, N, 1e-4, 0, wp, wn))
        return call

    E = 4.0 * H * W * Cc * N
    t = {}
    for label, sets in (("cold", COLD_SETS), ("warm", 1)):
        call = make(sets)
        for _ in range(COLD_SETS):
            call()
        _sync()
        t_sums, _ = kernel_time(capi, "bnorm_sums", call, reps)
        t_apply, _ = kernel_time(capi, "bnorm_backward_apply", call, reps)
        _sync()
        t0 = time.perf_counter()
        for _ in range(reps):
            call()
        _sync()
        t[label] = (t_sums, t_apply, (time.perf_counter() - t0) / reps)
    rows = [
        dict(op="bnorm backward, pass 1 (sums)", kernel="bnorm_sums", workload="configs[1] 56x56x256x32", bound="hbm",
             achieved=2 * E / t["cold"][0] / 1e9, peak=PEAK_HBM / 1e9, unit="GB/s", frac=2 * E / t["cold"][0] / PEAK_HBM,
             avg_launch_us=t["cold"][0] * 1e6, achieved_warm=2 * E / t["warm"][0] / 1e9, traffic=TRAFFIC.get("cfg2/bnorm_sums")),
        dict(op="bnorm backward, pass 2 (apply)", kernel="bnorm_backward_apply", workload="configs[1] 56x56x256x32", bound="hbm",
             achieved=3 * E / t["cold"][1] / 1e9, peak=PEAK_HBM / 1e9, unit="GB/s", frac=3 * E / t["cold"][1] / PEAK_HBM,
             avg_launch_us=t["cold"][1] * 1e6, achieved_warm=3 * E / t["warm"][1] / 1e9, traffic=TRAFFIC.get("cfg2/bnorm_backward_apply")),
    ]
    t_all = t["cold"][2]
    whole = dict(gbs=5 * E / t_all / 1e9, frac=5 * E / t_all / PEAK_HBM, us=t_all * 1e6, gbs_compulsory=3 * E / t_all / 1e9,
                 gbs_warm=5 * E / t["warm"][2] / 1e9, us_warm=t["warm"][2] * 1e6)
    return rows, whole


def bench_pool_bwd(capi, workloads, reps):
    """BASELINE configs[2]: (a) max 3x3 s2 p1 on 112x112x64x32, (b) avg 2x2 s2 on 56x56x256x32."""
    import ctypes as C
    import torch
    L = capi.lib()
    rows = []
    for name, shape, pool, pad, method in (("max-pool backward", (112, 112, 64, 32), 3, 1, "max"),
                                           ("avg-pool backward", (56, 56, 256, 32), 2, 0, "avg")):
        g = capi.pool_geom(shape, pool, 2, pad, method)
        oshape = capi.pool_out_shape(g)
        xs = [torch.randn(tuple(reversed(shape)), device="cuda") for _ in range(COLD_SETS)]
        dys = [torch.randn(tuple(reversed(oshape)), device="cuda") for _ in range(COLD_SETS)]
        dxs = [capi.empty(shape) for _ in range(COLD_SETS)]
        st = capi.stream()
        turn = [0]

        def make(sets):
            def call():
                i = turn[0] % sets
                turn[0] += 1
                capi.check(L.mcn_pool_backward(st, C.byref(g), capi.ptr(dxs[i]), capi.ptr(xs[i]), capi.ptr(dys[i]), 0))
            return call

        e, o = 4.0 * np.prod(shape), 4.0 * np.prod(oshape)
        nbytes = (2 * e + o) if method == "max" else (e + o)
        t = {}
        for label, sets in (("cold", COLD_SETS), ("warm", 1)):
            call = make(sets)
            for _ in range(COLD_SETS):
                call()
            _sync()
            t[label], _ = kernel_time(capi, "pool_backward", call, reps)
        rows.append(dict(op=name, kernel="pool_max_backward_stream" if method == "max" else "pool_backward_avg_tiles",
                         workload="configs[2] %s on %s" % (method, "x".join(map(str, shape))),
                         bound="hbm", achieved=nbytes / t["cold"] / 1e9, peak=PEAK_HBM / 1e9, unit="GB/s",
                         frac=nbytes / t["cold"] / PEAK_HBM, avg_launch_us=t["cold"] * 1e6,
                         achieved_warm=nbytes / t["warm"] / 1e9,
                         traffic=TRAFFIC.get("cfg3a/pool" if method == "max" else "cfg3b/pool")))
        del xs, dys, dxs
    return rows


def _event_time(fn, reps, warm=2):
    """Mean wall time (s) of fn() over `reps` back-to-back calls, from a pair of events on the stream the library
    launches on (torch's current stream is the one capi.stream() hands to every entry point)."""
    import torch
    for _ in range(warm):
        fn()
    spin_up(fn)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    _sync()
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    _sync()
    return a.elapsed_time(b) * 1e-3 / reps


def bench_hbm_ceiling(capi, reps):
    """A small sweep of the plain streaming kernels (mcn_hbm_yardstick: the launch shapes that came out on top of the
    full sweep of `mcn_bench --only yardstick`, profiles/hbm_yardstick_sweep.txt), 256 MiB per stream, cold (buffer sets
    in turn): the measured ceiling of read-only, write-only and copy traffic on this device."""
    import ctypes as C
    import torch
    L = capi.lib()
    nbytes = 256 << 20
    src = [torch.ones(nbytes // 4, device="cuda") for _ in range(COLD_SETS)]
    dst = [torch.empty(nbytes // 4, device="cuda") for _ in range(COLD_SETS)]
    cus = int(L.mcn_device_compute_units())
    st = capi.stream()
    out = {}
    # (mode, width, accesses in flight, workgroups per CU (0: one step each), flags (1: non-temporal stores))
    shapes = {"read": [(0, 4, 4, 0, 0), (0, 4, 8, 4, 0), (0, 16, 2, 4, 0), (0, 4, 4, 16, 0)],
              "write": [(1, 4, 2, 0, 1), (1, 16, 1, 0, 0), (1, 16, 1, 0, 1), (1, 4, 4, 0, 0)],
              "copy": [(2, 4, 4, 0, 1), (2, 4, 4, 0, 0), (2, 16, 1, 0, 0), (2, 16, 1, 4, 0)]}
    def sweep(cands, nb):
        best = None
        for mode, width, in_flight, per_cu, flags in cands:
            turn = [0]

            def call():
                i = turn[0] % COLD_SETS
                turn[0] += 1
                capi.check(L.mcn_hbm_yardstick(st, capi.ptr(dst[i]), capi.ptr(src[i]), nb, mode, width, in_flight,
                                               per_cu * cus, flags))
            for _ in range(COLD_SETS):
                call()
            t, _ = kernel_time(capi, "yardstick_kernel", call, reps)
            gbs = (2 if mode == 2 else 1) * nb / t / 1e9
            if best is None or gbs > best["gbs"]:
                best = dict(gbs=gbs, frac_of_peak=gbs * 1e9 / PEAK_HBM, us=t * 1e6, width_bytes=width, in_flight=in_flight,
                            workgroups_per_cu=per_cu, non_temporal=bool(flags & 1), bytes_per_stream=nb)
        return best

    for name, cands in shapes.items():
        out[name] = sweep(cands, nbytes)
    # the same copy kernels moving what one max-pooling backward launch moves (231 MB in all: launch ramp and tail
    # weigh more on a 40 us kernel than on a 90 us one)
    out["copy_231MB"] = sweep(shapes["copy"], 110 << 20)
    return out


def bench_mfma_ceiling(capi, reps):
    """The matrix pipe alone (mcn_mfma_yardstick: four wavefronts per SIMD, each a dependent chain of matrix instructions
    and nothing else), timed in this run: what the chip reaches of its nominal peak at the clock it holds under such a
    stream.  Every matrix-bound row is also given as a fraction of that."""
    import ctypes as C
    import torch
    L = capi.lib()
    st = capi.stream()
    sink = torch.zeros(4, device="cuda")
    out = {}
    for name, is_double, peak, iters in (("fp32", 0, PEAK_MFMA_FP32, 2000), ("fp64", 1, 78.6e12, 1000)):
        flop = C.c_double(0.0)

        def call():
            capi.check(L.mcn_mfma_yardstick(st, capi.ptr(sink), iters, is_double, C.byref(flop)))
        for _ in range(3):
            call()
        t, _ = kernel_time(capi, "mfma_yardstick_kernel", call, reps)
        out[name] = dict(tflops=flop.value / t / 1e12, frac_of_peak=flop.value / t / peak, us=t * 1e6,
                         instruction="v_mfma_f64_16x16x4_f64" if is_double else "v_mfma_f32_32x32x2_f32")
    return out


def bench_forward(capi, reps):
    """Forward kernels on the graded shapes: convolution (the three layers of the block, configs[3], and configs[4]),
    batch normalisation (configs[1], moments from the batch) and pooling (configs[2]).  Convolutions: whole call, events
    on the launch stream.  The HBM-bound ones cold, like their backward rows."""
    import ctypes as C
    import torch
    L = capi.lib()
    st = capi.stream()
    rows = []
    ws = capi.Workspace()
    for label, xs, fs, pad in (("configs[3] conv1 1x1x256x64 on 56x56x256x32", (56, 56, 256, 32), (1, 1, 256, 64), 0),
                               ("configs[3] conv2 3x3x64x64 on 56x56x64x32", (56, 56, 64, 32), (3, 3, 64, 64), 1),
                               ("configs[3] conv3 1x1x64x256 on 56x56x64x32", (56, 56, 64, 32), (1, 1, 64, 256), 0),
                               ("configs[4] 3x3x256x256 on 56x56x256x64", (56, 56, 256, 64), (3, 3, 256, 256), 1)):
        g = capi.conv_geom(xs, fs, 1, pad, 1)
        ys = capi.conv_out_shape(g)
        sets = 2 if xs[3] == 64 else COLD_SETS
        xv = [torch.randn(tuple(reversed(xs)), device="cuda") for _ in range(sets)]
        yv = [capi.empty(ys) for _ in range(sets)]
        f = torch.randn(tuple(reversed(fs)), device="cuda") * float(np.sqrt(2.0 / (fs[0] * fs[1] * fs[2])))
        wp, wn = ws.get(L.mcn_conv_workspace_bytes(C.byref(g), 0))
        turn = [0]

        def call():
            i = turn[0] % sets
            turn[0] += 1
            capi.check(L.mcn_conv_forward(st, C.byref(g), capi.ptr(yv[i]), 0.0, capi.ptr(xv[i]), 1.0, capi.ptr(f), None, wp, wn))
        t = _event_time(call, reps, warm=sets)
        flops = 2.0 * ys[0] * ys[1] * ys[2] * ys[3] * fs[0] * fs[1] * fs[2]
        nbytes = 4.0 * (np.prod(xs) + np.prod(ys) + np.prod(fs))
        rows.append(dict(op="conv forward", workload=label, bound="mfma", achieved=flops / t / 1e12, peak=PEAK_MFMA_FP32 / 1e12,
                         unit="TFLOP/s", frac=flops / t / PEAK_MFMA_FP32, call_us=t * 1e6,
                         flop_per_byte=flops / nbytes, hbm_gbs=nbytes / t / 1e9))
        del xv, yv
    # batch normalisation forward, configs[1]: reads x twice (sums, apply), writes y
    H, W, Cc, N = 56, 56, 256, 32
    xv = [torch.randn((N, Cc, W, H), device="cuda") * 1.3 + 0.5 for _ in range(COLD_SETS)]
    yv = [capi.empty((H, W, Cc, N)) for _ in range(COLD_SETS)]
    gm, bs, mom = torch.rand(Cc, device="cuda") + 0.5, torch.randn(Cc, device="cuda") * 0.1, capi.empty((Cc, 2))
    wp, wn = ws.get(L.mcn_bnorm_workspace_bytes(H, W, Cc, N))
    turn = [0]

    def bn():
        i = turn[0] % COLD_SETS
        turn[0] += 1
        capi.check(L.mcn_bnorm_forward(st, capi.ptr(yv[i]), capi.ptr(mom), capi.ptr(xv[i]), capi.ptr(gm), capi.ptr(bs),
                                       H, W, Cc, N, 1e-4, 0, wp, wn))
    t = _event_time(bn, reps, warm=COLD_SETS)
    E = 4.0 * H * W * Cc * N
    rows.append(dict(op="bnorm forward (sums + apply)", workload="configs[1] 56x56x256x32", bound="hbm", achieved=3 * E / t / 1e9,
                     peak=PEAK_HBM / 1e9, unit="GB/s", frac=3 * E / t / PEAK_HBM, call_us=t * 1e6,
                     achieved_compulsory=2 * E / t / 1e9))
    del xv, yv
    for name, shape, pool, pad, method in (("max-pool forward", (112, 112, 64, 32), 3, 1, "max"),
                                           ("avg-pool forward", (56, 56, 256, 32), 2, 0, "avg")):
        g = capi.pool_geom(shape, pool, 2, pad, method)
        oshape = capi.pool_out_shape(g)
        xv = [torch.randn(tuple(reversed(shape)), device="cuda") for _ in range(COLD_SETS)]
        yv = [capi.empty(oshape) for _ in range(COLD_SETS)]
        turn = [0]

        def pf():
            i = turn[0] % COLD_SETS
            turn[0] += 1
            capi.check(L.mcn_pool_forward(st, C.byref(g), capi.ptr(yv[i]), capi.ptr(xv[i])))
        t = _event_time(pf, reps, warm=COLD_SETS)
        nbytes = 4.0 * (np.prod(shape) + np.prod(oshape))
        rows.append(dict(op=name, workload="configs[2] %s on %s" % (method, "x".join(map(str, shape))), bound="hbm",
                         achieved=nbytes / t / 1e9, peak=PEAK_HBM / 1e9, unit="GB/s", frac=nbytes / t / PEAK_HBM, call_us=t * 1e6))
        del xv, yv
    return rows


def bench_conv_single(capi, workloads, reps):
    """BASELINE configs[0]: one vl_nnconv layer, 5x5x3x32 on 32x32x3x100, stride 1, pad 2 -- forward, and backward (dzdx,
    dzdf, dzdb).  1.2 MB in, 13 MB out, 0.49 GFLOP per product: a launch-latency case (a handful of microseconds per
    launch), so the fractions of the matrix peak say little; the times are the figure."""
    import ctypes as C
    L = capi.lib()
    w = workloads.conv_single()
    g = capi.conv_geom(w["x"].shape, w["f"].shape, w["stride"], w["pad"], w["dilate"])
    x, f, b, dy = (capi.to_device(w[k]) for k in ("x", "f", "b", "dy"))
    y, dx, df, db = capi.empty(w["dy"].shape), capi.empty(w["x"].shape), capi.empty(w["f"].shape), capi.empty((32,))
    ws = capi.Workspace()
    wp, wn = ws.get(max(L.mcn_conv_workspace_bytes(C.byref(g), k) for k in range(4)))
    st = capi.stream()
    flops = 2.0 * 32 * 32 * 100 * 75 * 32
    calls = {
        "forward": lambda: capi.check(L.mcn_conv_forward(st, C.byref(g), capi.ptr(y), 0.0, capi.ptr(x), 1.0, capi.ptr(f), capi.ptr(b), wp, wn)),
        "backward-data": lambda: capi.check(L.mcn_conv_backward_data(st, C.byref(g), capi.ptr(dx), capi.ptr(f), capi.ptr(dy), wp, wn)),
        "backward-filter": lambda: capi.check(L.mcn_conv_backward_filter(st, C.byref(g), capi.ptr(df), capi.ptr(x), capi.ptr(dy), wp, wn)),
        "backward-bias": lambda: capi.check(L.mcn_conv_backward_bias(st, C.byref(g), capi.ptr(db), capi.ptr(dy), wp, wn)),
        # (what Convolution::backward calls when both are asked for: one pass over dzdy gives both)
        "backward-filter and -bias, one call": lambda: capi.check(L.mcn_conv_backward_filter_bias(
            st, C.byref(g), capi.ptr(df), capi.ptr(db), capi.ptr(x), capi.ptr(dy), wp, wn)),
    }
    rows = []
    for name, fn in calls.items():
        t = _event_time(fn, reps * 4, warm=3)
        row = dict(op="conv " + name, workload="configs[0] 5x5x3x32 on 32x32x3x100", call_us=t * 1e6, kind="latency case")
        if name != "backward-bias":
            row.update(bound="mfma", achieved=flops / t / 1e12, peak=PEAK_MFMA_FP32 / 1e12, unit="TFLOP/s", frac=flops / t / PEAK_MFMA_FP32)
        else:
            row.update(bound="hbm", achieved=w["dy"].nbytes / t / 1e9, peak=PEAK_HBM / 1e9, unit="GB/s", frac=w["dy"].nbytes / t / PEAK_HBM)
        rows.append(row)

    def backward():
        calls["backward-data"](); calls["backward-filter and -bias, one call"]()
    t = _event_time(backward, reps * 4, warm=3)
    whole = dict(backward_us=t * 1e6, backward_tflops=2 * flops / t / 1e12, backward_frac_of_mfma_peak=2 * flops / t / PEAK_MFMA_FP32)
    return rows, whole


def bench_double(capi, workloads, reps):
    """The double-precision instantiation on reduced forms of the graded configurations (convolutions on the fp64 matrix
    instruction where a product has sixteen columns or more, the pooling derivatives on single precision's streaming
    kernels instantiated for double, batch norm as two streaming passes): measured so that its distance to the roofline is on record."""
    import torch
    rows = []
    w = workloads.conv_single()
    g = capi.conv_geom(w["x"].shape, w["f"].shape, w["stride"], w["pad"], w["dilate"])
    x, f, dy = (capi.to_device(w[k], np.float64) for k in ("x", "f", "dy"))
    flops = 3 * 2.0 * 32 * 32 * 100 * 75 * 32
    t = _event_time(lambda: capi.conv_backward(x, f, dy, g), max(2, reps // 4), warm=1)
    rows.append(dict(op="conv backward (dzdx, dzdf, dzdb), double", workload="configs[0] 5x5x3x32 on 32x32x3x100", call_us=t * 1e6,
                     achieved=flops / t / 1e12, unit="TFLOP/s", peak=78.6, frac=flops / t / 78.6e12,
                     bound="fp64: dzdf on v_mfma_f64_16x16x4_f64, dzdx (3 channels) on vector FMAs"))
    del x, f, dy
    # a layer with enough channels for the matrix instruction in every product: configs[3]'s 3x3 convolution
    xs, fs = (56, 56, 64, 32), (3, 3, 64, 64)
    g = capi.conv_geom(xs, fs, 1, 1, 1)
    x = torch.randn(tuple(reversed(xs)), device="cuda", dtype=torch.float64)
    f = torch.randn(tuple(reversed(fs)), device="cuda", dtype=torch.float64)
    dy = torch.randn(tuple(reversed(xs)), device="cuda", dtype=torch.float64)
    flops = 2 * 2.0 * 56 * 56 * 32 * 576 * 64
    t = _event_time(lambda: capi.conv_backward(x, f, dy, g, want=(True, True, False)), max(2, reps // 4), warm=1)
    rows.append(dict(op="conv backward (dzdx, dzdf), double", workload="configs[3] conv2 3x3x64x64 on 56x56x64x32", call_us=t * 1e6,
                     achieved=flops / t / 1e12, unit="TFLOP/s", peak=78.6, frac=flops / t / 78.6e12, bound="fp64 mfma"))
    del x, f, dy
    H, W, Cc, N = 56, 56, 256, 8
    xb = torch.randn((N, Cc, W, H), device="cuda", dtype=torch.float64)
    dyb = torch.randn((N, Cc, W, H), device="cuda", dtype=torch.float64)
    gb = torch.rand(Cc, device="cuda", dtype=torch.float64) + 0.5
    t = _event_time(lambda: capi.bnorm_backward(xb, gb, dyb, 1e-4), reps, warm=2)
    nbytes = 5 * 8.0 * H * W * Cc * N
    rows.append(dict(op="bnorm backward, double", workload="56x56x256x8 (configs[1] at a quarter of the batch)", call_us=t * 1e6,
                     achieved=nbytes / t / 1e9, unit="GB/s", peak=PEAK_HBM / 1e9, frac=nbytes / t / PEAK_HBM, bound="hbm"))
    shape = (112, 112, 64, 8)
    gp = capi.pool_geom(shape, 3, 2, 1, "max")
    xp = torch.randn(tuple(reversed(shape)), device="cuda", dtype=torch.float64)
    dyp = torch.randn(tuple(reversed(capi.pool_out_shape(gp))), device="cuda", dtype=torch.float64)
    t = _event_time(lambda: capi.pool_backward(xp, dyp, gp), reps, warm=2)
    nbytes = 8.0 * (2 * np.prod(shape) + np.prod(capi.pool_out_shape(gp)))
    rows.append(dict(op="max-pool backward, double", workload="112x112x64x8 (configs[2]a at a quarter of the batch)", call_us=t * 1e6,
                     achieved=nbytes / t / 1e9, unit="GB/s", peak=PEAK_HBM / 1e9, frac=nbytes / t / PEAK_HBM, bound="hbm"))
    del xp, dyp
    shape = (56, 56, 256, 8)
    gp = capi.pool_geom(shape, 2, 2, 0, "avg")
    xp = torch.empty(tuple(reversed(shape)), device="cuda", dtype=torch.float64)
    dyp = torch.randn(tuple(reversed(capi.pool_out_shape(gp))), device="cuda", dtype=torch.float64)
    t = _event_time(lambda: capi.pool_backward(xp, dyp, gp), reps, warm=2)
    nbytes = 8.0 * (np.prod(shape) + np.prod(capi.pool_out_shape(gp)))
    rows.append(dict(op="avg-pool backward, double", workload="56x56x256x8 (configs[2]b at a quarter of the batch)", call_us=t * 1e6,
                     achieved=nbytes / t / 1e9, unit="GB/s", peak=PEAK_HBM / 1e9, frac=nbytes / t / PEAK_HBM, bound="hbm"))
    return rows


def bench_resnet50(vlapi, batch, steps, warmup):
    """Whole ResNet-50 (224 x 224, 1000 classes; examples/imagenet/cnn_imagenet_init_resnet.m) through the same
    operator classes: forward alone (training-mode batch normalisation), the training step forward + loss derivative
    (softmax log-loss on random labels) + backward + SGD update, and evaluation (stored moments; the mode of the reference's published 396 images/s,
    doc/site/docs/pretrained.md:233, measured there on other hardware), images/s."""
    import torch
    # (overlap: in backward the units' filter gradients run on a second stream beside the kernels that follow them on
    # the network's stream -- same bits, tests/test_gpu_resnet.py; the one-stream step is reported beside it)
    net = vlapi.ResNet50(N=batch, eps=1e-5, image_size=224, classes=1000, fused=True, seed=11, channel_sums=True, overlap=True)
    try:
        r = np.random.default_rng(12)
        net.set("input", np.asfortranarray(r.standard_normal((224, 224, 3, batch), dtype=np.float32)))
        net.set("labels", np.asfortranarray(r.integers(1, 1001, (1, 1, 1, batch)).astype(np.float32)))

        def timed(fn):
            for _ in range(warmup):
                fn()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            _sync()
            a.record()
            for _ in range(steps):
                fn()
            b.record()
            _sync()
            return a.elapsed_time(b) / steps

        def train():
            net.forward()
            net.loss_derivative()
            net.backward()
            net.sgd_step(1e-3, 0.9, 1e-4)

        fwd_ms, step_ms = timed(net.forward), timed(train)
        net.set_overlap(False)
        one_stream_ms = timed(train)
        net.set_overlap(True)
        net.set_test_mode(True)     # evaluation: batch normalisation with the moving averages of the steps above
        eval_ms = timed(net.forward)
        net.set_test_mode(False)
        flops = net.forward_flops_per_image * batch
        return {"batch": batch, "eval_ms": eval_ms, "eval_images_per_s": batch / eval_ms * 1e3,
                "forward_ms": fwd_ms, "forward_images_per_s": batch / fwd_ms * 1e3,
                "train_step_ms": step_ms, "train_images_per_s": batch / step_ms * 1e3,
                "train_conv_tflops": 3 * flops / step_ms / 1e9, "parameters": net.parameters,
                "schedule": "filter gradients on a second stream", "train_step_ms_on_one_stream": one_stream_ms}
    finally:
        net.close()


def bench_resnet50_sections(capi, batch, reps):
    """The convolutions of ResNet-50 (examples/imagenet/cnn_imagenet_init_resnet.m:52-134) section by section, each layer
    shape timed on its own through the C ABI (whole call, events on the launch stream, one set of buffers reused) and
    weighted by how often the network has it: TFLOP/s of the forward, backward-data and backward-filter products per
    section.  Where the whole-network step loses against these figures is batch normalisation, pooling, the update and
    cold caches between layers."""
    import ctypes as C
    import torch
    L = capi.lib()
    st = capi.stream()
    layers = [("conv1", "stem 7x7 3->64 /2", 224, 3, 7, 64, 2, 3, 1)]
    H, Cc = 56, 64
    for s_, units in enumerate((3, 4, 6, 3)):
        M, Co = 64 << s_, 256 << s_
        stride = 2 if s_ >= 1 else 1
        sec = "conv%d_x" % (s_ + 2)
        layers.append((sec, "1x1 %d->%d" % (Cc, M), H, Cc, 1, M, 1, 0, 1))
        layers.append((sec, "3x3 %d->%d /%d" % (M, M, stride), H, M, 3, M, stride, 1, 1))
        layers.append((sec, "1x1 %d->%d /%d (shortcut)" % (Cc, Co, stride), H, Cc, 1, Co, stride, 0, 1))
        H = (H - 1) // stride + 1
        layers.append((sec, "1x1 %d->%d" % (M, Co), H, M, 1, Co, 1, 0, units))
        layers.append((sec, "1x1 %d->%d" % (Co, M), H, Co, 1, M, 1, 0, units - 1))
        layers.append((sec, "3x3 %d->%d" % (M, M), H, M, 3, M, 1, 1, units - 1))
        Cc = Co
    ws = capi.Workspace()
    table = {}
    for sec, _, Hh, Cin, fh, Cout, stride, pad, count in layers:
        xs, fs = (Hh, Hh, Cin, batch), (fh, fh, Cin, Cout)
        g = capi.conv_geom(xs, fs, stride, pad, 1)
        ys = capi.conv_out_shape(g)
        flops = 2.0 * ys[0] * ys[1] * batch * fh * fh * Cin * Cout
        x = torch.randn(tuple(reversed(xs)), device="cuda")
        f = torch.randn(tuple(reversed(fs)), device="cuda") * 0.05
        dy = torch.randn(tuple(reversed(ys)), device="cuda")
        dx, y, df = capi.empty(xs), capi.empty(ys), capi.empty(fs)
        wp, wn = ws.get(max(L.mcn_conv_workspace_bytes(C.byref(g), k) for k in range(4)))
        calls = (lambda: capi.check(L.mcn_conv_forward(st, C.byref(g), capi.ptr(y), 0.0, capi.ptr(x), 1.0, capi.ptr(f), None, wp, wn)),
                 lambda: capi.check(L.mcn_conv_backward_data(st, C.byref(g), capi.ptr(dx), capi.ptr(f), capi.ptr(dy), wp, wn)),
                 lambda: capi.check(L.mcn_conv_backward_filter(st, C.byref(g), capi.ptr(df), capi.ptr(x), capi.ptr(dy), wp, wn)))
        row = table.setdefault(sec, dict(section=sec, gflop_per_pass=0.0, forward_us=0.0, backward_data_us=0.0, backward_filter_us=0.0))
        row["gflop_per_pass"] += count * flops / 1e9
        for key, fn in zip(("forward_us", "backward_data_us", "backward_filter_us"), calls):
            if sec == "conv1" and key == "backward_data_us":
                continue  # (nothing consumes the input gradient of the first layer: the network driver skips it)
            row[key] += count * _event_time(fn, reps, warm=2) * 1e6
        del x, f, dy, dx, y, df
    out = []
    for row in table.values():
        for key in ("forward", "backward_data", "backward_filter"):
            us = row[key + "_us"]
            row[key + "_tflops"] = row["gflop_per_pass"] / us * 1e3 if us > 0 else None
        out.append(row)
    return out


def cpu_baseline(workloads):
    """The CPU restatement of the reference path on this host: one forward+backward of the same block
    (same N = 32 inputs), GEMMs threaded like the reference's BLAS, everything else serial."""
    from oracle import binding as ob
    from oracle import blocks
    blas = ob.use_openblas(True)
    w = workloads.bottleneck_case()
    N = w["x"].shape[3]
    blocks.bottleneck(workloads.bottleneck_case(N=2))  # warm the threads and pages
    t0 = time.perf_counter()
    reps = 0
    while reps < 1 or (time.perf_counter() - t0 < 12.0 and reps < 20):   # about 12 s of CPU work
        blocks.bottleneck(w)
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    ob.use_openblas(False)
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    return dict(value=N / dt, unit="images/s", cores=cores, kind="port",
                sample="%d full forward+backward passes of the same N=%d block; oracle/ (im2row + sgemm per image, serial "
                       "bnorm/relu loops); sgemm = %s" % (reps, N, "OpenBLAS (numpy wheel), threaded" if blas else "built-in OpenMP kernel"),
                ms_per_step=dt * 1e3)


def _cpu_time(fn, budget_s, max_reps=50):
    fn()  # pages and threads warm
    t0 = time.perf_counter()
    reps = 0
    while reps < 1 or (time.perf_counter() - t0 < budget_s and reps < max_reps):
        fn()
        reps += 1
    return (time.perf_counter() - t0) / reps, reps


def cpu_per_config(workloads):
    """One CPU leg per configuration, beside the GPU rows: the reference's own compiled loops where oracle/_ref holds them
    (batch normalisation bits/nnbnorm.cu:101-164, pooling bits/nnpooling.cu:170-214; kind "reference", serial as the
    reference runs them), the restatement in oracle/ for convolution (bits/nnconv.cu:225-312 + impl/im2row_cpu.cpp:52-230
    with a threaded sgemm; kind "port").  About 2 s each; configs[4] on 4 of its 64 images, scaled per image."""
    from oracle import binding as ob
    have_ref = ob.ref() is not None
    blas = ob.use_openblas(True)
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    gemm = "OpenBLAS (numpy wheel), threaded" if blas else "built-in OpenMP kernel"
    legs = []
    # configs[0]
    w = workloads.conv_single()
    g = ob.conv_geom(w["x"].shape, w["f"].shape, w["stride"], w["pad"], w["dilate"])
    flops = 2.0 * 32 * 32 * 100 * 75 * 32
    t, n = _cpu_time(lambda: ob.conv_forward(w["x"], w["f"], w["b"], g), 1.0)
    legs.append(dict(config="configs[0] conv forward", ms=t * 1e3, tflops=flops / t / 1e12, cores=cores, kind="port", sample="%d full passes; sgemm = %s" % (n, gemm)))
    t, n = _cpu_time(lambda: ob.conv_backward(w["x"], w["f"], w["dy"], g), 1.5)
    legs.append(dict(config="configs[0] conv backward (dzdx, dzdf, dzdb)", ms=t * 1e3, tflops=2 * flops / t / 1e12, cores=cores, kind="port",
                     sample="%d full passes; sgemm = %s" % (n, gemm)))
    # configs[4] on a few images
    Nc = 4
    r = np.random.default_rng(7)
    x = np.asfortranarray(r.standard_normal((56, 56, 256, Nc), dtype=np.float32))
    dy = np.asfortranarray(r.standard_normal((56, 56, 256, Nc), dtype=np.float32))
    f = workloads.he_normal(r, (3, 3, 256, 256))
    g = ob.conv_geom(x.shape, f.shape, 1, 1, 1)
    flops = 2.0 * 56 * 56 * 9 * 256 * 256 * Nc
    t, n = _cpu_time(lambda: ob.conv_backward(x, f, dy, g), 2.5)
    legs.append(dict(config="configs[4] conv backward (dzdx, dzdf, dzdb)", ms_per_image=t / Nc * 1e3, ms_at_64_images=t / Nc * 64 * 1e3,
                     tflops=2 * flops / t / 1e12, cores=cores, kind="port",
                     sample="%d passes over %d of the 64 images (the reference loops over images: time scales with their number); sgemm = %s" % (n, Nc, gemm)))
    ob.use_openblas(False)
    # configs[1]
    w = workloads.bnorm_case()
    E = float(w["x"].nbytes)
    if have_ref:
        fn, kind = (lambda: ob.ref_bnorm_backward(w["x"], w["g"], w["b"], w["dy"], w["eps"])), "reference"
    else:
        fn, kind = (lambda: ob.bnorm_backward(w["x"], w["g"], w["dy"], w["eps"])), "port"
    t, n = _cpu_time(fn, 2.0)
    legs.append(dict(config="configs[1] bnorm backward", ms=t * 1e3, gbs=5 * E / t / 1e9, gbs_compulsory=3 * E / t / 1e9, cores=1, kind=kind,
                     sample="%d full passes, 56x56x256x32" % n))
    # configs[2]
    for label, w in (("configs[2]a max-pool backward", workloads.pool_max_case()), ("configs[2]b avg-pool backward", workloads.pool_avg_case())):
        g = ob.pool_geom(w["x"].shape, w["pool"], w["stride"], w["pad"], w["method"])
        nbytes = (2.0 if w["method"] == "max" else 1.0) * w["x"].nbytes + w["dy"].nbytes
        if have_ref:
            fn, kind = (lambda: ob.ref_pool_backward(w["x"], w["dy"], g)), "reference"
        else:
            fn, kind = (lambda: ob.pool_backward(w["x"], w["dy"], g)), "port"
        t, n = _cpu_time(fn, 2.0)
        legs.append(dict(config=label, ms=t * 1e3, gbs=nbytes / t / 1e9, cores=1, kind=kind,
                         sample="%d full passes, %s" % (n, "x".join(map(str, w["x"].shape)))))
    return legs


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.stderr.write("bench.py measures one GPU: this hot path does not shard in this build (run with --gpus 1)\n")
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        sys.stderr.write("bench.py needs a GPU\n")
        sys.exit(2)
    from matconvnet_amd import capi, vlapi, workloads
    capi.lib()
    vlapi.lib()

    images_per_s, ms_per_step, roof, breakdown, block_plain = bench_block(vlapi, capi, workloads, args.steps, args.warmup)
    block_two_streams = block_plain.pop("timed_schedule_on_two_streams")
    conv_rows, conv_whole = bench_conv_bwd(capi, workloads, max(5, args.steps // 5))
    bn_rows, bn_whole = bench_bnorm_bwd(capi, workloads, args.steps)
    pool_rows = bench_pool_bwd(capi, workloads, args.steps)
    ceiling = bench_hbm_ceiling(capi, max(8, args.steps // 2))
    mfma_ceiling = bench_mfma_ceiling(capi, 5)
    forward_rows = bench_forward(capi, max(5, args.steps // 2))
    single_rows, single_whole = bench_conv_single(capi, workloads, args.steps)
    for row in bn_rows + pool_rows + forward_rows:
        if row["bound"] == "hbm":   # beside the fraction of the nominal 8 TB/s: of what a plain copy reaches here
            row["frac_of_measured_copy"] = row["achieved"] / ceiling["copy"]["gbs"]
    pool_rows[0]["frac_of_measured_copy_of_same_size"] = pool_rows[0]["achieved"] / ceiling["copy_231MB"]["gbs"]
    for row in conv_rows + forward_rows:
        if row["bound"] == "mfma":  # beside the fraction of the nominal 157.3 TFLOP/s: of what the matrix pipe reaches alone
            row["frac_of_measured_mfma"] = row["achieved"] / mfma_ceiling["fp32"]["tflops"]
    roof["frac_of_measured_mfma"] = roof["achieved"] / mfma_ceiling["fp32"]["tflops"]
    graded = conv_rows + bn_rows + pool_rows
    # the per-operator figures once more inside `roofline`, in short form (fraction of the nominal roof, achieved, mean
    # launch time): records that keep `roofline` whole and only the names of the other keys still carry them
    roof["per_operator"] = {r["op"]: dict(frac=r["frac"], achieved=r["achieved"], unit=r["unit"], us=r["avg_launch_us"])
                            for r in graded}
    roof["per_operator"]["conv backward, all launches"] = dict(frac=conv_whole["frac"], achieved=conv_whole["tflops"],
                                                              unit="TFLOP/s", us=conv_whole["ms"] * 1e3)
    roof["per_operator"]["bnorm backward, both passes"] = dict(frac=bn_whole["frac"], achieved=bn_whole["gbs"], unit="GB/s",
                                                              us=bn_whole["us"], frac_compulsory_bytes=bn_whole["gbs_compulsory"] * 1e9 / PEAK_HBM)
    roof["per_operator"]["copy of the max-pool's 231 MB"] = dict(frac=ceiling["copy_231MB"]["frac_of_peak"], achieved=ceiling["copy_231MB"]["gbs"],
                                                                unit="GB/s", us=ceiling["copy_231MB"]["us"])
    line = {
        "metric": "ResNet-50-block fwd+bwd images/s; conv-bwd TFLOP/s; bnorm/pool-bwd GB/s",
        "value": images_per_s, "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "BASELINE configs[3]: ResNet-50 bottleneck fwd+bwd, 56x56, 256->64->64->256, N=32, timed schedule "
                               "(vl::nn::Convolution + folded batch-norm entry points; `block_plain`: reference interface only)",
                   "parity": "tests/test_gpu_frontend.py"},
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(workloads)
        per_config = cpu_per_config(workloads)
    # ---- the bulky tables (not graded rows) in the middle of the line
    line.update({
        "step_breakdown_ms": breakdown,
        "hbm_timing": "cold: %d tensor sets in rotation; *_warm: one set reused" % COLD_SETS,
        "forward_rows": forward_rows,
        "latency_rows": single_rows, "conv_single": single_whole,
        "double_rows": bench_double(capi, workloads, max(4, args.steps // 2)),
        # beyond the headline block: the whole network the block comes from, per-image rates of whole training steps
        # (64 is the reference's own sub-batch for this network: batchSize 256 in 4 sub-batches,
        # examples/imagenet/cnn_imagenet_init_resnet.m:170-171)
        "resnet50": [bench_resnet50(vlapi, b, max(3, args.steps // 10), 2) for b in (32, 64, 128)],
        "resnet50_sections_batch32": bench_resnet50_sections(capi, 32, max(3, args.steps // 5)),
    })
    if not args.no_cpu_baseline:
        line["cpu_baseline_per_config"] = per_config
    # ---- the graded per-operator figures last: the end of the line is what a truncating record keeps
    line.update({
        "hbm_ceiling": ceiling,
        "mfma_ceiling": mfma_ceiling,
        "block_plain": block_plain,
        "block_two_streams": block_two_streams,
        "conv_bwd_tflops": conv_whole["tflops"], "conv_bwd_frac_of_mfma_peak": conv_whole["frac"], "conv_bwd_ms": conv_whole["ms"],
        "bnorm_bwd_gbs": bn_whole["gbs"], "bnorm_bwd_frac_of_hbm_peak": bn_whole["frac"], "bnorm_bwd_us": bn_whole["us"],
        "bnorm_bwd_gbs_warm": bn_whole["gbs_warm"], "bnorm_bwd_gbs_compulsory": bn_whole["gbs_compulsory"],
        "bnorm_bwd_frac_of_hbm_peak_compulsory": bn_whole["gbs_compulsory"] * 1e9 / PEAK_HBM,
        "maxpool_bwd_gbs": pool_rows[0]["achieved"], "avgpool_bwd_gbs": pool_rows[1]["achieved"],
        "maxpool_bwd_gbs_warm": pool_rows[0]["achieved_warm"], "avgpool_bwd_gbs_warm": pool_rows[1]["achieved_warm"],
        "rooflines": graded,
    })
    line = _sig(line)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
