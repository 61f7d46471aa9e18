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
  cpu_baseline  the CPU restatement of the reference path (oracle/) timed on this machine's host cores.
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
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/*.txt), scaled by what the same counters
# read for a 256 MiB streaming copy (FETCH_SIZE: 2 KiB per unit, WRITE_SIZE: 1 KiB per unit).  Counters are not
# readable from inside this process, so these are the profiled values of exactly these launches.
TRAFFIC = {
    "block/conv_ws_mfma": 1.161e8,     # mean of the 6 launches of a step (profiles/bottleneck_block_56x56_N32_fwd_bwd.txt; operands 1.028e8)
    "cfg5/conv_pix_mfma": 5.579e8,     # profiles/conv_vgg_3x3x256x256_N64_backward.txt (operands 4.13e8: dzdy in, dzdx out, bank)
    "cfg5/conv_wgrad_mfma": 9.06e8,    # (operands 4.13e8: x and dzdy are both re-read by the filter-volume tiles)
    "cfg2/bnorm_sums": 2.058e8,        # profiles/bnorm_56x56x256x32_backward.txt
    "cfg2/bnorm_backward_apply": 3.086e8,
    "cfg3a/pool": 2.518e8,             # profiles/maxpool_112x112x64x32_backward.txt (halo columns fetched by two workgroups)
    "cfg3b/pool": 1.286e8,             # profiles/avgpool_56x56x256x32_backward.txt
}
COLD_SETS = 4              # tensor sets used in turn by the HBM-bound measurements (> 256 MB between reuses)


def _sync():
    import torch
    torch.cuda.synchronize()


def kernel_time(capi, kernel, launch, reps):
    """Mean duration (s) of `kernel` over `reps` calls of `launch`, from HIP events bracketing each launch."""
    capi.profile_begin(kernel)
    for _ in range(reps):
        launch()
    n, ms = capi.profile_end()
    return (ms / n) * 1e-3 if n else float("nan"), n


def bench_block(vlapi, capi, workloads, steps, warmup):
    w = workloads.bottleneck_case()
    N = w["x"].shape[3]
    # fused: ReLU / shortcut sum folded into batch normalisation; packed: the filter banks are re-laid for the matrix
    # kernels by ONE launch at the start of every step (as after an update of the filters) instead of one per product
    # deferred: the sums over reduction splits that finish the three filter gradients run in one launch at the end
    blk = vlapi.Bottleneck(N=N, eps=w["eps"], fused=True, packed=True, deferred=True)
    for k in ("x", "f1", "f2", "f3", "g1", "b1", "g2", "b2", "g3", "b3"):
        blk.set(k, w[k])
    blk.set("dzdy", w["dy"])
    blk.run(warmup)
    _sync()
    t0 = time.perf_counter()
    blk.run(steps)
    _sync()
    dt = time.perf_counter() - t0
    # which kernel family dominates the step, and its live duration
    P = 56 * 56
    # per launch family per step.  The six forward + backward-data launches go to the weights-stationary kernel
    # (conv_ws_mfma) when the bank fits in LDS, else to the tiled one (conv_pix_mfma); if a step ever mixes them,
    # they are reported as one family.
    pix_flops = 2.0 * (2.0 * P * N * (256 * 64 + 9 * 64 * 64 + 64 * 256))
    conv_flops = {"conv_wgrad_mfma": 2.0 * P * N * (256 * 64 + 9 * 64 * 64 + 64 * 256)}
    eS, eB = 4.0 * P * 64 * N, 4.0 * P * 256 * N
    hbm_bytes = {  # algorithmic bytes per step of the memory-bound families (reads + writes once each)
        # forward reads x; backward reads x and dzdy; bn3's backward also reads the block output (mask) and writes
        # the masked derivative
        "bnorm_sums": (eS + eS + eB) + 2 * (eS + eS + eB) + 2 * eB,
        "bnorm_forward_apply": 2 * eS + 2 * eS + 3 * eB,          # bn1, bn2 with ReLU; bn3 with shortcut sum and ReLU
        "bnorm_backward_apply": 3 * (eS + eS + eB),
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
    else:
        work = hbm_bytes.get(top, float("nan"))
        achieved = work * steps / total
        roof = dict(kernel=top, bound="hbm", achieved=achieved / 1e9, peak=PEAK_HBM / 1e9, unit="GB/s",
                    frac=achieved / PEAK_HBM, traffic=TRAFFIC.get("block/" + top), launches_per_step=n // steps, avg_launch_us=total / n * 1e6)
    breakdown = {k: round(v[1] / steps * 1e3, 4) for k, v in fam.items()}  # ms per step by kernel family
    return N * steps / dt, dt / steps * 1e3, roof, breakdown


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
    t_data, _ = kernel_time(capi, "conv_pix_mfma", data, reps)
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
    for name, kern, t in (("conv backward-data", "conv_pix_mfma", t_data), ("conv backward-filter", "conv_wgrad_mfma", t_filt)):
        out.append(dict(op=name, kernel=kern, workload="configs[4] 3x3x256x256 on 56x56x256x64", bound="mfma",
                        achieved=flops / t / 1e12, peak=PEAK_MFMA_FP32 / 1e12, unit="TFLOP/s", frac=flops / t / PEAK_MFMA_FP32,
                        avg_launch_us=t * 1e6, traffic=TRAFFIC["cfg5/" + kern]))
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
             avg_launch_us=t["cold"][0] * 1e6, achieved_warm=2 * E / t["warm"][0] / 1e9, traffic=TRAFFIC["cfg2/bnorm_sums"]),
        dict(op="bnorm backward, pass 2 (apply)", kernel="bnorm_backward_apply", workload="configs[1] 56x56x256x32", bound="hbm",
             achieved=3 * E / t["cold"][1] / 1e9, peak=PEAK_HBM / 1e9, unit="GB/s", frac=3 * E / t["cold"][1] / PEAK_HBM,
             avg_launch_us=t["cold"][1] * 1e6, achieved_warm=3 * E / t["warm"][1] / 1e9, traffic=TRAFFIC["cfg2/bnorm_backward_apply"]),
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
        rows.append(dict(op=name, kernel="pool_max_backward_stream" if method == "max" else "pool_backward_passes",
                         workload="configs[2] %s on %s" % (method, "x".join(map(str, shape))),
                         bound="hbm", achieved=nbytes / t["cold"] / 1e9, peak=PEAK_HBM / 1e9, unit="GB/s",
                         frac=nbytes / t["cold"] / PEAK_HBM, avg_launch_us=t["cold"] * 1e6,
                         achieved_warm=nbytes / t["warm"] / 1e9,
                         traffic=TRAFFIC["cfg3a/pool" if method == "max" else "cfg3b/pool"]))
        del xs, dys, dxs
    return rows


def bench_resnet50(vlapi, batch, steps, warmup):
    """Whole ResNet-50 (224 x 224, 1000 classes; examples/imagenet/cnn_imagenet_init_resnet.m) through the same
    operator classes: forward alone (training-mode batch normalisation), the training step forward + loss derivative
    (softmax log-loss on random labels) + backward + SGD update, and evaluation (stored moments; the mode of the reference's published 396 images/s,
    doc/site/docs/pretrained.md:233, measured there on other hardware), images/s."""
    import torch
    net = vlapi.ResNet50(N=batch, eps=1e-5, image_size=224, classes=1000, fused=True, seed=11)
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
        net.set_test_mode(True)     # evaluation: batch normalisation with the moving averages of the steps above
        eval_ms = timed(net.forward)
        net.set_test_mode(False)
        flops = net.forward_flops_per_image * batch
        return {"batch": batch, "eval_ms": eval_ms, "eval_images_per_s": batch / eval_ms * 1e3,
                "forward_ms": fwd_ms, "forward_images_per_s": batch / fwd_ms * 1e3,
                "train_step_ms": step_ms, "train_images_per_s": batch / step_ms * 1e3,
                "train_conv_tflops": 3 * flops / step_ms / 1e9, "parameters": net.parameters}
    finally:
        net.close()


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

    images_per_s, ms_per_step, roof, breakdown = bench_block(vlapi, capi, workloads, args.steps, args.warmup)
    conv_rows, conv_whole = bench_conv_bwd(capi, workloads, max(5, args.steps // 5))
    bn_rows, bn_whole = bench_bnorm_bwd(capi, workloads, args.steps)
    pool_rows = bench_pool_bwd(capi, workloads, args.steps)
    line = {
        "metric": "ResNet-50-block fwd+bwd images/s; conv-bwd TFLOP/s; bnorm/pool-bwd GB/s",
        "value": images_per_s, "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "BASELINE configs[3]: ResNet-50 bottleneck fwd+bwd, 56x56, 256->64->64->256, N=32, via vl::nn operators"},
        "roofline": roof,
        "step_breakdown_ms": breakdown,
        "conv_bwd_tflops": conv_whole["tflops"], "conv_bwd_frac_of_mfma_peak": conv_whole["frac"], "conv_bwd_ms": conv_whole["ms"],
        "bnorm_bwd_gbs": bn_whole["gbs"], "bnorm_bwd_frac_of_hbm_peak": bn_whole["frac"], "bnorm_bwd_us": bn_whole["us"],
        "bnorm_bwd_gbs_warm": bn_whole["gbs_warm"],
        "maxpool_bwd_gbs": pool_rows[0]["achieved"], "avgpool_bwd_gbs": pool_rows[1]["achieved"],
        "maxpool_bwd_gbs_warm": pool_rows[0]["achieved_warm"], "avgpool_bwd_gbs_warm": pool_rows[1]["achieved_warm"],
        "hbm_timing": "cold: %d tensor sets in rotation; *_warm: one set reused" % COLD_SETS,
        "rooflines": conv_rows + bn_rows + pool_rows,
        # beyond the headline block: the whole network the block comes from, per-image rates of whole training steps
        # (64 is the reference's own sub-batch for this network: batchSize 256 in 4 sub-batches,
        # examples/imagenet/cnn_imagenet_init_resnet.m:170-171)
        "resnet50": [bench_resnet50(vlapi, b, max(3, args.steps // 10), 2) for b in (32, 64, 128)],
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(workloads)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
