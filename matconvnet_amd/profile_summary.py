"""Turns the rocprofv3 output of matconvnet_amd/profile_run.sh into the short summaries under profiles/ and into
profiles/traffic.json (HBM bytes per launch of the kernels bench.py reports, which it cannot read from inside its own
process):

    python3 -m matconvnet_amd.profile_summary <profile_run.sh output directory> <destination, e.g. profiles>

FETCH_SIZE and WRITE_SIZE are scaled by what they read for the 256 MiB streaming copy of `mcn_bench --only copy`, whose
traffic is known (the factors are written into every summary and into traffic.json)."""
import glob
import json
import os
import re
import sqlite3
import sys

PRE = "cd /tmp && export TMPDIR=/tmp   (then, from the repository root on the MI355X box:)\n"
COPY_BYTES = 268435456.0  # mcn_bench --only copy reads and writes this much per launch


def short(name):
    name = re.sub(r"^void ", "", name).replace("mcn::(anonymous namespace)::", "")
    return name.split("(")[0][:90]


def _db(path):
    hits = glob.glob(os.path.join(path, "**", "*_results.db"), recursive=True)
    if not hits:
        raise SystemExit("no rocprofv3 database under " + path)
    return sqlite3.connect(hits[0]).cursor()


def durations(path):
    c = _db(path)
    rows = list(c.execute("select name, count(*), sum(end-start), avg(end-start), min(end-start), max(end-start) from kernels "
                          "group by name order by sum(end-start) desc"))
    total = sum(r[2] for r in rows) or 1
    out = ["%-90s %6s %10s %10s %10s %10s %6s" % ("kernel", "calls", "total ms", "avg us", "min us", "max us", "%")]
    for n, calls, t, avg, mn, mx in rows:
        out.append("%-90s %6d %10.3f %10.2f %10.2f %10.2f %6.1f" % (short(n), calls, t / 1e6, avg / 1e3, mn / 1e3, mx / 1e3, 100 * t / total))
    return out


def counters(path):
    """{kernel: {counter: (n, avg, min, max)}}"""
    c = _db(path)
    out = {}
    for name, counter, n, avg, mn, mx in c.execute("select kernel_name, counter_name, count(*), avg(value), min(value), max(value) "
                                                   "from counters_collection group by kernel_name, counter_name"):
        out.setdefault(short(name), {})[counter] = (n, avg, mn, mx)
    return out


def counter_table(table, keep=None):
    out = ["%-90s %-26s %4s %14s %14s %14s" % ("kernel", "counter", "n", "avg", "min", "max")]
    rows = [(k, cn, v) for k, d in table.items() for cn, v in d.items() if keep is None or keep(k)]
    for k, cn, (n, avg, mn, mx) in sorted(rows, key=lambda r: -r[2][1]):
        out.append("%-90s %-26s %4d %14.1f %14.1f %14.1f" % (k, cn, n, avg, mn, mx))
    return out


def program_output(path):
    return "".join(l for l in open(path) if not l.startswith(("W2", "E2", "I2")) and "rocprof" not in l)


def main(src, dst):
    os.makedirs(dst, exist_ok=True)

    def write(name, text):
        with open(os.path.join(dst, name), "w") as f:
            f.write(text)
        print(name, len(text))

    # ---- calibration: the copy of known size
    copy_fetch = [v["FETCH_SIZE"][1] for k, v in counters(src + "/fetch_copy").items() if "eltwise" in k or "relu" in k][0]
    copy_write = [v["WRITE_SIZE"][1] for k, v in counters(src + "/write_copy").items() if "eltwise" in k or "relu" in k][0]
    fetch_unit, write_unit = COPY_BYTES / copy_fetch, COPY_BYTES / copy_write
    calib_f = "FETCH_SIZE per dispatch (counter units; the 256 MiB copy reads 262144 KiB and the counter shows %.0f: 1 unit = %.1f bytes):\n" % (copy_fetch, fetch_unit)
    calib_w = "WRITE_SIZE per dispatch (the 256 MiB copy writes 262144 KiB and the counter shows %.0f: 1 unit = %.1f bytes):\n" % (copy_write, write_unit)
    traffic = {"calibration": {"FETCH_SIZE_bytes_per_unit": fetch_unit, "WRITE_SIZE_bytes_per_unit": write_unit,
                               "yardstick": "256 MiB streaming copy (mcn_bench --only copy): FETCH_SIZE reads %.0f, WRITE_SIZE %.0f for 268435456 bytes each"
                                            % (copy_fetch, copy_write)},
               "kernels": {}}

    write("bench_bottleneck_block_kernel_trace.txt",
          "Kernel trace of the default benchmark (ResNet-50 bottleneck fwd+bwd, N=32; then the per-operator configurations).\n"
          "command: " + PRE + "  rocprofv3 --kernel-trace --stats -d " + src + "/bench -o bench -- python3 bench.py --steps 20 --warmup 5 --no-cpu-baseline\n"
          "(all commands of this folder: bash matconvnet_amd/profile_run.sh; summaries: python3 -m matconvnet_amd.profile_summary " + src + " profiles)\n"
          "Durations are per dispatch, from the profiler's kernel table (ns converted to us / ms).\n\n" + "\n".join(durations(src + "/bench")) + "\n")

    names = {"conv5": ("conv_vgg_3x3x256x256_N64_backward", "conv 3x3x256x256 on 56x56x256x64 (BASELINE configs[4]), backward data + filter + bias"),
             "bnorm": ("bnorm_56x56x256x32_backward", "batch-norm backward 56x56x256x32, moments from the batch (BASELINE configs[1])"),
             "maxpool": ("maxpool_112x112x64x32_backward", "max-pool 3x3 s2 p1 backward on 112x112x64x32 (BASELINE configs[2]a)"),
             "avgpool": ("avgpool_56x56x256x32_backward", "avg-pool 2x2 s2 backward on 56x56x256x32 (BASELINE configs[2]b)"),
             "blocktimed": ("bottleneck_block_56x56_N32_fwd_bwd", "ResNet-50 bottleneck block forward+backward, N=32 (BASELINE configs[3]): the schedule bench.py times "
                            "(ReLU / shortcut sum folded into batch normalisation, banks packed by one launch, filter gradients summed by one, channel sums "
                            "from the convolutions, last ReLU mask as bits)"),
             "copy": ("copy_256MiB_counter_yardstick", "plain streaming copy (ReLU of positive data): reads 268435456 B, writes 268435456 B per launch; yardstick for FETCH_SIZE / WRITE_SIZE")}
    # first layers (kernel traces only: latency-sized launches)
    first = "first layers (three input channels): kernel traces of their backward products\n\ncommands: " + PRE
    for k in ("conv1", "stem"):
        first += "  rocprofv3 --kernel-trace --stats -d %s/kt_%s -o kt -- ./matconvnet_amd/mcn_bench --only %s --iters 12 --warmup 4\n" % (src, k, k)
    for k, title in (("conv1", "BASELINE configs[0]: 5x5x3x32 on 32x32x3x100, stride 1, pad 2"),
                     ("stem", "a ResNet stem: 7x7x3x64 on 224x224x3x32, stride 2, pad 3")):
        first += "\n" + title + "\nprogram output under the kernel trace:\n" + program_output("%s/kt_%s.txt" % (src, k)) + "\nkernel durations:\n"
        first += "\n".join(durations("%s/kt_%s" % (src, k))) + "\n"
    write("conv_first_layers_backward.txt", first)

    per_kernel = {}
    for k, (fn, desc) in names.items():
        t = desc + "\n\ncommands: " + PRE
        t += "  rocprofv3 --kernel-trace --stats -d %s/kt_%s -o kt -- ./matconvnet_amd/mcn_bench --only %s --iters 12 --warmup 4\n" % (src, k, k)
        t += "  rocprofv3 --pmc FETCH_SIZE -d %s/fetch_%s -o pmc -- ./matconvnet_amd/mcn_bench --only %s --iters 8 --warmup 4\n" % (src, k, k)
        t += "  rocprofv3 --pmc WRITE_SIZE -d %s/write_%s -o pmc -- ./matconvnet_amd/mcn_bench --only %s --iters 8 --warmup 4\n" % (src, k, k)
        t += ("(mcn_bench is built from matconvnet_amd/bits/mcn_bench.cpp by `python -m matconvnet_amd.build`; the bandwidth-bound\n"
              " operators run COLD: mcn_bench cycles over 4 sets of tensors, --rotate 4 is its default)\n\n")
        t += "program output under the kernel trace:\n" + program_output("%s/kt_%s.txt" % (src, k)) + "\n"
        if k == "blocktimed":
            t += "the other schedules of the same block (mcn_bench --only block, kernel trace):\n" + program_output(src + "/kt_block.txt") + "\n"
        t += "kernel durations:\n" + "\n".join(durations("%s/kt_%s" % (src, k))) + "\n\n"
        f, w = counters("%s/fetch_%s" % (src, k)), counters("%s/write_%s" % (src, k))
        t += calib_f + "\n".join(counter_table(f)) + "\n\n" + calib_w + "\n".join(counter_table(w)) + "\n\n"
        t += "HBM bytes per launch (counter average x bytes per unit):\n"
        for kern in f:
            fb = f[kern]["FETCH_SIZE"][1] * fetch_unit
            wb = w.get(kern, {}).get("WRITE_SIZE", (0, 0.0))[1] * write_unit
            per_kernel[(k, kern)] = (fb, wb, fn + ".txt")
            t += "  %-80s fetch %8.1f MB  write %8.1f MB  total %8.1f MB\n" % (kern, fb / 1e6, wb / 1e6, (fb + wb) / 1e6)
        write(fn + ".txt", t)

    def total(run, prefix):
        hits = [(v[0] + v[1], v[2]) for (r, kern), v in per_kernel.items() if r == run and kern.startswith(prefix)]
        return hits

    def put(key, run, prefix, note=None, mean=False):
        hits = total(run, prefix)
        if not hits:
            return
        val = sum(h[0] for h in hits) / (len(hits) if mean else 1)
        traffic["kernels"][key] = {"bytes": val, "source": "profiles/" + hits[0][1]}
        if note:
            traffic["kernels"][key]["note"] = note

    # the weights-stationary kernel's launches of a step differ (six launches, several instantiations): weighted mean
    c = _db(src + "/fetch_blocktimed")
    rows = list(c.execute("select kernel_name, value from counters_collection where counter_name='FETCH_SIZE'"))
    cw = _db(src + "/write_blocktimed")
    rows_w = list(cw.execute("select kernel_name, value from counters_collection where counter_name='WRITE_SIZE'"))
    ws_f = [v for n, v in rows if short(n).startswith("conv_ws_mfma")]
    ws_w = [v for n, v in rows_w if short(n).startswith("conv_ws_mfma")]
    if ws_f and ws_w:
        traffic["kernels"]["block/conv_ws_mfma"] = {"bytes": sum(ws_f) / len(ws_f) * fetch_unit + sum(ws_w) / len(ws_w) * write_unit,
                                                    "source": "profiles/bottleneck_block_56x56_N32_fwd_bwd.txt",
                                                    "note": "mean over the six launches of a step"}
    put("cfg5/conv_sb_mfma", "conv5", ("conv_sb_mfma", "conv_sb_tail_reduce"), note="the product's launches together")
    put("cfg5/conv_pix_mfma", "conv5", "conv_pix_mfma")
    put("cfg5/conv_wgrad_mfma", "conv5", "conv_wgrad_mfma")
    put("cfg2/bnorm_sums", "bnorm", "bnorm_sums")
    put("cfg2/bnorm_backward_apply", "bnorm", "bnorm_backward_apply")
    put("cfg3a/pool", "maxpool", "pool_max_backward_stream")
    put("cfg3b/pool", "avgpool", "pool_backward_avg_tiles")
    with open(os.path.join(dst, "traffic.json"), "w") as f:
        json.dump(traffic, f, indent=1, sort_keys=True)
        f.write("\n")
    print("traffic.json", len(traffic["kernels"]))

    # ---- matrix-pipe counters
    t = ("Matrix-core utilisation counters of the convolution kernels (rocprofv3 --pmc, one pass).\n\ncommands: " + PRE)
    for k in ("conv5", "blocktimed"):
        t += ("  rocprofv3 --pmc SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_INSTS_VALU SQ_INSTS_LDS SQ_ACTIVE_INST_LDS "
              "GRBM_GUI_ACTIVE -d %s/sq_%s -o pmc -- ./matconvnet_amd/mcn_bench --only %s --iters 6 --warmup 3\n" % (src, k, k))
    t += ("\nReading: SQ_INSTS_MFMA counts v_mfma_f32_32x32x2_f32 instructions (4096 FLOP each); SQ_VALU_MFMA_BUSY_CYCLES is 64 cycles per\n"
          "such instruction, summed over the 1024 SIMDs; GRBM_GUI_ACTIVE is summed over the 8 XCDs.  Matrix-core utilisation of a launch =\n"
          "SQ_VALU_MFMA_BUSY_CYCLES / (1024 * GRBM_GUI_ACTIVE / 8).  (Durations under --pmc are longer than in the kernel trace: the counters\n"
          "serialise dispatches.)  VALU per MFMA = SQ_INSTS_VALU / SQ_INSTS_MFMA - 1 (the counter of vector instructions includes the MFMAs).\n")
    for k, title in (("conv5", "conv 3x3x256x256 on 56x56x256x64, backward"), ("blocktimed", "ResNet-50 bottleneck block, N=32, forward + backward (timed schedule)")):
        table = counters("%s/sq_%s" % (src, k))
        is_mfma = lambda kern: kern.startswith(("conv_pix_mfma", "conv_wgrad_mfma", "conv_ws_mfma", "conv_sb_mfma"))
        t += "\n%s:\n" % title + "\n".join(counter_table(table, is_mfma)) + "\n"
        for kern, d in table.items():
            if is_mfma(kern) and "SQ_VALU_MFMA_BUSY_CYCLES" in d and d.get("GRBM_GUI_ACTIVE", (0, 0))[1]:
                util = d["SQ_VALU_MFMA_BUSY_CYCLES"][1] / (1024 * d["GRBM_GUI_ACTIVE"][1] / 8)
                extra = ""
                if "SQ_INSTS_VALU" in d and d.get("SQ_INSTS_MFMA", (0, 0))[1]:
                    extra = "   vector instructions per MFMA %.2f" % (d["SQ_INSTS_VALU"][1] / d["SQ_INSTS_MFMA"][1])
                t += "  utilisation %-60s %.3f%s\n" % (kern, util, extra)
    write("conv_mfma_utilisation_counters.txt", t)

    # ---- whole network
    t = ("Whole ResNet-50 (224x224x3, 1000 classes, 32 images): kernel trace of forward, forward + backward and whole training steps, layer by\n"
         "layer and with ReLU / shortcut sums folded into batch normalisation.\n\ncommand: " + PRE +
         "  rocprofv3 --kernel-trace --stats -d " + src + "/kt_resnet50 -o kt -- ./matconvnet_amd/mcn_bench --only resnet50 --batch 32 --iters 6 --warmup 2\n\n"
         "program output under the trace:\n" + program_output(src + "/kt_resnet50.txt") +
         "the same program untraced with the units' filter gradients on a second stream (./matconvnet_amd/mcn_bench --only resnet50 --batch 32\n"
         " --iters 6 --warmup 2 --two-streams):\n" + program_output(src + "/resnet50_two_streams.txt") +
         "(the replays from HIP graphs at the end of each line are slowed by the tracer, which serialises the nodes of a graph; untraced they take\n"
         " the same time as the eager calls)\n\nall launches of the run:\n" + "\n".join(durations(src + "/kt_resnet50")) + "\n")
    write("resnet50_224x224_N32_training_step.txt", t)

    # ---- the swept yardstick
    lines = [l for l in open(src + "/yardstick.txt") if l.startswith(("device", "read", "write", "copy", "best"))]
    ranked = {}
    for l in lines:
        m = re.search(r"(\d+) GB/s", l)
        if m and not l.startswith("best") and not l.startswith("device"):
            ranked.setdefault(l.split()[0], []).append((int(m.group(1)), l))
    t = ("Sweep of plain streaming kernels (read-only, write-only, copy; 256 MiB per stream, cold: 4 buffer sets in turn) over launch shape:\n"
         "access width, workgroups per compute unit (0 = one step per workgroup, not persistent), accesses in flight per lane, walk (slab by slab\n"
         "over the whole chip, or one contiguous run per workgroup), store hint.  The best line of each mode is the measured ceiling the\n"
         "bandwidth-bound operators are reported against beside the nominal 8 TB/s.\n\ncommand: " + PRE +
         "  ./matconvnet_amd/mcn_bench --only yardstick --iters 8 --warmup 2\n(%d configurations; the ten best of each mode, then the best)\n\n" % (len(lines) - 4))
    for mode in ("read", "write", "copy"):
        for _, l in sorted(ranked.get(mode, []), key=lambda r: -r[0])[:10]:
            t += l
        t += "\n"
    t += "".join(l for l in lines if l.startswith("best"))
    write("hbm_yardstick_sweep.txt", t)


if __name__ == "__main__":
    if len(sys.argv) != 3:
        raise SystemExit(__doc__)
    main(sys.argv[1].rstrip("/"), sys.argv[2])
