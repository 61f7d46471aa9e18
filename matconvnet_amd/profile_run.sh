#!/bin/bash
# Collects the rocprofv3 data behind profiles/*.txt and profiles/traffic.json on an MI355X box, from the repository root:
#     bash matconvnet_amd/profile_run.sh [output directory, default prof_out]
# then  python3 -m matconvnet_amd.profile_summary <output directory> profiles
# Kernel traces, FETCH_SIZE, WRITE_SIZE and the matrix-pipe counters each get a run of their own (rocprofv3 does not split
# counters over passes), every run under a time limit.  mcn_bench is built by `python -m matconvnet_amd.build`.
set -e
R=$(pwd)
O=${1:-prof_out}
case "$O" in /*) ;; *) O=$R/$O ;; esac
rm -rf "$O"; mkdir -p "$O"
cd /tmp && export TMPDIR=/tmp && cd "$R"
B=./matconvnet_amd/mcn_bench
timeout -k 10 600 rocprofv3 --kernel-trace --stats -d "$O/bench" -o bench -- python3 bench.py --steps 20 --warmup 5 --no-cpu-baseline > "$O/bench_stdout.txt" 2> "$O/bench_stderr.txt"
echo "done bench"
for k in copy bnorm maxpool avgpool conv5 blocktimed; do
  timeout -s KILL 90 rocprofv3 --kernel-trace --stats -d "$O/kt_$k" -o kt -- $B --only $k --iters 12 --warmup 4 > "$O/kt_$k.txt" 2>&1
  timeout -s KILL 90 rocprofv3 --pmc FETCH_SIZE -d "$O/fetch_$k" -o pmc -- $B --only $k --iters 8 --warmup 4 > "$O/fetch_$k.txt" 2>&1
  timeout -s KILL 90 rocprofv3 --pmc WRITE_SIZE -d "$O/write_$k" -o pmc -- $B --only $k --iters 8 --warmup 4 > "$O/write_$k.txt" 2>&1
  echo "done $k"
done
for k in conv1 stem; do
  timeout -s KILL 90 rocprofv3 --kernel-trace --stats -d "$O/kt_$k" -o kt -- $B --only $k --iters 12 --warmup 4 > "$O/kt_$k.txt" 2>&1
  echo "done $k"
done
timeout -s KILL 90 rocprofv3 --kernel-trace --stats -d "$O/kt_block" -o kt -- $B --only block --iters 12 --warmup 4 > "$O/kt_block.txt" 2>&1
for k in conv5 blocktimed; do
  timeout -s KILL 90 rocprofv3 --pmc SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_INSTS_VALU SQ_INSTS_LDS SQ_ACTIVE_INST_LDS GRBM_GUI_ACTIVE -d "$O/sq_$k" -o pmc -- $B --only $k --iters 6 --warmup 3 > "$O/sq_$k.txt" 2>&1
  echo "done counters $k"
done
timeout -s KILL 150 rocprofv3 --kernel-trace --stats -d "$O/kt_resnet50" -o kt -- $B --only resnet50 --batch 32 --iters 6 --warmup 2 > "$O/kt_resnet50.txt" 2>&1
timeout -s KILL 150 $B --only resnet50 --batch 32 --iters 6 --warmup 2 --two-streams > "$O/resnet50_two_streams.txt" 2>&1
echo "done resnet50"
timeout -s KILL 300 $B --only yardstick --iters 8 --warmup 2 > "$O/yardstick.txt" 2>&1
echo "done yardstick"
du -sh "$O"
