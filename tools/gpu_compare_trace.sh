#!/bin/bash
# tools/gpu_compare_trace.sh — rocprofv3 --kernel-trace --stats of `bench.py --compare-designs` for one design at a time, so that
# the per-kernel tables of two designs at equal sizes can be read side by side.
#   DESIGNS="lorulix kekapel" (default), SIZE=small|medium|wide (default small). Output: gpurun_out/trace_<design>_<size>.md
mkdir -p gpurun_out
REPO=$(pwd)
export TMPDIR=/tmp
cd /tmp
for d in ${DESIGNS:-lorulix kekapel}; do
  rm -rf $REPO/gpurun_out/prof_$d
  timeout -k 10 400 rocprofv3 --kernel-trace --stats -d $REPO/gpurun_out/prof_$d -o bench -- python3 $REPO/bench.py --compare-designs --compare $d --compare-sizes ${SIZE:-small} > $REPO/gpurun_out/trace_$d.log 2>&1 || exit 1
  echo "== $d rocprof rc=$?"; tail -1 $REPO/gpurun_out/trace_$d.log | cut -c1-300
  DB=$(find $REPO/gpurun_out/prof_$d -name "*.db" | head -1)
  python3 $REPO/tools/rocpd_stats.py $DB 40 > $REPO/gpurun_out/trace_${d}_${SIZE:-small}.md 2>&1; cat $REPO/gpurun_out/trace_${d}_${SIZE:-small}.md
  rm -rf $REPO/gpurun_out/prof_$d
done
