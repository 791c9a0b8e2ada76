#!/bin/bash
# Collects the rocprofv3 evidence for the pass kernels on benchmark configurations 2 and 4 (run from the repo
# root on a GPU box): kernel-trace statistics, then hardware counters in separate passes (one
# counter group per run), then the same HBM counters on a plain copy of known size for scaling.
# Raw output goes to the directory given as the first argument; flash-pop_amd/profile_summary.py turns
# it into the tables kept under profiles/.
#   usage: flash-pop_amd/profile_counters.sh <output directory>
set -e
R=$(cd "$(dirname "$0")/.." && pwd)
[ -n "$1" ] || { echo "usage: $0 <output directory>" >&2; exit 2; }
mkdir -p "$1"
O=$(cd "$1" && pwd)
cd /tmp && export TMPDIR=/tmp
# the trace run keeps bench.py's spin-up so that its durations are those of settled clocks; the counter runs skip it
TRACE="python3 $R/bench.py --steps 8 --warmup 4 --no-cpu --no-long --no-model"
BENCH="python3 $R/bench.py --steps 8 --warmup 4 --spin-up 0 --no-cpu --no-long --no-model"
COPY="python3 $R/bench.py --copy-calibration"
run() { name=$1; shift; timeout -s KILL 120 rocprofv3 "$@" --output-format csv -d "$O/$name" -o r -- $CMD > "$O/$name.log" 2>&1; }
CMD=$TRACE run trace --kernel-trace --stats
CMD=$BENCH run sq1 --pmc SQ_WAVES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_INSTS_VALU SQ_INSTS_MFMA SQ_INSTS_LDS SQ_INSTS_SALU SQ_WAIT_INST_LDS
CMD=$BENCH run sq2 --pmc SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_LDS SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_WAIT_INST_ANY SQ_WAIT_ANY SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_VALU_MFMA_MOPS_BF16
CMD=$BENCH run fetch --pmc FETCH_SIZE
CMD=$BENCH run write --pmc WRITE_SIZE
CMD=$COPY run copy_fetch --pmc FETCH_SIZE
CMD=$COPY run copy_write --pmc WRITE_SIZE
# long context, few streams (benchmark configuration 3): the split-sequence passes
LONG="python3 $R/bench.py --steps 8 --warmup 4 --no-cpu --no-pop --no-layer --no-model"
CMD=$LONG run long_trace --kernel-trace --stats
rm -f "$O/long_trace/r_kernel_trace.csv"
# the model-level step of benchmark configuration 5 (12-layer harness around the ops): which kernels its time goes to
MODEL="python3 $R/bench.py --steps 10 --warmup 2 --spin-up 0 --no-cpu --no-pop --no-long --no-layer"
CMD=$MODEL run model_trace --kernel-trace --stats
rm -f "$O/model_trace/r_kernel_trace.csv"   # tens of MB, one line per launch; the per-kernel statistics beside it are what is summarised
echo "done: $O"
