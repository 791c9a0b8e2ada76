#!/bin/bash
# Collects the rocprofv3 evidence for the library's kernels on the benchmark configurations (run from the repo
# root on a GPU box).  Per workload of bench.py (`--profile-leg`: exactly K steps of it and nothing else): a
# kernel trace with statistics at settled clocks, then hardware counters in separate runs (one counter group
# per run, no spin-up, so that a run holds exactly K steps), then the same HBM counters on a plain copy of
# known size for scaling, then a kernel trace of the model-level run.  Raw output goes to the directory given
# as the first argument; profile_summary.py turns it into the tables kept under profiles/.
#   usage: ./profile_counters.sh <output directory> [workloads, default: all]
set -e
R=$(cd "$(dirname "$0")" && pwd)
[ -n "$1" ] || { echo "usage: $0 <output directory> [headline pop_fused pop_two_op long layer5 layer_ops model]" >&2; exit 2; }
mkdir -p "$1"
O=$(cd "$1" && pwd)
shift
LEGS=${*:-headline pop_fused pop_two_op long layer5 layer_ops model}
STEPS=8
cd /tmp && export TMPDIR=/tmp
run() { name=$1; shift; echo "[profile] $name" ; timeout -s KILL 150 rocprofv3 "$@" --output-format csv -d "$O/$name" -o r -- $CMD > "$O/$name.log" 2>&1; }
for leg in $LEGS; do
  if [ "$leg" = model ]; then
    # the model-level step of benchmark configuration 5 (12-layer harness around the ops): which kernels its time goes to
    CMD="python3 $R/bench.py --steps 10 --warmup 2 --spin-up 0 --no-cpu --no-pop --no-long --no-layer5 --no-layer"
    run trace_model --kernel-trace --stats
    rm -f "$O/trace_model/r_kernel_trace.csv"   # tens of MB, one line per launch; the per-kernel statistics beside it are what is summarised
    continue
  fi
  CMD="python3 $R/bench.py --profile-leg $leg --steps $STEPS --spin-up 0.3"
  run trace_$leg --kernel-trace --stats
  rm -f "$O/trace_$leg/r_kernel_trace.csv"
  CMD="python3 $R/bench.py --profile-leg $leg --steps $STEPS --spin-up 0"
  run fetch_$leg --pmc FETCH_SIZE
  run write_$leg --pmc WRITE_SIZE
  run sq1_$leg --pmc SQ_WAVES SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_INSTS_VALU SQ_INSTS_MFMA SQ_INSTS_LDS SQ_INSTS_SALU SQ_WAIT_INST_LDS
  run sq2_$leg --pmc SQ_ACTIVE_INST_VALU SQ_ACTIVE_INST_LDS SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_WAIT_INST_ANY SQ_WAIT_ANY SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_VALU_MFMA_MOPS_BF16
done
CMD="python3 $R/bench.py --copy-calibration"
run copy_fetch --pmc FETCH_SIZE
run copy_write --pmc WRITE_SIZE
echo "done: $O"
