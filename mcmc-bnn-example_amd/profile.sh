#!/bin/bash
# Profiles the trajectory kernel on the benchmark workload with rocprofv3 and writes the raw output
# under the directory OUT set below.  Five passes, each its own run: kernel trace + stats, FETCH_SIZE,
# WRITE_SIZE (plus the same two counters on a plain copy kernel of known size for calibration), SQ
# counters, L2 counters.
# Usage: bash mcmc-bnn-example_amd/profile.sh [extra bench.py arguments]
set -e
ROOT="$(cd "$(dirname "$0")/.." && pwd)"
OUT="$ROOT/gpurun_out/${PROFILE_DIR:-profile}"
mkdir -p "$OUT"
BENCH_ARGS="--cpu-seconds 0 $*"
cd /tmp && export TMPDIR=/tmp
echo "== kernel trace + stats"
timeout -s KILL 300 rocprofv3 --kernel-trace --stats -d "$OUT/trace" -o trace --output-format csv -- \
  python3 "$ROOT/bench.py" $BENCH_ARGS > "$OUT/bench_trace.json" 2> "$OUT/trace.log"
for C in FETCH_SIZE WRITE_SIZE; do
  echo "== $C (trajectory kernel)"
  timeout -s KILL 300 rocprofv3 --pmc $C -d "$OUT/pmc_$C" -o pmc --output-format csv -- \
    python3 "$ROOT/bench.py" $BENCH_ARGS > "$OUT/bench_$C.json" 2> "$OUT/pmc_$C.log"
  echo "== $C (copy kernel, 1 GiB each way)"
  timeout -s KILL 120 rocprofv3 --pmc $C -d "$OUT/copy_$C" -o pmc --output-format csv -- \
    "$ROOT/mcmc-bnn-example_amd/copy_calibration" 1024 > "$OUT/copy_$C.txt" 2> "$OUT/copy_$C.log"
done
echo "== SQ counters (trajectory kernel)"
timeout -s KILL 300 rocprofv3 --pmc SQ_BUSY_CYCLES SQ_VALU_MFMA_BUSY_CYCLES SQ_ACTIVE_INST_VALU SQ_INSTS_VALU \
  SQ_INSTS_MFMA SQ_WAIT_INST_ANY SQ_WAVE_CYCLES SQ_ACTIVE_INST_ANY GRBM_GUI_ACTIVE -d "$OUT/pmc_SQ" -o pmc \
  --output-format csv -- python3 "$ROOT/bench.py" $BENCH_ARGS > "$OUT/bench_SQ.json" 2> "$OUT/pmc_SQ.log"
echo "== L2 counters (trajectory kernel)"
timeout -s KILL 300 rocprofv3 --pmc TCC_HIT_sum TCC_MISS_sum TCC_EA0_RDREQ_sum TCC_EA0_RDREQ_DRAM_sum -d "$OUT/pmc_TCC" -o pmc \
  --output-format csv -- python3 "$ROOT/bench.py" $BENCH_ARGS > "$OUT/bench_TCC.json" 2> "$OUT/pmc_TCC.log"
python3 "$ROOT/mcmc-bnn-example_amd/profile_summary.py" "$OUT"
