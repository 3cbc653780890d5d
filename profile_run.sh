#!/bin/bash
# Collect the rocprofv3 evidence for one benchmark configuration and condense it.
#   bash profile_run.sh <config id> <output summary file> [extra bench.py args]
# (extra args "--op quantize" etc. profile an operator beside the lookup; the config id is then unused)
# Runs from the repository root on a machine with the GPU. One rocprofv3 run per
# counter group (the hardware cannot collect them together); raw CSVs go to /tmp.
set -o pipefail
CFG=${1:-3}; OUT=${2:-profile_summary.txt}; shift; shift
export TMPDIR=/tmp
RAW=$(mktemp -d /tmp/fbgemm_amd_prof.XXXXXX)
mkdir -p "$(dirname "$OUT")"
# The counter passes run a handful of forwards, too few for the library to settle which lean kernel a
# forward of wide 4-bit bags takes (it times both first): they are told to take the one the kernel trace
# above shows for the steady state (PMC_EXTRA, "--wide4 on" for config 5).
PMC_EXTRA=${PMC_EXTRA:-}
case "$CFG $*" in "5 "*|"5") [ -z "$PMC_EXTRA" ] && PMC_EXTRA="--wide4 on";; esac
BENCH="python3 bench.py --config $CFG --no-cpu --no-also --one-mode --no-check --calibration-copy-mib 1024 $*"
{
  echo "# rocprofv3 summary, bench.py --config $CFG $*"
  echo "# commands (each its own run):"
  echo "#   rocprofv3 --kernel-trace --stats --output-format csv -d <dir> -o t -- $BENCH --steps 20 --warmup 3"
  echo "#   rocprofv3 --pmc <counters> --output-format csv -d <dir> -o p -- $BENCH --clock-warmup-s 0 $PMC_EXTRA --steps 3 --warmup 1"
  echo "# condensed with: python3 profile_summary.py <dir>"
} > "$OUT"
case "$*" in
  *--op*) echo "== kernel trace (--kernel-trace --stats)" >> "$OUT";;
  *) echo "== kernel trace (--kernel-trace --stats): 0.3 s of forwards to bring the clocks up, 3 warm-up forwards, 20 timed, 20 more without the scheduler" >> "$OUT";;
esac
echo "pass: kernel trace ($(date +%T))"
timeout -k 10 900 rocprofv3 --kernel-trace --stats --output-format csv -d $RAW/trace -o t -- $BENCH --steps 20 --warmup 3 > $RAW/trace.log 2>&1 || { echo "trace run failed" | tee -a "$OUT"; tail -5 $RAW/trace.log; exit 1; }
grep '^{' $RAW/trace.log | tail -1 | cut -c1-3000 >> "$OUT"
python3 profile_summary.py $RAW/trace | grep -v '^#' >> "$OUT"
# PROFILE_SHORT=1 keeps the byte counters only (for workloads whose set-up takes minutes);
# PROFILE_PASSES="A B;C" names the passes (counters of a pass separated by blanks, passes by semicolons)
if [ -n "$PROFILE_PASSES" ]; then
  IFS=';' read -r -a PASSES <<< "$PROFILE_PASSES"
elif [ -n "$PROFILE_SHORT" ]; then
  PASSES=("FETCH_SIZE" "WRITE_SIZE" "TCC_HIT_sum TCC_MISS_sum" "GRBM_GUI_ACTIVE")
else
  PASSES=("FETCH_SIZE" "WRITE_SIZE" "TCC_HIT_sum TCC_MISS_sum" "TCC_EA0_RDREQ_sum"
          "SQ_WAVES SQ_INSTS_VALU SQ_INSTS_VMEM_RD SQ_INSTS_LDS SQ_INSTS_SALU SQ_WAVE_CYCLES SQ_WAIT_INST_ANY SQ_ACTIVE_INST_VALU"
          "TCP_TCC_READ_REQ_sum TCP_TOTAL_CACHE_ACCESSES_sum TCP_TCC_READ_REQ_LATENCY_sum TCP_PENDING_STALL_CYCLES_sum"
          "TCP_UTCL1_REQUEST_sum TCP_UTCL1_TRANSLATION_MISS_sum TCP_UTCL1_TRANSLATION_HIT_sum" "GRBM_GUI_ACTIVE")
fi
for pass in "${PASSES[@]}"; do
  n=$(echo $pass | tr ' ' '_' | cut -c1-40)
  echo "pass: $pass ($(date +%T))"
  echo "== --pmc $pass" >> "$OUT"
  timeout -s KILL 600 rocprofv3 --pmc $pass --output-format csv -d $RAW/pmc_$n -o p -- $BENCH --clock-warmup-s 0 $PMC_EXTRA --steps 3 --warmup 1 > $RAW/pmc_$n.log 2>&1 || { echo "pass failed: $pass" >> "$OUT"; tail -3 $RAW/pmc_$n.log >> "$OUT"; exit 1; }
  python3 profile_summary.py $RAW/pmc_$n | grep -v '^#\|^launch' >> "$OUT"
done
[ -d $RAW/pmc_GRBM_GUI_ACTIVE ] && python3 profile_summary.py $RAW/pmc_GRBM_GUI_ACTIVE | grep '^launch' >> "$OUT"
rm -rf $RAW
echo "summary written to $OUT"
