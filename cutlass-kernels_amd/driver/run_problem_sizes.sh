#!/usr/bin/bash
# Where do the hand-scheduled persistent builds pay?  Runs the fmha_forward driver over a range of problem sizes (the
# number of work items = batch * heads * query tiles is what matters) several times each: the automatic choice, the
# compiler-scheduled builds only (CFK_FMHA_HANDLOOP=0), and the hand-scheduled builds by wish (CFK_FMHA_TILE=...h: 256
# and 128 query rows), and prints kernel, milliseconds and TFLOP/s per run.  The thresholds of the automatic choice (fmha_fwd_kernel.h:
# hand_loop_pays) come from this table on an MI355X; the reference has no counterpart (its tile is a compile-time choice,
# src/fmha-pipeline/compile_run_all_config.sh:3-6).
#   ./run_problem_sizes.sh [fp16|fp8]        (default: both)
HERE="$(cd "$(dirname "$0")" && pwd)"
ITERS=${ITERS:-300}
run() {  # label env... -- args...
  local label=$1; shift
  local out
  out=$("$@" 2>&1) || { echo "  $label: FAILED"; return; }
  local kernel gf ms
  kernel=$(sed -n 's/^KERNEL = //p' <<<"$out")
  gf=$(sed -n 's/^CUTE_FMHA: *\[ *\([0-9.]*\)\]Gflop.*/\1/p' <<<"$out")
  ms=$(sed -n 's/^CUTE_FMHA:.*(\([0-9.]*\))ms.*/\1/p' <<<"$out")
  printf "  %-12s %-48s %8s ms %7.0f TFLOP/s\n" "$label" "$kernel" "$ms" "$(awk -v g="$gf" 'BEGIN{print g/1000}')"
}
sweep() {  # prec flags, head, seq, "wish ...", heads...
  local flags=$1 head=$2 seq=$3 wishes=$4; shift 4
  for H in "$@"; do
    echo "head dim $head, seq $seq, heads $H: $(( H * seq / 128 )) items of 128 rows"
    local args=(--batch-size=1 --seq-length=$seq --dim-size=$(( H * head )) --head-size=$head --iterations=$ITERS --reference-check=false $flags)
    run auto "$HERE/fmha_forward" "${args[@]}"
    run compiler env CFK_FMHA_HANDLOOP=0 "$HERE/fmha_forward" "${args[@]}"
    for W in $wishes; do run "$W" env CFK_FMHA_TILE=$W "$HERE/fmha_forward" "${args[@]}"; done
  done
}
if [[ ${1:-fp16} == fp16 ]]; then
  sweep "--prec-type=1" 128 2048 "256x128/16h 128x128/16h" 6 8 12 16 20 24 32 40 48 64 128
  sweep "--prec-type=1" 128 8192 "256x128/16h 128x128/16h" 2 4 8
  sweep "--prec-type=1" 128 1024 "256x128/16h 128x128/16h" 16 32 64
  sweep "--prec-type=1" 128 512 "256x128/16h 128x128/16h" 32 64 128
  sweep "--prec-type=1" 64 2048 "256x128/16h 128x128/16h" 6 8 12 16 20 24 32 40 64
  sweep "--prec-type=1" 64 8192 "256x128/16h 128x128/16h" 2 4 8
  sweep "--prec-type=1" 256 8192 128x64/16h 1 2 3 4 6 8 16
  sweep "--prec-type=1" 256 1024 128x64/16h 2 8 32
  sweep "--prec-type=1" 256 512 128x64/16h 2 8 32
  sweep "--prec-type=1" 256 256 128x64/16h 8 32
fi
if [[ ${1:-fp8} == fp8 ]]; then
  sweep "--prec-type=2 --gemm2-fp8=true" 128 4096 "256x128/32h 128x128/32h" 2 4 6 8 10 12 16 20 24 28 32 64
  sweep "--prec-type=2 --gemm2-fp8=true" 128 16384 "256x128/32h 128x128/32h" 1 2 4
  sweep "--prec-type=2 --gemm2-fp8=true" 128 3072 "256x128/32h 128x128/32h" 4 8 12 16 20 24 28 32 40 64
  sweep "--prec-type=2 --gemm2-fp8=true" 128 3136 "256x128/32h 128x128/32h" 8 16 32
  sweep "--prec-type=2 --gemm2-fp8=true" 128 3584 "256x128/32h 128x128/32h" 8 20 32
  # (below 3072 keys the automatic choice stays off the hand-scheduled e4m3 builds for accuracy, not for speed)
  sweep "--prec-type=2 --gemm2-fp8=true" 128 2048 "256x128/32h 128x128/32h" 8 16 20 32 64
  sweep "--prec-type=2 --gemm2-fp8=true" 128 1024 "256x128/32h 128x128/32h" 16 32 64 128
  sweep "--prec-type=2 --gemm2-fp8=true" 128 512 "256x128/32h 128x128/32h" 64 128 256
fi
