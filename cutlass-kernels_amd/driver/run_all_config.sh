#!/usr/bin/bash
# Sweep of the fmha_forward driver over precision mode x head size x query tile x key tile, after the reference's
# src/fmha-pipeline/compile_run_all_config.sh (same problem: batch 4, seq 4096, dim 2048; verify / verify-all modes run
# the reference check with --iterations=1, the FLOP run uses --iterations=1000).  The reference rebuilds for each
# QBLKSIZE x KBLKSIZE in {64,128}^2 (:3-6); here every tile shape is built and CFK_FMHA_TILE=<query rows>x<keys> picks
# one at run time (a suffix /16 asks for the fp16 build on 16x16x32 MFMAs, /16h and /32h for the builds with the
# hand-scheduled main loop, 32x64 is the small-grid build), so nothing is rebuilt.  Precision modes: fp16; fp8 = the
# reference's -DGEMM2FP8 build with V in [B,S,H,D]; fp8-bdhs = the same with V pre-transposed offline
# (src/fmha-pipeline/README.md:22, fmha_forward.cu:514-532); hybrid = the reference's default fp8 build (e4m3 Q,K; fp16
# P,V; :446-450).
#   ./run_all_config.sh            FLOP runs only
#   ./run_all_config.sh verify     reference check + FLOP runs
#   ./run_all_config.sh verify-all reference check including the score / row-max / row-sum taps, no FLOP runs
# Problem size and iteration count can be overridden: BATCH=2 SEQ=1024 DIM=512 ITERS=100 ./run_all_config.sh verify-all
HERE="$(cd "$(dirname "$0")" && pwd)"
BATCH=${BATCH:-4}; SEQ=${SEQ:-4096}; DIM=${DIM:-2048}; ITERS=${ITERS:-1000}
MODES=( fp16 fp8 fp8-bdhs hybrid )
HEADSIZES=( 64 128 256 )
TILES=( 128x64 256x64 128x128 256x128 128x64/16 256x64/16 128x128/16 256x128/16 256x128/16h 128x64/16h 256x128/32h 32x64 )
MODE=$1
STATUS=0
# the tile shapes that exist per mode and head size (the others would silently run the default tile)
has_tile() {  # mode head tile
  case "$1:$2" in
    fp16:64) [[ $3 != 128x32 && $3 != 256x64/16 && $3 != *x128/16 && $3 != 128x64/16h && $3 != */32h ]] ;;
    fp16:128) [[ $3 != 128x32 && $3 != 128x64/16h && $3 != */32h ]] ;;
    fp16:256) [[ $3 == 128x32 || $3 == 128x64 || $3 == 128x64/16h ]] ;;
    hybrid:256) [[ $3 == 128x32 ]] ;;
    fp8:128) [[ $3 != 128x32 && $3 != */16 && $3 != */16h && $3 != 32x64 ]] ;;
    fp8:64|fp8:256) [[ $3 == 128x64 || $3 == 128x128 ]] ;;
    fp8-bdhs:*) [[ $3 == 128x64 ]] ;;
    hybrid:64) [[ $3 == 128x64 || $3 == 128x128 ]] ;;
    hybrid:128) [[ $3 == 128x64 || $3 == 256x64 || $3 == 256x128 ]] ;;
    *) return 1 ;;
  esac
}
for M in "${MODES[@]}"; do
for HEAD in "${HEADSIZES[@]}"; do
for TILE in "${TILES[@]}" 128x32; do
  has_tile $M $HEAD $TILE || continue
  case $M in
    fp16) FLAGS="--prec-type=1" ;;
    fp8) FLAGS="--prec-type=2 --gemm2-fp8=true" ;;
    fp8-bdhs) FLAGS="--prec-type=2 --gemm2-fp8=true --v-layout=bdhs" ;;
    hybrid) FLAGS="--prec-type=2 --gemm2-fp8=false" ;;
  esac
  export CFK_FMHA_TILE=$TILE
  echo "CONFIG MODE=$M, HEAD=$HEAD, TILE=$TILE"
  if [[ $MODE == verify || $MODE == verify-all ]]; then
    VA=false; [[ $MODE == verify-all ]] && VA=true
    "$HERE/fmha_forward" --batch-size=$BATCH --seq-length=$SEQ --dim-size=$DIM --iterations=1 --head-size=$HEAD \
        --reference-check=true --verify-all=$VA $FLAGS || STATUS=1
  fi
  if [[ $MODE != verify-all ]]; then
    echo "FLOP RUN BEGIN"
    "$HERE/fmha_forward" --batch-size=$BATCH --seq-length=$SEQ --dim-size=$DIM --iterations=$ITERS --head-size=$HEAD \
        --reference-check=false $FLAGS || STATUS=1
    echo "FLOP RUN END"
  fi
done
done
done
exit $STATUS
