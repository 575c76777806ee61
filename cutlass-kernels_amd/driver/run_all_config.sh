#!/usr/bin/bash
# Sweep of the fmha_forward driver over precision x head size x tile shape, after the reference's
# src/fmha-pipeline/compile_run_all_config.sh (same problem: batch 4, seq 4096, dim 2048; verify / verify-all modes
# run the reference check with --iterations=1, the FLOP run uses --iterations=1000).  The reference rebuilds for each
# QBLKSIZE x KBLKSIZE; here the tile shape is a run-time choice (CFK_FMHA_TILE=small|large), so nothing is rebuilt.
#   ./run_all_config.sh            FLOP runs only
#   ./run_all_config.sh verify     reference check + FLOP runs
#   ./run_all_config.sh verify-all reference check including the row-max / row-sum taps, no FLOP runs
HERE="$(cd "$(dirname "$0")" && pwd)"
TILES=( small large )
HEADSIZES=( 64 128 256 )
PRECS=( 1 2 )
MODE=$1
STATUS=0
for TILE in "${TILES[@]}"; do
for PREC in "${PRECS[@]}"; do
for HEAD in "${HEADSIZES[@]}"; do
  if [[ $TILE == large && ( $HEAD == 256 || ( $PREC == 2 && $HEAD == 64 ) ) ]]; then continue; fi   # no large tile there
  export CFK_FMHA_TILE=$TILE
  if [[ $MODE == verify || $MODE == verify-all ]]; then
    VA=false; [[ $MODE == verify-all ]] && VA=true
    "$HERE/fmha_forward" --batch-size=4 --seq-length=4096 --dim-size=2048 --iterations=1 --head-size=$HEAD \
        --reference-check=true --verify-all=$VA --prec-type=$PREC || STATUS=1
  fi
  if [[ $MODE != verify-all ]]; then
    echo "FLOP RUN BEGIN"
    echo "PREC=$PREC, TILE=$TILE, HEAD=$HEAD"
    "$HERE/fmha_forward" --batch-size=4 --seq-length=4096 --dim-size=2048 --iterations=1000 --head-size=$HEAD \
        --reference-check=false --prec-type=$PREC || STATUS=1
    echo "FLOP RUN END"
  fi
done
done
done
exit $STATUS
