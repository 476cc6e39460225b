#!/bin/bash
# Benchmark sweep over op kinds and feature widths with the GPU tester/timer,
# the counterpart of the reference's runtime.sh (kernel in {g,m,s,t} x dataset
# x K = 32..256 step 32, -nrep 5 -skHd 1, one CSV per dataset and kind;
# runtime.sh:21-25, 63-64, 146-191).
#
#   fusedmm_amd/runtime_sweep.sh [-p s|d] [-i 32|64] [-r resultdir] graph1.mtx [graph2.mtx ...]
#
# Writes <resultdir>/<dataset>-<kind>-<p>real-gpu.csv with the timer's CSV lines.
set -e
here="$(cd "$(dirname "$0")" && pwd)"
pre=s; ibit=64; resdir=results
while getopts "p:i:r:" opt; do
  case $opt in
    p) pre=$OPTARG ;;
    i) ibit=$OPTARG ;;
    r) resdir=$OPTARG ;;
    *) echo "usage: $0 [-p s|d] [-i 32|64] [-r resultdir] file.mtx ..."; exit 1 ;;
  esac
done
shift $((OPTIND - 1))
[ $# -ge 1 ] || { echo "need at least one .mtx file"; exit 1; }
if [ "$pre" = d ]; then exe="$here/bin/xfusedMMtime_d_i$ibit"; else exe="$here/bin/xfusedMMtime_i$ibit"; fi
[ -x "$exe" ] || { echo "$exe is not built: python -m fusedmm_amd.build"; exit 1; }
mkdir -p "$resdir"
for data in "$@"; do
  dset=$(basename "$data" .mtx)
  for kern in g m s t f; do
    out="$resdir/$dset-$kern-${pre}real-gpu.csv"
    "$exe" -input "$data" -t $kern -K 32 -nrep 5 -skHd 0 | grep "," > "$out"
    for k in 64 96 128 160 192 224 256; do
      "$exe" -input "$data" -t $kern -K $k -nrep 5 -skHd 1 | grep "," >> "$out"
    done
    echo "wrote $out"
  done
done
