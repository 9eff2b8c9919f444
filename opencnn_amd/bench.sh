#!/bin/bash
# Sweep of the reference's benchmark shapes (bench/bench.sh:3-21) through the wgrad CLI.
cd "$(dirname "$0")"
echo "in_n,in_c,in_h,filt_k,filt_w,ms,ref_formula_tflops,effective_tflops,mfma_pct_of_fp32_peak,hbm_gbs_min_bytes,ms_fused_kernel,ms_filter_transform"
for shape in "64 56 56 64" "128 28 28 128" "256 14 14 256" "512 7 7 512"; do
  set -- $shape
  for n in 32 64 96 128; do
    ./wgrad $n $1 $2 $3 $4 $1 3 3 | head -1 || exit 1
  done
done
