#!/bin/bash
# Regenerates the result tables of this directory on one MI355X: the run lines of the
# reference's compile.sh:12-29 (`--if_bench 2`: every logN at logBS + logN = 28) for the plain,
# fault-tolerant and error-injecting kernels and for the vendor library (`--if_bench 12`), in
# the reference's line format (`data/benchmark_*_A100_*.csv`), plus the fault-tolerance tables
# over all batch sizes (`--if_bench 1`, the reference's `data_ft/ft_scheme_threadblock_bs=*`).
#   usage: data/run_benchmarks.sh [output directory, default data]      (from the repository root)
set -u
out=${1:-data}
bin=turbofft_amd/bin/turbofft
gpu=MI355X
mkdir -p "$out/ft"
run() {   # run <file> <line prefix> <flags...>: keep the metric lines only, as the reference's files do,
          # as a CSV with a header and the fraction of the 8 TB/s HBM peak as a last column
    local file=$1 prefix=$2; shift 2
    echo "$file" >&2
    timeout -k 10 300 "$bin" "$@" --gpu $gpu | grep "^$prefix" |
        awk -F', *' 'BEGIN { print "library,logN,log2_batch,ms,GFLOPS,GBps,pct_of_hbm_peak" }
                     { printf "%s,%d,%d,%.3f,%.3f,%.3f,%.2f\n", $1, $2, $3, $4, $5, $6, $6 / 80.0 }' > "$file"
    [ "$(wc -l < "$file")" -gt 1 ] || { echo "failed: $bin $*" >&2; exit 1; }
}
for dt in 0 1; do
    p=$([ $dt = 0 ] && echo fp32 || echo fp64)
    run "$out/benchmark_TurboFFT_${gpu}_$p.csv"     "turboFFT," --if_bench 2  --thread_bs 1  --datatype $dt --if_ft 0 --if_err 0
    run "$out/benchmark_TurboFFT_ft_${gpu}_$p.csv"  "turboFFT," --if_bench 2  --thread_bs 32 --datatype $dt --if_ft 1 --if_err 0
    run "$out/benchmark_TurboFFT_err_${gpu}_$p.csv" "turboFFT," --if_bench 2  --thread_bs 32 --datatype $dt --if_ft 1 --if_err 1
    run "$out/benchmark_hipFFT_${gpu}_$p.csv"       "hipFFT,"   --if_bench 12 --datatype $dt
    # plans that hold the fused kernel of their two launches (fp32 2^16, fp64 2^15 and 2^16; the other sizes run as above)
    TURBOFFT_FUSED=1 run "$out/benchmark_TurboFFT_fused_${gpu}_$p.csv" "turboFFT," --if_bench 2 --thread_bs 1 --datatype $dt --if_ft 0 --if_err 0
    for t in 1 2 4 8 16 32; do
        run "$out/ft/ft_scheme_threadblock_bs=${t}_${gpu}_$p.csv" "turboFFT," --if_bench 1 --thread_bs $t --datatype $dt --if_ft 1 --if_err 1
    done
    # thread-level verification (the scheme of the reference's data_ft/ft_scheme_thread_bs=1_*): clean, and with the injection cadence
    run "$out/benchmark_TurboFFT_thread_level_${gpu}_$p.csv" "turboFFT," --if_bench 2 --thread_bs 1 --datatype $dt --if_ft 1 --if_err 0 --ft_scheme 1
    run "$out/ft/ft_scheme_thread_bs=1_${gpu}_$p.csv"        "turboFFT," --if_bench 1 --thread_bs 1 --datatype $dt --if_ft 1 --if_err 1 --ft_scheme 1
done
