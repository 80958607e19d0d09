#!/bin/bash
# The shape grid of the reference's kernel_benchmark/benchmark.sh (12 OPT weight shapes x batch x sparsity),
# run through spmm_test with SplitK 0 = the library's heuristic for MI355X (the reference lists a
# hand-tuned SplitK per shape for A100).  Usage: benchmark.sh [sparsities, default "70 80 90"]
cd "$(dirname "$0")" || exit 1
M=(21504 7168 28672 7168 27648 9216 36864 9216 36864 12288 49152 12288)
K=(7168 7168 7168 28672 9216 9216 9216 36864 12288 12288 12288 49152)
N=(8 16 32 64)
SPARSITY=(${1:-70 80 90})
for n in "${N[@]}"; do
    for i in "${!M[@]}"; do
        for s in "${SPARSITY[@]}"; do
            ./spmm_test "${M[i]}" "${K[i]}" "$n" "$s" 0 || exit 1
        done
    done
done
