#!/bin/bash
# Autotune sweep over the twelve bit combinations at decode shapes, one result file per
# (shape, combination) under ./results -- the flow of the reference's engine/test.sh, driven by
# build/test_any_mma.  Usage: engine/test.sh [M] (default 1); run from abq-llm_amd/.
set -e
M=${1:-1}
BIN=./build/test_any_mma
rm -rf results
mkdir -p results
# "x_bits w_bits" pairs: the symmetric widths, then the mixed ones
COMBOS="2:2 3:3 4:4 5:5 6:6 7:7 8:8 4:2 6:2 8:2 8:3 8:4"
for shape in "4096 4096" "8192 1024" "11008 4096" "5120 5120" "4096 11008"; do
    set -- $shape
    N=$1
    K=$2
    for c in $COMBOS; do
        q=${c%%:*}
        p=${c##*:}
        $BIN "$M" "$N" "$K" "$q" "$p" 1 --tuning-out results/tuning.txt > "results/${M}x${N}x${K}_w${p}a${q}.txt"
    done
    echo "M=$M N=$N K=$K: $(cat results/${M}x${N}x${K}_*.txt | grep -c PASSED) lines PASSED, $(cat results/${M}x${N}x${K}_*.txt | grep -c 'FAILED\|ERROR') FAILED or ERROR"
done
grep -h "best kernel config" results/*.txt | sort | uniq -c | sort -rn | head
# results/tuning.txt now holds the best tile of every operand layout per shape: load it with abq_tuning_load (or
# test_any_mma --tuning), or append it to engine/tuning_mi355x.txt and rebuild to make it the library's default.
echo "tuning table: results/tuning.txt ($(wc -l < results/tuning.txt) entries)"
