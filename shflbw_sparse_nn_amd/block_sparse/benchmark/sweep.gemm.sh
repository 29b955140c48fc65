#! /bin/bash
# Sweep of the SpMM benchmark over shapes, densities and block sizes, one CSV-like line per run
# appended to result/gemm.block_sparse.csv (same loop and output file as the reference's
# scripts/benchmark/gemm.block_sparse.sh).  Run from the directory that contains block_sparse/.
mkdir -p result
log_file=result/gemm.block_sparse.csv
echo "Benchmark.gemm.block_sparse"

# m,n,k: the graded shapes first, then transformer projections / FFNs at a few token counts
shapes="1024,1024,1024 4096,4096,4096 4096,4096,1024 \
1024,512,1024 1024,2048,1024 4096,512,1024 1024,512,4096 \
4096,2048,1024 1024,2048,4096 3072,512,768 768,512,3072 \
2048,128,2048 4096,128,4096 8192,1024,2048"

for shape in $shapes; do
IFS=","; set -- $shape
m=$1; n=$2; k=$3
for d in 0.02 0.05 0.1 0.15 0.2 0.25 0.5; do
for block_sz in 16 32 64 128; do
block_sparse/benchmark/benchmark.spmm.out --m $m --n $n --k $k --d $d --sparsity-type block --block-size $block_sz --row-permute --one-tile >> $log_file
done; done; done
