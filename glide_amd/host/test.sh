#!/bin/bash
# The reference's test.sh on synthetic data: same variables, same four commands, same result.csv.
# Usage: glide_amd/host/test.sh [work_dir]      (needs one MI355X, `make -C glide_amd/csrc` and `make -C glide_amd/host`)
set -e
here="$(cd "$(dirname "$0")" && pwd)"
root="$(cd "$here/../.." && pwd)"
bin="$root/glide_amd/bin"
work="${1:-/tmp/glide_test}"
mkdir -p "$work/temp"

data_file="$work/base.fbin"
query_file="$work/query.fbin"
truth_file="$work/query_gt100"
result_file="$work/result.csv"
dataset='synthetic100k'

metric=Euclidean

#preprocess
centroid_num=10
boundary_factor=1.04
sample_factor=0.01
#build
knn_degree=32
graph_degree=64
relaxant_factor=1.05
build_beam=64
refine_beam=128
#search
topk=10
search_beam=50

# 100 000 x 128 integer-valued rows of low intrinsic dimension, 1 000 queries, exact top-100 by brute force
PYTHONPATH="$root" python3 - "$data_file" "$query_file" "$truth_file" <<'PY'
import sys
import numpy as np
from glide_amd import datasets as D

def rows(m, seed):
    a = np.random.default_rng(0).standard_normal((12, 128)).astype(np.float32)
    r = np.random.default_rng(seed)
    z = r.standard_normal((m, 12)).astype(np.float32)
    return np.rint(np.clip(z @ a * 20 + 128 + r.standard_normal((m, 128)).astype(np.float32) * 3, 0, 255)).astype(np.float32)

base, queries = rows(100_000, 1), rows(1_000, 2)
d = (queries ** 2).sum(1)[:, None] + (base ** 2).sum(1)[None] - 2.0 * queries @ base.T
truth = np.argsort(d, axis=1, kind="stable")[:, :100].astype(np.uint32)
D.write_fbin(sys.argv[1], base)
D.write_fbin(sys.argv[2], queries)
D.write_fbin(sys.argv[3], truth)
PY

preprocess_file="$work/temp/${dataset}_centroid_${centroid_num}_boundary_${boundary_factor}_sample_${sample_factor}"
knn_file="$work/temp/${dataset}_knn_${knn_degree}"
graph_base_file="$work/temp/${dataset}_degree_${graph_degree}_relaxant_${relaxant_factor}_beam_${build_beam}_refinebeam${refine_beam}"
rm -f "$result_file"

"$bin/small_preprocess" ${data_file} ${preprocess_file} ${result_file} ${centroid_num} ${boundary_factor} ${sample_factor} ${metric}

"$bin/small_knn" ${preprocess_file} ${knn_file} ${result_file} ${knn_degree}

"$bin/small_build" ${data_file} ${preprocess_file} ${knn_file} ${graph_base_file} ${result_file} ${metric} ${graph_degree} ${knn_degree} ${relaxant_factor} ${build_beam} ${refine_beam}

"$bin/small_search" ${data_file} ${query_file} ${truth_file} ${preprocess_file} ${graph_base_file} ${result_file} ${metric} ${topk} ${search_beam}

cat "$result_file"
