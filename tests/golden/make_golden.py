"""Writes the golden fixtures under tests/golden/ (run once, in the container that holds the
reference tree; the GPU box only reads the JSON it produced).

Sources of truth, none of them this repository's own code:
  * /root/reference/example/mtx_dump.txt -- the dump the reference's example wrote for
    init_random(1024, 1024, 32, 1, 0.2, false, 2021): pins the mask generator and the
    rand()%9-4 value stream (fixture data held by the reference itself);
  * oracle/_ref/libref_mask.so -- the reference's own util/random_mask.cc compiled as is:
    pins the mask at the graded sizes (including the un-paired shuffle path that the dump does
    not reach) and the divisor/padding form;
  * libstdc++'s std::shuffle + std::default_random_engine called from a 10-line C++ program:
    pins the row permutation (spmm/blockwise_format.h:89-95 makes exactly this call).
Only digests and short prefixes are stored, not the 538 KB dump.
"""
import ctypes as C
import hashlib
import json
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
REF = "/root/reference"


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def dump_fixture():
    lines = open(os.path.join(REF, "example", "mtx_dump.txt")).read().split("\n")
    hdr = [int(x) for x in lines[:6]]
    indptr = np.array(lines[6].split(), dtype=np.int32)
    indices = np.array(lines[7].split(), dtype=np.int32)
    values = np.array(lines[8].split(), dtype=np.float32)
    return dict(
        header=hdr,  # nrow ncol nnzb brow bcol row_permute
        text_sha256=hashlib.sha256(open(os.path.join(REF, "example", "mtx_dump.txt"), "rb").read()).hexdigest(),
        text_len=os.path.getsize(os.path.join(REF, "example", "mtx_dump.txt")),
        indptr=indptr.tolist(),
        indices_sha256=sha(indices), indices_head=indices[:32].tolist(), indices_len=int(indices.size),
        values_sha256=sha(values), values_head=values[:32].tolist(), values_len=int(values.size),
    )


def ref_masks():
    from oracle import oracle as O
    assert O.ref_lib() is not None, "build oracle/_ref first (make -C oracle)"
    cases = [  # nrow ncol brow bcol density seed divisor padding
        (1024, 1024, 64, 1, 0.25, 2021, 1, 1), (4096, 4096, 64, 1, 0.1, 2021, 1, 1), (4096, 1024, 32, 1, 0.2, 2021, 1, 1),
        (2048, 4608, 64, 1, 0.1, 2021, 1, 1), (512, 2304, 32, 1, 0.3, 2021, 1, 1), (1024, 1024, 16, 1, 0.1, 2021, 1, 1),
        (1024, 1024, 128, 1, 0.1, 2021, 1, 1), (1024, 1024, 32, 1, 0.1, 2021, 1, 1), (256, 256, 16, 1, 0.3, 7, 4, 8),
        (128, 64, 16, 1, 0.25, 7, 1, 1), (64, 48, 32, 1, 1.0, 3, 1, 1), (64, 48, 32, 1, 0.0, 3, 1, 1),
    ]
    out = []
    for c in cases:
        nnzb, indptr, indices = O.ref_random_mask(c[0], c[1], c[2], c[3], c[4], c[5], c[6], c[7])
        out.append(dict(args=list(c), nnzb=nnzb, indptr=indptr.tolist() if len(indptr) <= 40 else None,
                        indptr_sha256=sha(indptr), indices_sha256=sha(indices), indices_len=int(indices.size),
                        indices_head=indices[:16].tolist()))
    return out


def stdlib_permutations():
    src = r'''
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <numeric>
#include <random>
#include <vector>
int main(int argc, char** argv) {
    int n = atoi(argv[1]); unsigned seed = (unsigned)strtoul(argv[2], 0, 10);
    std::vector<int> p(n); std::iota(p.begin(), p.end(), 0);
    std::shuffle(p.begin(), p.end(), std::default_random_engine(seed));
    for (int x : p) printf("%d\n", x);
}'''
    with tempfile.TemporaryDirectory() as d:
        open(os.path.join(d, "p.cc"), "w").write(src)
        subprocess.check_call(["g++", "-O2", "-std=c++11", "-o", os.path.join(d, "p"), os.path.join(d, "p.cc")])
        out = []
        for n, seed in [(16, 2021), (17, 2021), (64, 5), (1024, 2021), (4096, 2021), (2048, 2021), (512, 2021),
                        (70000, 11), (1, 3), (2, 3)]:
            txt = subprocess.check_output([os.path.join(d, "p"), str(n), str(seed)]).decode()
            p = np.array(txt.split(), dtype=np.int32)
            out.append(dict(n=n, seed=seed, sha256=sha(p), head=p[:16].tolist()))
    return out


if __name__ == "__main__":
    g = dict(dump=dump_fixture(), ref_masks=ref_masks(), permutations=stdlib_permutations())
    json.dump(g, open(os.path.join(HERE, "golden.json"), "w"), indent=1)
    print("wrote", os.path.join(HERE, "golden.json"))
