"""Runs the C++ programs of tests/cpp and the benchmark command lines (built beforehand by __graft_entry__.build()): every entry of the SpMM and
SpConv operator tables, called through the veneer that mirrors the reference's headers and linked against
libblock_sparse.a, checked against the CPU oracle with the reference's own acceptance rule."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin")


def _run(name, timeout):
    exe = os.path.join(BIN, name)
    assert os.path.exists(exe), "%s is not built: run __graft_entry__.build()" % exe
    print("running", exe, flush=True)
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout)
    print(p.stdout[-4000:], flush=True)
    assert p.returncode == 0, p.stdout[-4000:]
    assert "ALL PASSED" in p.stdout
    return p.stdout


@pytest.mark.gpu
def test_spmm_operator_table(torch_gpu):
    out = _run("test_spmm_blockwise", 100)
    assert out.count("Passed") > 60 and "Failed" not in out


@pytest.mark.gpu
def test_spconv_operator_table(torch_gpu):
    out = _run("test_spconv_blockwise", 110)
    assert out.count("Passed") > 60 and "Failed" not in out


@pytest.mark.gpu
def test_reference_example_flows(torch_gpu):
    # the reference's three example programs as flows over this library's headers, checked with the library's
    # own get_host_reference, linked against libblock_sparse.a only
    out = _run("test_example_flows", 100)
    assert out.count("Passed") == 7 and "Failed" not in out


BENCH = os.path.join(ROOT, "shflbw_sparse_nn_amd", "block_sparse", "benchmark")


def _bench(name, args):
    exe = os.path.join(BENCH, name)
    assert os.path.exists(exe), "%s is not built: run __graft_entry__.build()" % exe
    print("running", exe, " ".join(args), flush=True)
    return subprocess.run([exe] + args, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=100)


@pytest.mark.gpu
def test_benchmark_spmm_command_line(torch_gpu):
    # one sweep line of the reference's scripts/benchmark/gemm.block_sparse.sh; the output line has the reference's
    # fields (benchmark/benchmark.spmm.cu:109-118): arch, the matrix config, n, ten tile numbers, time, tflop/s
    p = _bench("benchmark.spmm.out", "--m 1024 --n 960 --k 1024 --d 0.1 --sparsity-type block --block-size 64 --row-permute".split())
    assert p.returncode == 0, p.stderr
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) >= 10  # every tile name of the block size
    for l in lines:
        f = l.split()
        assert f[0] == "950" and f[1:5] == ["1024", "1024", "64", "1"] and f[7] == "row-permute"
        assert f[8] == "960" and f[9] == "64" and f[-1] == "tflop/s)" and f[-4] == "(us)"
        assert 0.5 < float(f[-5]) < 500 and float(f[-3]) > 0
    # m is padded up to the block size and n to 32 like the reference does, --one-tile prints one line
    p = _bench("benchmark.spmm.out", "--m 1000 --n 100 --k 512 --d 0.2 --sparsity-type block --block-size 32 --one-tile".split())
    assert p.returncode == 0 and "m padded to : 1024" in p.stderr and "n padded to : 128" in p.stderr
    assert len(p.stdout.strip().splitlines()) == 1
    # the complaints of the reference's parser
    p = _bench("benchmark.spmm.out", ["--m", "4"])
    assert p.returncode != 0 and "Forget to set m,n,k or density?" in p.stderr
    p = _bench("benchmark.spmm.out", "--m 64 --n 64 --k 64 --d 0.5 --sparsity-type block --block-size 48".split())
    assert p.returncode != 0 and "Unsupported block size" in p.stderr


@pytest.mark.gpu
def test_benchmark_spconv_command_line(torch_gpu):
    p = _bench("benchmark.spconv.out", ("--B 16 --H 14 --W 14 --C 256 --F 256 --R 3 --S 3 --stride 2 --d 0.1 "
                                        "--sparsity-type block --block-size 64 --row-permute --one-tile").split())
    assert p.returncode == 0, p.stderr
    f = p.stdout.split()
    assert f[0] == "950" and f[1:5] == ["256", "3", "3", "256"] and "filter-permute" in f
    i = f.index("filter-permute")
    assert f[i + 1:i + 5] == ["16", "14", "14", "2"] and f[i + 5] == "64" and f[-1] == "tflop/s)"
    assert 0.5 < float(f[-5]) < 500
