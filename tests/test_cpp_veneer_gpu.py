"""Runs the C++ programs of tests/cpp (built beforehand by __graft_entry__.build()): every entry of the SpMM and
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
