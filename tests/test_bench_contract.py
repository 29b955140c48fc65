"""bench.py and workloads.py, as far as a box without a GPU can hold them to their contract: one GPU only, no
CPU stand-in for the measured path, and the five measured problems are the ones BASELINE.json describes."""
import json
import os
import subprocess
import sys

import workloads as P

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], cwd=ROOT, capture_output=True,
                          text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)
    assert not [l for l in r.stdout.splitlines() if l.startswith("{")]


def test_no_json_line_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        return  # the GPU suite and the driver run the real thing
    r = _run("--steps", "2", "--warmup", "1")
    assert r.returncode != 0, "bench.py must not fall back to a CPU path"
    assert not [l for l in r.stdout.splitlines() if l.startswith("{")]


def test_measured_problems_are_the_baseline_configs():
    cfgs = json.load(open(os.path.join(ROOT, "BASELINE.json")))["configs"]
    assert len(cfgs) == 5
    c0, c1, c2 = (P.SPMM_CONFIGS[k] for k in ("cfg0", "cfg1", "cfg2"))
    assert (c0["M"], c0["K"], c0["N"], c0["V"], c0["d"]) == (1024, 1024, 1024, 64, 0.25)
    assert "M=1024" in cfgs[0] and "block_size=64" in cfgs[0] and "d=0.25" in cfgs[0] and "uniform" in cfgs[0]
    assert c0["a_dist"][0] == c0["b_dist"][0] == "uniform"
    assert (c1["M"], c1["K"], c1["N"], c1["V"], c1["d"]) == (4096, 4096, 4096, 64, 0.1)
    assert "M=K=N=4096" in cfgs[1] and "block_size=64" in cfgs[1] and "d=0.1" in cfgs[1]
    assert c1["a_dist"] == ("uniform", 1.0) and c1["b_dist"] == ("uniform", 1.0)
    assert (c2["M"], c2["K"], c2["N"], c2["V"], c2["d"]) == (4096, 1024, 4096, 32, 0.2)
    assert "M=4096" in cfgs[2] and "K=1024" in cfgs[2] and "block_size=32" in cfgs[2] and "d=0.2" in cfgs[2]
    assert c2["a_dist"] == ("normal", 0.02) and c2["b_dist"] == ("normal", 1.0)
    c3, c4 = P.CONV_CONFIGS["cfg3"], P.CONV_CONFIGS["cfg4"]
    assert [c3[k] for k in ("B", "H", "W", "C", "F", "R", "S", "stride", "V", "d")] == [16, 14, 14, 512, 2048, 3, 3, 1, 64, 0.1]
    assert "B=16" in cfgs[3] and "C=512" in cfgs[3] and "F=2048" in cfgs[3] and "block_size=64" in cfgs[3] and "NHWC" in cfgs[3]
    assert [c4[k] for k in ("B", "H", "W", "C", "F", "R", "S", "stride", "V", "d")] == [32, 28, 28, 256, 512, 3, 3, 2, 32, 0.3]
    assert "B=32" in cfgs[4] and "C=256" in cfgs[4] and "stride 2" in cfgs[4] and "block_size=32" in cfgs[4] and "d=0.3" in cfgs[4]
    assert c4["w_dist"] == ("normal", 0.05)
