#!/usr/bin/env python3
"""Benchmark of the Shfl-BW hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config all|cfg0|cfg1|cfg2|cfg3|cfg4|refconv]

Default (`--config all`): every graded configuration is measured - the SpMM configs cfg0, cfg1 (the headline:
M = K = N = 4096, block size 64, density 0.1, row-permuted) and cfg2, the sparse Conv2D configs cfg3 and cfg4 - and
ONE JSON line is printed: its top-level figures are the headline's, its `configs` array holds kernel, time,
effective TFLOP/s, share of the fp16 MFMA peak and roofline of all five.  `--config <name>` measures one
configuration alone (what the profiles under profiles/ were taken with) and prints its full line.

A step is one `exec` of the operator on device-resident operands (fp16 in, fp32 accumulate, fp16 out): one launch
for the SpMM configs, the whole convolution (every launch of the form the library chooses) for cfg3 / cfg4.  Every
configuration first passes a correctness gate (bit-exact against the CPU oracle on the integer twin of the
workload).  Timing follows the reference's benchmark (benchmark/benchmark.spmm.cu:29-50, benchmark.spconv.cu:29-50):
W warm-up launches, then K back-to-back launches between two events on the launch stream - here WINDOWS such
windows in a row; `ms_per_step` is the median window, the fastest and slowest are reported beside it.  A single
window of a few launches falls into the clock ramp of an idle GPU (the first ~10 ms of a burst run 8-10 % slower), so
SETTLE_MS of untimed launches go in front of the warm-up; the reference's own loop from an idle GPU is reported
beside it (`reference_timing_loop`).  The line carries the roofline of the kernel and
the CPU oracle timed on the host cores as a baseline (headline only); the headline also carries a dense fp16 GEMM of
the same shape.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 matrix-core peak
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
WINDOWS = 5                    # timed windows of `steps` launches each; the median is the figure
SETTLE_MS = 20.0               # untimed launches in front of the warm-up until the shader clock has settled


def measured_traffic(config, kernel):
    """HBM-side bytes per step from the tracked counter summary (profiles/traffic.json: FETCH_SIZE and
    WRITE_SIZE runs of this script under rocprofv3 --pmc, each scaled by what the same counter reads for a
    device copy of known size).  An entry only applies to the kernel it names; None when there is none."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        table = json.load(f)
    for e in table.get("entries", []):
        if e["config"] == config and e["kernel"] == kernel:
            return round(e["fetch_kib"] * 1024 * e["fetch_scale"] + e["write_kib"] * 1024 * e["write_scale"])
    return None


def time_launches(torch, stream, op, n):
    """Mean milliseconds of n back-to-back launches of `op` between two events on `stream`."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(n):
        op(stream.cuda_stream)
    e1.record(stream)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / n


def reference_loop(torch, stream, op):
    """The reference's own loop (1 + 10 warm-ups, 100 launches) from an idle GPU: the clock is still ramping."""
    torch.cuda.synchronize()
    time.sleep(0.05)
    for _ in range(11):
        op(stream.cuda_stream)
    return time_launches(torch, stream, op, 100)


def timed_windows(torch, stream, op, steps, warmup, windows=WINDOWS):
    """`warmup` untimed launches, then `windows` windows of `steps` launches each, every window between its own pair
    of events, all back to back on the stream.  Returns the per-launch milliseconds of every window and the wall
    time of the timed part."""
    # an idle GPU needs about 10 ms of load before its clock settles (the first launches of a burst run 8-10 % slower):
    # SETTLE_MS of untimed launches first, whatever `warmup` is
    t_end = time.time() + SETTLE_MS * 1e-3
    while time.time() < t_end:
        for _ in range(50):
            op(stream.cuda_stream)
        torch.cuda.synchronize()
    for _ in range(warmup):
        op(stream.cuda_stream)
    torch.cuda.synchronize()
    wall0 = time.time()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(windows + 1)]
    ev[0].record(stream)
    for i in range(windows):
        for _ in range(steps):
            op(stream.cuda_stream)
        ev[i + 1].record(stream)
    torch.cuda.synchronize()
    return [ev[i].elapsed_time(ev[i + 1]) / steps for i in range(windows)], time.time() - wall0


def spread(ms_list):
    return {"median": round(statistics.median(ms_list), 6), "min": round(min(ms_list), 6), "max": round(max(ms_list), 6),
            "windows": len(ms_list)}


def roofline(eff_flops, alg_bytes, t, traffic):
    """The bound of the workload (MFMA when its arithmetic intensity is above the ridge, else HBM) and the
    fraction of it reached in t seconds."""
    ai = eff_flops / alg_bytes
    if ai * HBM_PEAK_GBS * 1e9 > MFMA_F16_PEAK_TFLOPS * 1e12:
        a = eff_flops / t / 1e12
        r = {"bound": "mfma", "achieved": round(a, 2), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
             "frac": round(a / MFMA_F16_PEAK_TFLOPS, 4)}
    else:
        a = alg_bytes / t / 1e9
        r = {"bound": "hbm", "achieved": round(a, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
             "frac": round(a / HBM_PEAK_GBS, 4)}
    r.update({"traffic": traffic, "algorithmic_bytes": alg_bytes, "effective_flops": eff_flops})
    return r


def cpu_baseline(run_all, run_one, eff_flops, sub_flops, what_all, what_one, threads):
    """The oracle (a port of the reference's get_host_reference) on the host cores: about 10 s with every
    core on the whole workload, about 5 s with a single thread on a sample of it."""
    run_all()  # page in
    reps, t_sum = 0, 0.0
    while t_sum < 10.0 and reps < 400:
        t0 = time.time()
        run_all()
        t_sum += time.time() - t0
        reps += 1
    t_all = t_sum / reps
    reps1, t1_sum = 0, 0.0
    while t1_sum < 5.0 and reps1 < 200:
        t0 = time.time()
        run_one()
        t1_sum += time.time() - t0
        reps1 += 1
    t_one = t1_sum / reps1
    return {"value": round(eff_flops / t_all / 1e12, 6), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "%s on %d threads, mean of %d runs (%.1f s of CPU work): %.4f s per pass; one thread on %s, "
                      "mean of %d runs: %.4f s = %.4f TFLOP/s"
                      % (what_all, threads, reps, t_sum, t_all, what_one, reps1, t_one, sub_flops / t_one / 1e12)}


def timing_note(args):
    return ("%g ms of untimed launches (clock settling) + %d warm-up launches, then %d windows of %d back-to-back launches, "
            "each between two events on the launch stream, operands resident; ms_per_step = median window"
            % (SETTLE_MS, args.warmup, WINDOWS, args.steps))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=500,
                    help="untimed launches before the timed ones; the shader clock needs about 10 ms of load to settle")
    ap.add_argument("--config", default="all",
                    help="all (default: every graded config, headline cfg1 on top) | cfg0 | cfg1 | cfg2 (SpMM) | cfg3 | cfg4 "
                         "(SpConv2D) | refconv (the reference's own conv test case on its own tensor layout; not graded)")
    ap.add_argument("--variant", type=int, default=-1, help="force a kernel variant (default: library choice)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--traffic", default=None,
                    help="HBM bytes per step from a newer rocprofv3 --pmc measurement; default: the tracked "
                         "figure for this config and kernel, null if there is none")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import shflbw_sparse_nn_amd as S  # raises if the HIP library is missing: there is no fallback
    import workloads as P

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if args.config != "all":
        fn = bench_conv if args.config in P.CONV_CONFIGS else bench_spmm
        print(json.dumps(fn(args, args.config, np, torch, S, P, full=True, cpu=not args.no_cpu)))
        return
    # every graded configuration; the CPU leg, the dense GEMM and the cold-cache rotation for the headline only
    lines = {}
    for name in ("cfg0", "cfg2", "cfg3", "cfg4", "cfg1"):
        fn = bench_conv if name in P.CONV_CONFIGS else bench_spmm
        lines[name] = fn(args, name, np, torch, S, P, full=name == "cfg1", cpu=name == "cfg1" and not args.no_cpu)
    out = lines["cfg1"]
    out["configs"] = [{"config": n, "workload": lines[n]["config"]["workload"], "kernel": lines[n]["config"]["kernel"],
                       "ms_per_step": lines[n]["ms_per_step"], "ms_per_step_spread": lines[n]["ms_per_step_spread"],
                       "tflops": lines[n]["value"], "pct_mfma_peak": lines[n]["pct_mfma_peak"],
                       "integer_valued_operands_ms": lines[n]["integer_valued_operands"]["ms_per_step"],
                       "gate": lines[n]["gate"], "roofline": lines[n]["roofline"]}
                      for n in ("cfg0", "cfg1", "cfg2", "cfg3", "cfg4")]
    print(json.dumps(out))


def bench_spmm(args, name, np, torch, S, P, full, cpu):
    from oracle import oracle as O  # correctness gate and CPU baseline only
    c = P.SPMM_CONFIGS[name]
    M, K, N, V, d = c["M"], c["K"], c["N"], c["V"], c["d"]
    w = P.make_weight(M, K, V, d, True, 2021, dist=c["a_dist"])
    B = P.make_dense(K, N, 2021, dist=c["b_dist"])
    nnzb = w["nnzb"]
    eff_flops = 2.0 * nnzb * V * N
    # algorithmic bytes of one launch: A values + (indices, indptr, perm) + B once + D once
    alg_bytes = nnzb * V * 2 + (nnzb + M // V + 1 + M) * 4 + K * N * 2 + M * N * 2

    mat = P.upload_weight(w)
    dB = P.to_dev(torch, B)
    dD = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    op = S.SpmmBlockwiseOp(args.variant)
    st = op.initialize(mat, N, dB.data_ptr(), dD.data_ptr())
    variant_name = S.spmm_variants(V)[st.variant]
    stream = torch.cuda.current_stream()

    # correctness gate before any timing: bit-exact against the oracle on the integer twin of the workload
    wi = P.make_weight(M, K, V, d, True, 2021, integer=True)
    Bi = P.make_dense(K, N, 2021, integer=True)
    mi = P.upload_weight(wi)
    dBi = P.to_dev(torch, Bi)
    dDi = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    opi = S.SpmmBlockwiseOp(args.variant)
    opi.initialize(mi, N, dBi.data_ptr(), dDi.data_ptr())
    opi(stream.cuda_stream)
    torch.cuda.synchronize()
    ref_i = O.float_to_half(P.spmm_oracle(wi, Bi))
    if not np.array_equal(dDi.cpu().numpy().view(np.uint16), ref_i.view(np.uint16)):
        print("correctness gate failed (%s): GPU result differs from the CPU oracle" % name, file=sys.stderr)
        sys.exit(1)

    ref_loop_ms = reference_loop(torch, stream, op)
    windows, wall = timed_windows(torch, stream, op, args.steps, args.warmup)
    ms_per_step = statistics.median(windows)
    t = ms_per_step * 1e-3
    eff_tflops = eff_flops / t / 1e12
    # the same launch on the integer twin (values of the reference's generator, rand() % 9 - 4): the shader clock
    # under MFMA load depends on the operand values, so this is reported beside the graded figure
    int_windows, _ = timed_windows(torch, stream, opi, args.steps, args.warmup)
    del mi, dBi, dDi, opi

    traffic = measured_traffic(name, variant_name) if args.traffic is None else round(float(args.traffic))
    out = {
        "metric": "effective sparse TFLOP/s + % fp16 MFMA peak, SpMM 4096^3 d=0.1 blk64" if name == "cfg1"
                  else "effective sparse TFLOP/s + %% fp16 MFMA peak, SpMM %s" % name,
        "value": round(eff_tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "ms_per_step_spread": spread(windows),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 (fp32 accumulate)",
        "data": "synthetic: seeded Shfl-BW mask + permutation (reference generators, seed 2021), values A %s(%g), B %s(%g)"
                % (c["a_dist"] + c["b_dist"]),
        "config": {"workload": "%s: Shfl-BW SpMM M=%d K=%d N=%d, block %d, density %g, row-permuted; nnzb=%d"
                               % (name, M, K, N, V, d, nnzb),
                   "kernel": variant_name, "timing": timing_note(args)},
        "gate": "bit-exact against the CPU oracle on the integer twin",
        "pct_mfma_peak": round(100.0 * eff_tflops / MFMA_F16_PEAK_TFLOPS, 2),
        "reference_timing_loop": {"what": "11 warm-ups + 100 launches from an idle GPU (clock still ramping)",
                                  "ms_per_step": round(ref_loop_ms, 6),
                                  "tflops": round(eff_flops / (ref_loop_ms * 1e-3) / 1e12, 1)},
        "integer_valued_operands": {"what": "same mask and shape, values in {-4..4} (the reference's generator)",
                                    "ms_per_step": round(statistics.median(int_windows), 6),
                                    "tflops": round(eff_flops / (statistics.median(int_windows) * 1e-3) / 1e12, 1)},
        "dense_equivalent_tflops": round(2.0 * M * N * K / t / 1e12, 1),
        "roofline": roofline(eff_flops, alg_bytes, t, traffic),
    }
    if full:
        # ---- cold-cache variant: rotate operand sets larger than the 256 MB last-level cache
        nsets = max(2, min(8, int(320e6 // (2 * (K * N + M * N))) + 1))
        Bs = [dB] + [dB.clone() for _ in range(nsets - 1)]
        Ds = [dD] + [torch.zeros_like(dD) for _ in range(nsets - 1)]
        ops = []
        for i in range(nsets):
            o = S.SpmmBlockwiseOp(st.variant)
            o.initialize(mat, N, Bs[i].data_ptr(), Ds[i].data_ptr())
            ops.append(o)
        for i in range(nsets):
            ops[i](stream.cuda_stream)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(args.steps):
            ops[i % nsets](stream.cuda_stream)
        e1.record(stream)
        torch.cuda.synchronize()
        out["cold_cache_ms_per_step"] = round(e0.elapsed_time(e1) / args.steps, 6)
        del Bs, Ds, ops

        # ---- dense fp16 GEMM of the same shape (library GEMM behind torch.matmul) as a reference point
        Ad = torch.randn((M, K), dtype=torch.float16, device="cuda")
        for _ in range(5):
            torch.matmul(Ad, dB, out=dD)
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(20):
            torch.matmul(Ad, dB, out=dD)
        e1.record(stream)
        torch.cuda.synchronize()
        dense_ms = e0.elapsed_time(e1) / 20
        out["dense_gemm"] = {"what": "torch.matmul fp16 %dx%dx%d (hipBLASLt/rocBLAS)" % (M, N, K),
                             "ms": round(dense_ms, 6), "tflops": round(2.0 * M * N * K / (dense_ms * 1e-3) / 1e12, 1)}
    out["cpu_baseline"] = None
    if cpu:
        X = M // V
        XS = max(1, X // 8)
        sub = dict(w, nrow=XS * V, indptr=w["indptr"][:XS + 1], indices=w["indices"][:w["indptr"][XS]],
                   values=w["values"][:w["indptr"][XS] * V], row_permute_ids=None)
        out["cpu_baseline"] = cpu_baseline(lambda: P.spmm_oracle(w, B), lambda: P.spmm_oracle(sub, B, nthreads=1),
                                           eff_flops, 2.0 * int(w["indptr"][XS]) * V * N,
                                           "whole workload (%d panels)" % X, "the first %d panels" % XS, O.max_threads())
    out["wall_s_timed_region"] = round(wall, 4)
    out["device"] = S.device_info()
    return out


def bench_conv(args, name, np, torch, S, P, full, cpu):
    """The sparse Conv2D configs (cfg3, cfg4: NHWC; refconv: the reference's test case on its C-H-W-B / F-H-W-B
    tensors); one step = one exec of the operator, i.e. every launch the chosen form of the convolution puts on
    the stream.  Same JSON shape as the SpMM line."""
    from oracle import oracle as O  # correctness gate and CPU baseline only
    c = P.CONV_CONFIGS[name]
    B, H, W, C, F, R, Sx, stride, V, d = [c[k] for k in ("B", "H", "W", "C", "F", "R", "S", "stride", "V", "d")]
    batch_first = c.get("layout") == "chwb"
    if batch_first:
        Ho, Wo = H, W
        in_shape, out_shape, variant = (C, H, W, B), (F, H, W, B), -1
        oracle = lambda w, x, **kw: P.conv_oracle_batch_first(w, R, Sx, C, x, stride)
    else:
        Ho, Wo = (H + 2 * (R // 2) - R) // stride + 1, (W + 2 * (Sx // 2) - Sx) // stride + 1
        in_shape, out_shape, variant = (B, H, W, C), (B, Ho, Wo, F), args.variant
        oracle = lambda w, x, **kw: P.conv_oracle(w, R, Sx, C, x, stride, **kw)
    npix = B * Ho * Wo
    stream = torch.cuda.current_stream()

    def make_op(w, x):
        f = P.upload_weight(w, R, Sx, C, cls=S.BlockwiseSpFilter)
        dX = P.to_dev(torch, x)
        dY = torch.full(out_shape, float("nan"), dtype=torch.float16, device="cuda")
        op = S.SpconvBlockwiseOp(variant)
        op.initialize(f, B, H, W, stride, dX.data_ptr(), dY.data_ptr(), batch_innermost=batch_first)
        return op, f, dX, dY

    # correctness gate: bit-exact against the oracle on the integer twin
    wi = P.make_weight(F, R * Sx * C, V, d, True, 2021, integer=True)
    xi = np.random.default_rng(2022).integers(-4, 5, size=in_shape).astype(np.float16)
    opi, fi, dXi, dYi = make_op(wi, xi)
    opi(stream.cuda_stream)
    torch.cuda.synchronize()
    opi.check()
    ref_i = O.float_to_half(oracle(wi, xi))
    if not np.array_equal(dYi.cpu().numpy().view(np.uint16), ref_i.view(np.uint16)):
        print("correctness gate failed (%s): GPU result differs from the CPU oracle" % name, file=sys.stderr)
        sys.exit(1)

    w = P.make_weight(F, R * Sx * C, V, d, True, 2021, dist=c["w_dist"])
    x = P.make_dense(B * H * W, C, 2021, dist=c["x_dist"]).reshape(in_shape)
    op, f, dX, dY = make_op(w, x)
    nnzb = w["nnzb"]
    eff_flops = 2.0 * nnzb * V * npix
    alg_bytes = nnzb * V * 2 + (nnzb + F // V + 1 + F) * 4 + B * H * W * C * 2 + npix * F * 2

    ref_loop_ms = reference_loop(torch, stream, op)
    windows, wall = timed_windows(torch, stream, op, args.steps, args.warmup)
    ms = statistics.median(windows)
    t = ms * 1e-3
    int_windows, _ = timed_windows(torch, stream, opi, args.steps, args.warmup)
    op.check()
    opi.check()
    del opi, fi, dXi, dYi

    cpu_line = None
    if cpu:
        X = F // V
        XS = max(1, X // 8)
        sub = dict(w, nrow=XS * V, indptr=w["indptr"][:XS + 1], indices=w["indices"][:w["indptr"][XS]],
                   values=w["values"][:w["indptr"][XS] * V], row_permute_ids=None)
        # the literal restatement of the reference's loop nest (batch-first layout) runs on one thread
        if batch_first:  # one thread throughout: a bounded sample, the first panels, stands for the workload
            cpu_line = cpu_baseline(lambda: oracle(sub, x), lambda: oracle(sub, x), 2.0 * int(w["indptr"][XS]) * V * npix,
                                    2.0 * int(w["indptr"][XS]) * V * npix, "the first %d of %d panels" % (XS, X),
                                    "the same", 1)
        else:
            cpu_line = cpu_baseline(lambda: oracle(w, x),
                                    lambda: oracle(sub, x, nthreads=1), eff_flops,
                                    2.0 * int(w["indptr"][XS]) * V * npix, "whole workload (%d panels)" % X,
                                    "the first %d panels" % XS, O.max_threads())

    eff_tflops = eff_flops / t / 1e12
    kernel = S.spconv_variant_name(op._state.variant)
    traffic = measured_traffic(name, kernel) if args.traffic is None else round(float(args.traffic))
    return {
        "metric": "effective sparse TFLOP/s + %% fp16 MFMA peak, SpConv2D %s" % name,
        "value": round(eff_tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 6), "ms_per_step_spread": spread(windows), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16 (fp32 accumulate)",
        "data": "synthetic: seeded Shfl-BW filter mask + permutation (seed 2021), filter %s(%g), input %s(%g)"
                % (c["w_dist"] + c["x_dist"]),
        "config": {"workload": "%s: sparse Conv2D %s %dx%dx%dx%d -> %d, %dx%d stride %d, block %d, density %g; "
                               "nnzb=%d" % (name, "C-H-W-B / F-H-W-B, B x H x W x C =" if batch_first else "NHWC",
                                            B, H, W, C, F, R, Sx, stride, V, d, nnzb),
                   "kernel": kernel, "timing": timing_note(args)},
        "gate": "bit-exact against the CPU oracle on the integer twin",
        "pct_mfma_peak": round(100.0 * eff_tflops / MFMA_F16_PEAK_TFLOPS, 2),
        "reference_timing_loop": {"what": "11 warm-ups + 100 execs from an idle GPU (clock still ramping)",
                                  "ms_per_step": round(ref_loop_ms, 6),
                                  "tflops": round(eff_flops / (ref_loop_ms * 1e-3) / 1e12, 1)},
        "integer_valued_operands": {"what": "same mask and shape, values in {-4..4} (the reference's generator)",
                                    "ms_per_step": round(statistics.median(int_windows), 6),
                                    "tflops": round(eff_flops / (statistics.median(int_windows) * 1e-3) / 1e12, 1)},
        "dense_equivalent_tflops": round(2.0 * npix * F * R * Sx * C / t / 1e12, 1),
        "roofline": roofline(eff_flops, alg_bytes, t, traffic), "cpu_baseline": cpu_line,
        "wall_s_timed_region": round(wall, 4), "device": S.device_info()}


if __name__ == "__main__":
    main()
