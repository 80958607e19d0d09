#!/usr/bin/env python3
"""Headline benchmark: one SpMM_SplitK_API call per step on one MI355X.

Workload (BASELINE.json configs[2], the shape the metric is quoted on): the FFN up-projection
A = 36864 x 9216 fp16 at 80 % unstructured sparsity, nonzeros ~ N(0, 0.02); B = 9216 x 16 fp16 ~ N(0,1).
A step is the whole API call (SpMM kernel + split-K reduction) with Compressed_A, TileOffsets and B
resident in HBM.  Steps rotate over several device copies of Compressed_A (272 MB each, more than the
256 MB Infinity Cache together) so every launch streams its weights from HBM.

Each figure is the median of `--repeats` (5) timed windows of `--steps` calls, with the fastest and slowest
window beside it.  Prints one JSON line; `value` = dense-equivalent TFLOPS = 2*M*N*K / t (the reference's formula,
kernel_benchmark/spmm_test.cu:314-316) of the whole call.  `roofline`: `frac` (= `kernel_frac`) is for the
dominant kernel alone (the SpMM kernel, timed live with events on the launch stream in a second loop
without the reduction); `whole_call_frac` is the same algorithmic bytes over the time of the whole call,
the figure `value` corresponds to.  `traffic` is the HBM bytes per SpMM-kernel launch measured with
rocprofv3 counters, read from the summary under profiles/ whose workload line matches this run (null when
none does).  `cpu_baseline` times the CPU oracle (compression on one thread, fp32 GEMM on all host cores)
on the same workload and is a reported figure, not a target.
"""
import argparse
import glob
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "flash-llm_amd"))

HBM_PEAK_GBS = 8000.0


def measured_traffic(m, k, n, split_k, nnz_padded):
    """HBM bytes per SpMM-kernel launch from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary of this
    very workload under profiles/ (each counter scaled by what it reads for a plain 256 MiB copy): the
    summary carries a line `traffic_bytes_per_launch: <bytes> M=.. K=.. N=.. split_k=.. nnz_padded=..`.
    Returns (bytes, file) or (None, None) when no summary matches this run."""
    pat = re.compile(r"traffic_bytes_per_launch:\s*(\d+)\s+M=(\d+)\s+K=(\d+)\s+N=(\d+)\s+split_k=(\d+)\s+nnz_padded=(\d+)")
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.md"))):
        with open(path) as f:
            for hit in pat.finditer(f.read()):
                if tuple(int(x) for x in hit.groups()[1:]) == (m, k, n, split_k, nnz_padded):
                    return int(hit.group(1)), os.path.relpath(path, ROOT)
    return None, None


def algorithmic_bytes(nnz_padded, m, n, k):
    """Compressed_A + TileOffsets + B once + C once."""
    return 4 * nnz_padded + 4 * ((m // 128) * (k // 64) + 2) + 2 * k * n + 2 * m * n


def cpu_baseline(a, b, n):
    """The reference's CPU path restated by the oracle: host compression (single thread, as the
    reference) and an fp32 GEMM on the decompressed weights over all host cores."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle

    m, k = a.shape
    t0 = time.perf_counter()
    _, items, offsets = oracle.compress_reorder(a)
    t_compress = time.perf_counter() - t0
    dense = oracle.scatter(items, offsets, m, k)
    best = None
    threads = 1
    for _ in range(3):
        t0 = time.perf_counter()
        _, threads = oracle.gemm_f32(dense, b, n)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return {
        "value": 2.0 * m * n * k / best / 1e12,
        "unit": "TFLOPS",
        "cores": threads,
        "kind": "port",
        "sample": f"whole workload {m}x{k}x{n}: fp32 GEMM on decompressed weights, best of 3 on {threads} threads; "
                  f"Tiled-CSL compression of the same matrix on 1 thread reported beside it",
        "gemm_ms": best * 1e3,
        "compress_s_1thread": t_compress,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="untimed run of the same step before the warm-up, so that clocks have left their idle state")
    ap.add_argument("--repeats", type=int, default=5,
                    help="timed windows of --steps calls each; the median window is reported, min and max beside it")
    ap.add_argument("--m", type=int, default=36864)
    ap.add_argument("--k", type=int, default=9216)
    ap.add_argument("--n", type=int, default=16)
    ap.add_argument("--sparsity", type=float, default=0.8)
    ap.add_argument("--split-k", type=int, default=0, help="0 = the library's heuristic")
    ap.add_argument("--copies", type=int, default=4, help="device copies of Compressed_A to rotate over")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain device-to-device copy of 256 MiB: the known-size kernel the FETCH_SIZE / "
                         "WRITE_SIZE counters are scaled by")
    ap.add_argument("--no-dense", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (rows of A would shard across GPUs with no "
                 "exchange, a split of K adds one all-reduce of C). Run with --gpus 1.")

    import numpy as np
    import torch

    import flashllm_spmm as F
    import synth

    F.lib()  # fails loudly if libSpMM_API.so is not built
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    m, k, n = args.m, args.k, args.n
    threads = min(16, os.cpu_count() or 1)
    a = synth.sparse_matrix(m, k, args.sparsity, 0, dist="normal", sigma=0.02, threads=threads)
    b_h = synth.dense_b(k, n, 0, dist="normal")
    items, offsets = F.init_sparse_matrix_a(a)
    nnz = int(items.size)
    split_k = args.split_k or F.splitk_heuristic(m, n, k)

    dev = "cuda"
    comps = [torch.from_numpy(items.view(np.int32)).to(dev) for _ in range(max(1, args.copies))]
    offs = torch.from_numpy(offsets).to(dev)
    b = torch.from_numpy(b_h).to(dev)
    c = torch.empty(n * m, dtype=torch.float16, device=dev)
    ws = torch.empty(max(1, split_k) * n * m, dtype=torch.float16, device=dev)

    # The C entry points with their arguments converted once: the timed region may be as short as 20 calls
    # (1 ms), where the host time before the first launch reaches the GPU is part of what is measured.
    lib = F.lib()
    stream = F._stream(None)
    whole_args = [(stream, None, F._ptr(cp), F._ptr(offs), F._ptr(b), F._ptr(c), m, n, k, F._ptr(ws), split_k) for cp in comps]
    part_args = [(stream, F._ptr(cp), F._ptr(offs), F._ptr(b), F._ptr(c), m, n, k, F._ptr(ws), split_k, F.SLABS_BY_WORKGROUP)
                 for cp in comps]

    def step(i):
        rc = lib.flashllm_spmm_splitk(*whole_args[i % len(whole_args)])
        if rc:
            raise F.HipError(rc)

    def kernel_only(i):
        rc = lib.flashllm_spmm_partials(*part_args[i % len(part_args)])
        if rc:
            raise F.HipError(rc)

    def settle(fn):
        # The GPU leaves its idle clocks only after a few hundred ms of work (the reference times 10 000
        # launches after 100 warm-ups for the same reason, kernel_benchmark/spmm_test_utils.h:21-22).
        t0 = time.perf_counter()
        i = 0
        while (time.perf_counter() - t0) * 1e3 < args.settle_ms:
            for _ in range(100):
                fn(i)
                i += 1
            torch.cuda.synchronize()

    def windows(fn, steps, warmup, repeats):
        """ms per call of `repeats` timed windows of `steps` back-to-back calls each, after one settle phase and
        `warmup` untimed calls (the reference times one window of 10 000 launches after 100 warm-ups,
        kernel_benchmark/spmm_test_utils.h:21-22; several shorter windows show the spread as well).  The whole
        timed region is bracketed by a synchronize on both sides; inside it the windows follow each other on the
        stream, separated only by the events that delimit them, so that none but the first starts on an idle GPU
        (with windows of 20 calls a start from idle costs each call of the window about 0.7 us)."""
        settle(fn)
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(repeats + 1)]
        marks[0].record()
        for r in range(repeats):
            for i in range(steps):
                fn(i)
            marks[r + 1].record()
        torch.cuda.synchronize()
        return sorted(marks[r].elapsed_time(marks[r + 1]) / steps for r in range(repeats))

    def timed(fn, steps, warmup):
        return windows(fn, steps, warmup, 1)[0]

    w_step = windows(step, args.steps, args.warmup, args.repeats)
    w_kernel = windows(kernel_only, args.steps, args.warmup, args.repeats)
    ms_step = w_step[len(w_step) // 2]      # the median window is the reported figure
    ms_kernel = w_kernel[len(w_kernel) // 2]

    # correctness of what was just timed (cheap sample of rows against an fp32 product)
    step(0)
    torch.cuda.synchronize()
    rows = np.arange(0, m, max(1, m // 512))
    ref = b_h.astype(np.float32) @ a[rows].astype(np.float32).T
    got = c.cpu().numpy().reshape(n, m)[:, rows].astype(np.float32)
    rel_err = float(np.max(np.abs(got - ref)) / np.max(np.abs(ref)))

    alg = algorithmic_bytes(nnz, m, n, k)
    flops = 2.0 * m * n * k
    achieved = alg / (ms_kernel * 1e-3) / 1e9
    traffic, traffic_source = measured_traffic(m, k, n, split_k, nnz)
    xcd = F.xcd_of_workgroups((m // 128) * split_k)
    out = {
        "metric": "dense-equiv TFLOPS + % HBM roofline, M=36864 K=9216 N=16, 80% sparse fp16",
        "value": flops / (ms_step * 1e-3) / 1e12,
        "unit": "TFLOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": args.settle_ms,
        "ms_per_step": ms_step,
        "repeats": args.repeats,
        "ms_per_step_min": w_step[0],
        "ms_per_step_max": w_step[-1],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp16",
        "data": "synthetic",
        "config": {
            "workload": f"SpMM_SplitK_API {m}x{k} (80% sparse ffn up-projection) x {k}x{n}, Tiled-CSL, fp16 in / fp32 accumulate",
            "M": m, "K": k, "N": n, "sparsity": args.sparsity, "split_k": split_k,
            "nnz_padded": nnz, "compressed_a_copies_rotated": len(comps),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic,
            "traffic_source": traffic_source,
            "kernel": "spmm_stream_kernel",
            "kernel_ms": ms_kernel,
            "kernel_ms_min": w_kernel[0],
            "kernel_ms_max": w_kernel[-1],
            "kernel_frac": achieved / HBM_PEAK_GBS,
            "whole_call_frac": alg / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "algorithmic_bytes": alg,
        },
        "whole_call": {
            "effective_GBps": alg / (ms_step * 1e-3) / 1e9,
            "frac_of_hbm_peak": alg / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "reduction_ms": max(ms_step - ms_kernel, 0.0),
        },
        "max_rel_err_sampled_rows": rel_err,
        # the placement of slices and reduction workgroups counts on workgroup w running on XCD w % 8
        "xcd_round_robin": bool((xcd == xcd[[i % 8 for i in range(xcd.size)]]).all()),
    }

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        ms_copy = timed(lambda i: dst.copy_(src), 10, 2)
        out["copy_256MiB"] = {"ms": ms_copy, "GBps_read_plus_write": 2 * (256 << 20) / (ms_copy * 1e-3) / 1e9}
        del src, dst

    if not args.no_dense:
        # dense fp16 GEMM of the same shape through the BLAS library torch ships (hipBLASLt/rocBLAS)
        a_d = torch.from_numpy(a).to(dev)
        bt = b.view(n, k).t().contiguous()  # K x N
        ms_dense = timed(lambda i: torch.matmul(a_d, bt), max(10, args.steps // 4), 5)
        out["dense_fp16_gemm"] = {"ms": ms_dense, "tflops": flops / (ms_dense * 1e-3) / 1e12,
                                  "speedup_of_spmm": ms_dense / ms_step}
        del a_d

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(a, b_h, n)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
