#!/usr/bin/env python3
"""Shape sweeps of SpMM_SplitK_API on one MI355X: the counterpart of the reference's
kernel_benchmark/benchmark.sh + spmm_test.cu (12 OPT shapes x N x sparsity), for the configurations
this build is measured on.  Prints one JSON line per case.

    python flash-llm_amd/sweep.py ffn        # FFN shapes, sparsity {70,80,90} %, N {8,16,32,64} (and 128, 256 on the up-projection)
    python flash-llm_amd/sweep.py hidden12k  # hidden-12288 projections, Beta(2,8) row densities, N = 32
    python flash-llm_amd/sweep.py square     # 9216 x 9216, N = 16, Split_K {1,2,4,8,heuristic}
    python flash-llm_amd/sweep.py layers     # four chained linears per layer, hidden 9216, 16 tokens, 8 layers
    python flash-llm_amd/sweep.py compress   # Tiled-CSL compression of 36864 x 9216: host threads vs the device-side compressor

Every case reports ms per call, dense-equivalent TFLOPS (2MNK/t, kernel_benchmark/spmm_test.cu:314-316),
algorithmic GB/s and its fraction of the 8 TB/s HBM peak, a dense fp16 GEMM of the same shape through
torch, and the relative error of sampled rows against an fp32 product.
"""
import json
import os
import sys
import time

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)

import flashllm_spmm as F  # noqa: E402
import synth  # noqa: E402

HBM_PEAK = 8000.0


def timed(torch, fn, steps=300, settle_ms=200.0):
    t0 = time.perf_counter()
    i = 0
    while (time.perf_counter() - t0) * 1e3 < settle_ms:
        for _ in range(50):
            fn(i)
            i += 1
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(steps):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def run_case(torch, name, a, n, split_k=None, b_dist="normal", dense=True, copies=None):
    m, k = a.shape
    items, offsets = F.init_sparse_matrix_a(a)
    nnz = int(items.size)
    copies = copies or max(1, min(4, int(1.2e9 // max(1, 4 * nnz))))
    comps = [torch.from_numpy(items.view(np.int32) if nnz else np.zeros(1, np.int32)).cuda() for _ in range(copies)]
    offs = torch.from_numpy(offsets).cuda()
    b_h = synth.dense_b(k, n, 1, dist=b_dist)
    b = torch.from_numpy(b_h).cuda()
    s = split_k or F.splitk_heuristic(m, n, k)
    c = torch.empty(n * m, dtype=torch.float16, device="cuda")
    ws = torch.empty(max(1, s) * n * m, dtype=torch.float16, device="cuda")
    ms = timed(torch, lambda i: F.spmm_splitk(comps[i % copies], offs, b, c, m, n, k, ws, s))
    ms_kernel = timed(torch, lambda i: F.spmm_partials(comps[i % copies], offs, b, c, m, n, k, ws, s, slab_order=F.SLABS_BY_WORKGROUP))
    F.spmm_splitk(comps[0], offs, b, c, m, n, k, ws, s)
    torch.cuda.synchronize()
    rows = np.arange(0, m, max(1, m // 256))
    ref = b_h.astype(np.float32) @ a[rows].astype(np.float32).T
    got = c.cpu().numpy().reshape(n, m)[:, rows].astype(np.float32)
    err = float(np.max(np.abs(got - ref)) / max(np.max(np.abs(ref)), 1e-30))
    # a sweep line is only worth reporting for a correct product: the stated bar on C, on the sampled rows
    assert np.all(np.isfinite(got)) and err <= 1e-2, f"{name} N={n} split_k={s}: max|d|/max|ref| = {err:.3e} on {rows.size} sampled rows"
    alg = 4 * nnz + 4 * offsets.size + 2 * k * n + 2 * m * n
    out = {"case": name, "M": m, "K": k, "N": n, "sparsity": round(1.0 - float(np.count_nonzero(a)) / a.size, 4), "split_k": s,
           "ms": ms, "kernel_ms": ms_kernel, "tflops": 2.0 * m * n * k / ms / 1e9,
           "alg_GBps_kernel": alg / ms_kernel / 1e6, "frac_hbm_kernel": alg / ms_kernel / 1e6 / HBM_PEAK,
           "frac_hbm_whole_call": alg / ms / 1e6 / HBM_PEAK,
           "mfma_tflops_kernel": 2.0 * m * n * k / ms_kernel / 1e9, "max_rel_err": err,
           "compressed_MB": 4 * nnz / 1e6, "dense_MB": 2 * m * k / 1e6}
    if dense:
        a_d = torch.from_numpy(a).cuda()
        bt = b.view(n, k).t().contiguous()
        md = timed(torch, lambda i: torch.matmul(a_d, bt), steps=100)
        out["dense_ms"] = md
        out["speedup_vs_dense"] = md / ms
        del a_d
    print(json.dumps(out), flush=True)
    return out


def main():
    import torch

    what = sys.argv[1] if len(sys.argv) > 1 else "square"
    F.lib()
    assert torch.cuda.is_available()
    threads = min(16, os.cpu_count() or 1)
    if what == "square":
        a = synth.sparse_matrix(9216, 9216, 0.8, 0, threads=threads)
        for s in (1, 2, 4, 8, None):
            run_case(torch, "9216x9216", a, 16, split_k=s, b_dist="uniform", dense=s is None)
    elif what == "ffn":
        for (m, k) in ((36864, 9216), (9216, 36864)):
            for sp in (0.7, 0.8, 0.9):
                a = synth.sparse_matrix(m, k, sp, 0, dist="normal", sigma=0.02, threads=threads)
                # N = 128 / 256 (the kernel for wide B) on the up-projection: where the dense library takes over
                for n in (8, 16, 32, 64) + ((128, 256) if m > k else ()):
                    run_case(torch, f"ffn {m}x{k} s{int(sp * 100)}", a, n, dense=(sp == 0.8 or n >= 128))
    elif what == "hidden12k":
        for (m, k) in ((36864, 12288), (12288, 12288), (49152, 12288), (12288, 49152)):
            a = synth.sparse_matrix(m, k, 0.8, 0, dist="normal", sigma=0.02, row_beta=True, threads=threads)
            run_case(torch, f"hidden12288 {m}x{k} beta rows", a, 32)
    elif what == "layers":
        hidden, tokens, layers = 9216, 16, int(sys.argv[2]) if len(sys.argv) > 2 else 8
        shapes = [(3 * hidden, hidden), (hidden, hidden), (4 * hidden, hidden), (hidden, 4 * hidden)]
        built, comp_bytes, dense_bytes = [], 0, 0
        for layer in range(layers):
            ws = []
            for w, (m, k) in enumerate(shapes):
                a = synth.sparse_matrix(m, k, 0.8, layer * 4 + w, dist="normal", sigma=0.02, threads=threads)
                sw = F.SparseWeight(a)
                comp_bytes += 4 * sw.nnz + 4 * sw.num_offsets
                dense_bytes += 2 * m * k
                ws.append(sw)
            built.append(F.DecoderLayer(*ws))
        x = torch.from_numpy(synth.dense_b(hidden, tokens, 99, dist="normal")).cuda()
        bufs = [torch.empty(n * tokens, dtype=torch.float16, device="cuda") for n in (3 * hidden, hidden, hidden, 4 * hidden, hidden)]
        wsp = torch.empty(max(l.workspace_halfs(tokens) for l in built), dtype=torch.float16, device="cuda")

        def all_layers(i):
            cur = x
            for l in built:
                cur, _ = l.forward(cur, tokens, buffers=bufs, workspace=wsp)

        ms = timed(torch, all_layers, steps=50)
        # the same chain recorded once into a HIP graph and replayed (the calls allocate nothing and never wait)
        all_layers(0)
        torch.cuda.synchronize()
        eager = bufs[4].clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            cur = x
            for l in built:
                cur, _ = l.forward(cur, tokens, buffers=bufs, workspace=wsp, stream=torch.cuda.current_stream())
        bufs[4].fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(bufs[4].view(torch.int16), eager.view(torch.int16)), "graph replay differs from the eager chain"
        ms_graph = timed(torch, lambda i: graph.replay(), steps=50)
        per_layer = []
        for l in built:
            per_layer.append(timed(torch, lambda i: l.forward(x, tokens, buffers=bufs, workspace=wsp), steps=100, settle_ms=50))
        flops = layers * sum(2.0 * m * k * tokens for m, k in shapes)
        print(json.dumps({"case": "chained decoder-layer linears", "hidden": hidden, "tokens": tokens, "layers": layers,
                          "ms_all_layers": ms, "ms_all_layers_graph_replay": ms_graph, "ms_per_layer": per_layer, "tflops": flops / ms / 1e9,
                          "weight_GB_compressed": comp_bytes / 1e9, "weight_GB_dense": dense_bytes / 1e9,
                          "alg_GBps": comp_bytes / ms / 1e6, "frac_hbm": comp_bytes / ms / 1e6 / HBM_PEAK}), flush=True)
    elif what == "compress":
        # Tiled-CSL compression of the headline weight: host (threaded, and on one thread as the reference
        # runs it) against the device-side compressor on a device-resident matrix.

        m, k = 36864, 9216
        a = synth.sparse_matrix(m, k, 0.8, 0, dist="normal", sigma=0.02, threads=threads)
        t0 = time.perf_counter()
        items, offsets = F.init_sparse_matrix_a(a, threads=threads)
        t_host = time.perf_counter() - t0
        t0 = time.perf_counter()
        F.init_sparse_matrix_a(a, threads=1)
        t_host1 = time.perf_counter() - t0
        F.lib().flashllm_set_compress_threads(0)
        a_dev = torch.from_numpy(a).cuda()
        comp, offs = F.device_compress(a_dev)
        torch.cuda.synchronize()
        same = bool(np.array_equal(comp.cpu().numpy().view(np.uint32), items) and np.array_equal(offs.cpu().numpy(), offsets))

        def both(i):
            F.lib().flashllm_device_tile_offsets(None, a_dev.data_ptr(), m, k, offs.data_ptr(), None)
            F.lib().flashllm_device_compress(None, a_dev.data_ptr(), m, k, offs.data_ptr(), comp.data_ptr())

        ms = timed(torch, both, steps=20, settle_ms=100)
        ms_offsets = timed(torch, lambda i: F.lib().flashllm_device_tile_offsets(None, a_dev.data_ptr(), m, k, offs.data_ptr(), None),
                           steps=20, settle_ms=100)
        moved = 2 * 2.0 * m * k + 4.0 * items.size + 2 * 4.0 * offsets.size
        print(json.dumps({"case": "Tiled-CSL compression 36864x9216 80%", "host_threads": threads, "host_s": t_host,
                          "host_1thread_s": t_host1, "device_ms": ms, "device_offsets_ms": ms_offsets,
                          "device_encode_ms": ms - ms_offsets, "device_bytes_moved_MB": moved / 1e6,
                          "device_GBps": moved / ms / 1e6, "frac_hbm": moved / ms / 1e6 / HBM_PEAK,
                          "bit_identical_to_host": same}), flush=True)
    else:
        sys.exit(__doc__)


if __name__ == "__main__":
    main()
