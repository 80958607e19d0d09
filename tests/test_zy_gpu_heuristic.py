"""The Split_K the library recommends (flashllm_splitk_heuristic, which stands in for the reference's per-shape
tables hand-tuned for A100, kernel_benchmark/benchmark.sh:13-15) against its neighbours on the benchmark shapes:
the whole SpMM_SplitK_API call at the recommended value may take at most 8 % longer than at the best of
{s-2 .. s+2}.  Weights are pruned and compressed on the GPU; every timed loop rotates over enough copies of
Compressed_A that the weights come from HBM; each figure is the smallest of five loops (the least disturbed
one).  Wide-B cases (N a multiple of 128, whose timings step with the number of workgroup rounds) are held to
15 %.  The file sorts behind every parity test on purpose: a wall-clock comparison on a shared machine must
not keep a parity test from running.  Before it is timed, the product at the recommended Split_K is compared
with an fp32 product on sampled rows, so the values the heuristic picks at full size are also checked for C."""
import sys
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

# (M, K, N, density of nonzeros, bound)
SHAPES = [(36864, 9216, 16, 0.2, 1.08), (9216, 36864, 16, 0.2, 1.08), (9216, 9216, 16, 0.2, 1.08), (36864, 12288, 32, 0.2, 1.08),
          (49152, 12288, 32, 0.2, 1.08), (36864, 9216, 16, 0.3, 1.08), (36864, 9216, 16, 0.1, 1.08), (9216, 36864, 32, 0.3, 1.08),
          (9216, 9216, 64, 0.1, 1.08), (36864, 9216, 128, 0.2, 1.15), (9216, 9216, 256, 0.2, 1.15)]


def best_time_us(torch, fn, loops=5, steps=150, settle_s=0.1):
    t0 = time.perf_counter()
    i = 0
    while time.perf_counter() - t0 < settle_s:
        for _ in range(50):
            fn(i)
            i += 1
        torch.cuda.synchronize()
    out = []
    for _ in range(loops):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(steps):
            fn(i)
        e1.record()
        torch.cuda.synchronize()
        out.append(e0.elapsed_time(e1) / steps * 1e3)
    return min(out)


@pytest.mark.parametrize("m,k,n,density,bound", SHAPES)
def test_recommended_split_k_is_close_to_the_best_of_its_neighbours(product, m, k, n, density, bound):
    import torch

    assert torch.cuda.is_available()
    print(f"split_k neighbourhood {m}x{k} N={n} density={density}", flush=True)
    sys.stdout.flush()
    g = torch.Generator(device="cuda").manual_seed(m + k + n)
    a = torch.randn(m, k, dtype=torch.float16, device="cuda", generator=g) * 0.02
    a = torch.where(torch.rand(m, k, device="cuda", generator=g) < density, a, torch.zeros((), dtype=torch.float16, device="cuda"))
    comp, offs = product.device_compress(a)
    rows = torch.arange(0, m, max(1, m // 256), device="cuda")
    a_rows = a[rows].float()
    del a
    copies = max(2, min(8, int(6e8 // (4 * comp.numel())) + 1))
    comps = [comp] + [comp.clone() for _ in range(copies - 1)]
    b = torch.randn(n * k, dtype=torch.float16, device="cuda", generator=g)
    c = torch.empty(n * m, dtype=torch.float16, device="cuda")
    s = product.splitk_heuristic(m, n, k)
    cands = [x for x in range(s - 2, s + 3) if 1 <= x <= min(32, k // 64)]
    ws = torch.empty(max(cands) * n * m, dtype=torch.float16, device="cuda")

    # the product at the recommended Split_K, sampled rows against an fp32 product
    product.spmm_splitk(comps[0], offs, b, c, m, n, k, ws, s)
    torch.cuda.synchronize()
    ref = (b.view(n, k).float() @ a_rows.t()).cpu().numpy()
    got = c.view(n, m)[:, rows].float().cpu().numpy()
    assert np.all(np.isfinite(got))
    assert np.max(np.abs(got - ref)) <= 1e-2 * np.max(np.abs(ref)), (m, k, n, s)

    times = {}
    for x in cands:
        times[x] = best_time_us(torch, lambda i: product.spmm_splitk(comps[i % copies], offs, b, c, m, n, k, ws, x))
    print("  " + "  ".join(f"{x}: {t:.2f} us" + ("*" if x == s else "") for x, t in times.items()), flush=True)
    assert times[s] <= bound * min(times.values()), (s, times)
