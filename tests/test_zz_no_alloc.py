"""The allocation-free entry point (flashllm_spmm_splitk_static: slabs in the library's own fixed device
array) against flashllm_spmm_splitk with a caller workspace: the same kernels, so C must be identical
bit for bit.  Two calls in a row, the second on a smaller input, so that whatever the first left in the
shared array is there when the second runs."""
import sys

import numpy as np
import pytest

import synth
from gpu_util import assert_close

pytestmark = pytest.mark.gpu


def one_call(product, torch, oracle, m, k, n, split_k, seed):
    print(f"static workspace {m}x{k} N={n} split_k={split_k}", flush=True)
    sys.stdout.flush()
    a = synth.sparse_matrix(m, k, 0.8, seed, dist="normal", sigma=0.05)
    b_h = synth.dense_b(k, n, seed + 1, dist="normal")
    w = product.SparseWeight(a)
    b = torch.from_numpy(b_h).cuda()
    want = torch.full((n * m,), float("nan"), dtype=torch.float16, device="cuda")
    ws = torch.full((max(split_k, 1) * n * m,), float("nan"), dtype=torch.float16, device="cuda")
    product.spmm_splitk(w.comp, w.offs, b, want, m, n, k, ws, split_k)
    got = torch.full((n * m,), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    # free device memory as the driver reports it: a hipMalloc inside the library would not go through torch's
    # allocator, so torch's own counters cannot see it (they are checked too, for the binding's sake)
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before, _ = torch.cuda.mem_get_info()
    product.spmm_splitk_static(w.comp, w.offs, b, got, m, n, k, split_k)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"device memory in use changed by {free_before - free_after} bytes across the call"
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    got_h, want_h = got.cpu().numpy(), want.cpu().numpy()
    assert np.array_equal(got_h.view(np.uint16), want_h.view(np.uint16))
    ref, _ = oracle.gemm_f32(a, b_h, n)
    assert_close(got_h.reshape(n, m), ref, f"static {m}x{k} split_k={split_k}")


def test_static_workspace_entry_point_matches_caller_workspace(product, oracle):
    import torch

    assert torch.cuda.is_available()
    one_call(product, torch, oracle, 2048, 2048, 32, 8, 70)   # 1 MiB of slabs
    one_call(product, torch, oracle, 512, 1024, 16, 3, 72)    # smaller: the array still holds the first call's slabs
    one_call(product, torch, oracle, 256, 512, 8, 1, 74)      # Split_K = 1 touches no slab storage at all


def test_static_workspace_call_under_stream_capture(product):
    """The callers this entry point is for include code under stream capture, where an allocation or a wait for
    the host invalidates the capture.  After one eager call (which resolves the array's address on this device)
    the call is recorded into a graph and replayed with new contents of B; every replay must equal the eager call
    with a caller workspace bit for bit."""
    import torch

    assert torch.cuda.is_available()
    print("static workspace under capture", flush=True)
    sys.stdout.flush()
    m, k, n, s = 1024, 1536, 16, 4
    w = product.SparseWeight(synth.sparse_matrix(m, k, 0.8, 76, dist="normal", sigma=0.05))
    b = torch.zeros(n * k, dtype=torch.float16, device="cuda")
    c = torch.zeros(n * m, dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        product.spmm_splitk_static(w.comp, w.offs, b, c, m, n, k, s, stream=side)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        product.spmm_splitk_static(w.comp, w.offs, b, c, m, n, k, s, stream=torch.cuda.current_stream())
    want = torch.empty_like(c)
    ws = torch.empty(s * n * m, dtype=torch.float16, device="cuda")
    for rep in range(3):
        b.copy_(torch.from_numpy(synth.dense_b(k, n, 80 + rep, dist="normal")).reshape(-1))
        c.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        product.spmm_splitk(w.comp, w.offs, b, want, m, n, k, ws, s)
        torch.cuda.synchronize()
        assert np.array_equal(c.cpu().numpy().view(np.uint16), want.cpu().numpy().view(np.uint16)), f"replay {rep}"


def test_static_workspace_rejects_what_does_not_fit(product, capfd):
    import torch

    assert torch.cuda.is_available()
    m, k, n, s = 36864, 128, 64, 8  # 8 * 36864 * 64 * 2 = 36 MiB > 32 MiB
    assert product.workspace_bytes(m, n, s) > product.STATIC_WORKSPACE_MAX_BYTES
    x = torch.zeros(16, dtype=torch.int32, device="cuda")
    with pytest.raises(product.HipError) as e:
        product.spmm_splitk_static(x, x, x, x, m, n, k, s)
    assert e.value.code == 1
    assert "exceeds" in capfd.readouterr().err
