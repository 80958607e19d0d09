"""Helpers shared by the GPU parity tests and the smoke check."""
import numpy as np

REL_TOL = 1e-2  # the stated bar: max relative error of C against the fp32-accumulated product


def errors(c, ref):
    """c, ref: (N, M) arrays.  Returns (max|d| / max|ref|, worst element-wise excess over
    1e-2*|ref| + 1e-2*rms(ref))."""
    c = np.asarray(c, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    d = np.abs(c - ref)
    scale = max(np.max(np.abs(ref)), 1e-30)
    rms = np.sqrt(np.mean(ref * ref))
    excess = np.max(d - (REL_TOL * np.abs(ref) + REL_TOL * rms))
    return float(np.max(d) / scale), float(excess)


def assert_close(c, ref, what=""):
    rel, excess = errors(c, ref)
    assert np.all(np.isfinite(np.asarray(c, dtype=np.float32))), what
    assert rel <= REL_TOL, f"{what}: max|d|/max|ref| = {rel:.3e}"
    assert excess <= 0, f"{what}: element-wise bound exceeded by {excess:.3e}"


def run_spmm(product, a_host, b_host, n, split_k, reorder=True, poison=True):
    """Compress on the host, run SpMM_SplitK on cuda:0 through the C ABI, return C as (N, M) fp16."""
    import torch

    m, k = a_host.shape
    w = product.SparseWeight(a_host, reorder=reorder)
    b = torch.from_numpy(np.ascontiguousarray(b_host)).cuda()
    c = torch.full((n * m,), float("nan"), dtype=torch.float16, device="cuda") if poison else None
    ws = None
    if split_k > 1:
        ws = torch.full((split_k * n * m,), float("nan"), dtype=torch.float16, device="cuda")
    c = w.matmul(b, n, c=c, workspace=ws, split_k=split_k)
    torch.cuda.synchronize()
    return c.cpu().numpy().reshape(n, m), w, ws
