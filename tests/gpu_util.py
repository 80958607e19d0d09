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


def slab_pages(slabs, m, n, rows=None):
    """Plain slabs (S, N, M) -> the same numbers in the by-workgroup order of the library (flat, S*N*M).

    Written from the layout's description, not from the kernels: a launch has units = (M/128) / rows x column
    groups; a unit is `rows` consecutive row tiles (8 for N = 64 when M/128 is a multiple of 8 and the launch has
    192 .. 256 workgroups of eight waves with a row tile each, (M/1024)*S; otherwise 1; `rows` given: that) by 16*nb columns (nb = 1 / 2 / 4 for N <= 16 / 32 / 64, 8 and 128-column
    groups for wide B); workgroup w = ((unit % per_xcd)*S + slice)*8 + unit // per_xcd with per_xcd = units // 8
    (units past a multiple of 8: w = unit*S + slice); the unit's pages are numbered row tile by row tile, the
    16-column blocks of a row tile in order (sub = row*nb + block), page sub*G + w; and inside a page the
    16-byte piece q*(4*cols) + g*cols + r16 holds rows 32q+4g..+3 and 32q+16+4g..+3 of column r16.
    """
    s = slabs.shape[0]
    slabs = slabs.reshape(s, n, m)
    wide = n % 128 == 0
    nb = 8 if wide else (1 if n <= 16 else (2 if n == 32 else 4))
    if rows is None:
        rows = 8 if n == 64 and (m // 128) % 8 == 0 and 192 <= (m // 1024) * s <= 256 else 1
    assert (m // 128) % rows == 0
    col_groups = n // 128 if wide else 1
    cols = 8 if n < 16 else 16
    row_tiles = m // 128
    units = -(-row_tiles // rows) * col_groups
    grid = units * s
    per_xcd = units // 8
    page_halfs = 128 * cols
    out = np.zeros(grid * nb * rows * page_halfs, dtype=slabs.dtype)
    q, g, r16, e = np.meshgrid(np.arange(4), np.arange(4), np.arange(cols), np.arange(8), indexing="ij")
    within_rows = 32 * q + 4 * g + (e % 4) + 16 * (e // 4)
    within = ((q * 4 * cols + g * cols + r16) * 8 + e).ravel()
    for unit in range(units):
        rowunit, cg = divmod(unit, col_groups)
        for sl in range(s):
            w = ((unit % per_xcd) * s + sl) * 8 + unit // per_xcd if unit < per_xcd * 8 else unit * s + sl
            for sub in range(nb * rows):
                rowtile = rowunit * rows + sub // nb
                if rowtile >= row_tiles:
                    continue
                col0 = (cg * nb + sub % nb) * 16
                block = slabs[sl, col0:col0 + cols, rowtile * 128:(rowtile + 1) * 128]   # (cols, 128)
                page = (sub * grid + w) * page_halfs
                out[page + within] = block[r16.ravel(), within_rows.ravel()]
    return out


def slabs_from_pages(pages, s, m, n, rows=None):
    """Inverse of slab_pages: (S, N, M) from the flat by-workgroup workspace."""
    index = slab_pages(np.arange(1, s * n * m + 1, dtype=np.int64).reshape(s, n, m), m, n, rows)
    used = np.flatnonzero(index)
    out = np.empty(s * n * m, dtype=pages.dtype)
    out[index[used] - 1] = pages.reshape(-1)[used]
    return out.reshape(s, n, m)
