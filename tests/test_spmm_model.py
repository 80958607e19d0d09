"""Pins the numerical model of SpMM + split-K (oracle_spmm_model, oracle_splitk_reduce,
oracle_gemm_f32, oracle_splitk_ranges) against what the mathematics fixes."""
import numpy as np
import pytest

import synth


def brute_f64(a, b):
    """a: (M,K) fp16, b: (N,K) fp16 -> (N,M) float64, exact products summed in float64."""
    return b.astype(np.float64) @ a.astype(np.float64).T


@pytest.mark.parametrize("m,n,k,sp", [(256, 8, 128, 0.8), (128, 16, 64, 0.5), (256, 32, 256, 0.9)])
def test_model_vs_float64(oracle, m, n, k, sp):
    a = synth.sparse_matrix(m, k, sp, 1)
    b = synth.dense_b(k, n, 2)
    c16, c32 = oracle.spmm_model(a, b, n, 1)
    ref = brute_f64(a, b)
    # fp32 accumulation of K exact products: error <= K * eps32 * sum|a||b|
    bound = k * 2.0 ** -24 * (np.abs(b.astype(np.float64)) @ np.abs(a.astype(np.float64)).T)
    assert np.all(np.abs(c32 - ref) <= bound + 1e-30)
    assert np.array_equal(c16, c32.astype(np.float16))
    g, threads = oracle.gemm_f32(a, b, n)
    assert threads >= 1 and np.array_equal(g, c32)


def test_ones_matrix_is_subset_sum(oracle):
    """The reference's own test data (kernel_benchmark/spmm_test_utils.h:103-118): A in {0,1},
    B in {-0.5,-0.3,-0.1,0.1,0.3}: C[m][n] = sum of B[k][n] over the kept k of row m."""
    m, n, k = 256, 8, 192
    a = synth.sparse_matrix(m, k, 0.8, 3, dist="ones")
    rng = np.random.default_rng(0)
    b = (rng.integers(0, 5, size=(n, k)) / 5 - 0.5).astype(np.float16)
    c16, c32 = oracle.spmm_model(a, b, n, 1)
    for row in (0, 17, 255):
        kept = np.flatnonzero(a[row] != 0)
        want = np.float32(0)
        for kk in kept:
            want = np.float32(want + np.float32(b[3, kk]))
        assert c32[3, row] == want


def test_scaled_permutation_is_exact(oracle):
    """A = 2 * permutation: every output is one product, so C = 2 * B[perm] exactly, for any Split_K."""
    k = m = 256
    perm = np.random.default_rng(1).permutation(k)
    a = np.zeros((m, k), dtype=np.float16)
    a[np.arange(m), perm] = 2.0
    b = synth.dense_b(k, 16, 5)
    for s in (1, 2, 4):
        c16, _ = oracle.spmm_model(a, b, 16, s)
        assert np.array_equal(c16, (b[:, perm] * np.float16(2.0)))


def test_splitk_ranges(oracle):
    assert oracle.splitk_ranges(9216, 3) == [(0, 48), (48, 96), (96, 144)]
    assert oracle.splitk_ranges(9216, 7) == [(0, 21), (21, 42), (42, 63), (63, 84), (84, 105), (105, 126), (126, 144)]
    # the reference's formula (csrc/SpMM_Kernel.cuh:196-204): Avg = ceil(16/3) = 6, last = 6 - (18-16) = 4
    assert oracle.splitk_ranges(1024, 3) == [(0, 6), (6, 12), (12, 16)]
    # more slices than k tiles: the surplus slices are empty
    assert oracle.splitk_ranges(128, 4) == [(0, 1), (1, 2), (2, 2), (2, 2)]
    for k, s in [(1024, 1), (1024, 5), (4096, 8), (640, 3)]:
        r = oracle.splitk_ranges(k, s)
        assert r[0][0] == 0 and r[-1][1] == k // 64
        assert all(r[i][1] == r[i + 1][0] for i in range(s - 1))


@pytest.mark.parametrize("s", [2, 3, 8])
def test_splitk_model_rounds_partials(oracle, s):
    m, n, k = 128, 8, 1024
    a = synth.sparse_matrix(m, k, 0.8, 9)
    b = synth.dense_b(k, n, 10)
    c16, c32 = oracle.spmm_model(a, b, n, s)
    acc = np.zeros((n, m), dtype=np.float32)
    whole = np.zeros((n, m), dtype=np.float32)
    for kb, ke in oracle.splitk_ranges(k, s):
        part, _ = oracle.spmm_model(np.ascontiguousarray(a[:, kb * 64:ke * 64]), np.ascontiguousarray(b[:, kb * 64:ke * 64]), n, 1) \
            if ke > kb else (np.zeros((n, m), np.float16), None)
        acc = acc + part.astype(np.float32)
    assert np.array_equal(c16, acc.astype(np.float16))
    # and it stays within fp16 rounding of the un-split product
    ref = brute_f64(a, b)
    assert np.max(np.abs(c16.astype(np.float64) - ref)) <= 1e-2 * np.max(np.abs(ref))


def test_reduce_closed_form(oracle):
    rng = np.random.default_rng(4)
    mn, s = 2048, 5
    ws = rng.standard_normal((s, mn)).astype(np.float16)
    got = oracle.splitk_reduce(ws, mn, s)
    # <= 2048 fp16 addends are summed exactly enough in fp32 that float64 rounding once agrees
    want = ws.astype(np.float32)
    acc = np.zeros(mn, dtype=np.float32)
    for i in range(s):
        acc = acc + want[i]
    assert np.array_equal(got, acc.astype(np.float16))


def test_slab_page_layout_helper_is_a_bijection_with_known_corners():
    """The host-side statement of the by-workgroup slab order that the GPU tests lay random slabs out with:
    a permutation of the S*N*M halfs, and a few entries placed by hand from the layout's description."""
    from gpu_util import slab_pages, slabs_from_pages

    for m, n, s in [(128, 8, 2), (1024, 16, 7), (1408, 64, 3), (256, 256, 11), (384, 128, 3), (1024, 64, 3), (2048, 32, 5), (512, 32, 2), (1536, 64, 4), (36864, 64, 7)]:
        x = np.arange(s * n * m, dtype=np.int64).reshape(s, n, m)
        p = slab_pages(x, m, n)
        assert np.array_equal(np.sort(p), np.arange(s * n * m))
        assert np.array_equal(slabs_from_pages(p, s, m, n), x)
        if n == 64 and m % 1024 == 0:   # the layout of workgroups of eight row tiles, whatever their number
            p = slab_pages(x, m, n, rows=8)
            assert np.array_equal(np.sort(p), np.arange(s * n * m))
            assert np.array_equal(slabs_from_pages(p, s, m, n, rows=8), x)
    # M = 1024 (8 row tiles = one per XCD), N = 16, S = 7: unit u, slice sl is workgroup sl*8 + u; its 4 KB page starts
    # at 2048 halfs * workgroup; piece q*64 + g*16 + r = rows 32q+4g.. and 32q+16+4g.. of column r
    m, n, s = 1024, 16, 7
    x = np.arange(s * n * m, dtype=np.int64).reshape(s, n, m)
    p = slab_pages(x, m, n)
    assert p[0] == x[0, 0, 0] and p[3] == x[0, 0, 3] and p[4] == x[0, 0, 16]
    assert p[8] == x[0, 1, 0]                                # piece 1: column 1
    assert p[16 * 8] == x[0, 0, 4]                           # piece 16: g = 1
    assert p[64 * 8] == x[0, 0, 32]                          # piece 64: q = 1
    assert p[2048 * 1] == x[0, 0, 128]                       # workgroup 1 = unit 1 (row tile 1), slice 0
    assert p[2048 * 8] == x[1, 0, 0]                         # workgroup 8 = unit 0, slice 1
    assert p[2048 * (6 * 8 + 5) + 8 * (2 * 64 + 3 * 16 + 9) + 6] == x[6, 9, 5 * 128 + 64 + 16 + 12 + 2]
    # M = 2048 (16 row tiles), N = 64, S = 3: workgroups of 8 row tiles, so 2 units (fewer than 8: workgroup =
    # unit*S + slice) and a launch of G = 6 workgroups; a unit's 32 pages are (row tile r, block b) -> sub = 4r + b
    # at page sub*G + workgroup
    m, n, s = 2048, 64, 3
    x = np.arange(s * n * m, dtype=np.int64).reshape(s, n, m)
    p = slab_pages(x, m, n, rows=8)
    assert p[0] == x[0, 0, 0]
    assert p[2048 * (1 * 6 + 0)] == x[0, 16, 0]              # sub 1: row tile 0, columns 16..31
    assert p[2048 * (4 * 6 + 0)] == x[0, 0, 128]             # sub 4: row tile 1, columns 0..15
    assert p[2048 * (0 * 6 + 1)] == x[1, 0, 0]               # workgroup 1 = unit 0, slice 1
    assert p[2048 * (0 * 6 + 3)] == x[0, 0, 8 * 128]         # workgroup 3 = unit 1 (row tiles 8..15), slice 0
    assert p[2048 * (31 * 6 + 5) + 8 * 17 + 1] == x[2, 48 + 1, 15 * 128 + 4 + 1]   # last page: piece 17 = g 1, column 1
