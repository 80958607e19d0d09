"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle.

Tolerance on C (floating point): max|C - ref| / max|ref| <= 1e-2 and element-wise
|C - ref| <= 1e-2*|ref| + 1e-2*rms(ref), ref = fp32-accumulated product on the decompressed
weights.  Everything integer (the compressed stream the kernel consumes, the reduction of given
slabs, exact special cases) is compared bit for bit.
"""
import sys

import numpy as np
import pytest

import synth
from gpu_util import assert_close, errors, run_spmm, slab_pages, slabs_from_pages

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture
def eight_row_tiles(product):
    """Makes the N = 64 launches of a test use workgroups of eight row tiles at any size (by itself the library
    takes them only when such workgroups fill most of the GPU); restored afterwards."""
    product.lib().flashllm_hip_set_rows_per_workgroup(8)
    yield
    product.lib().flashllm_hip_set_rows_per_workgroup(0)


@pytest.fixture(scope="module")
def torch_gpu():
    import torch

    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


# --- BASELINE config 1: 1024 x 1024, 80 %, U[-1,1], N = 8, Split_K = 1, seed 0 -----------------
def test_config1_plumbing(product, oracle, torch_gpu):
    say("config1 1024x1024 N=8 split_k=1")
    a = synth.sparse_matrix(1024, 1024, 0.8, 0)
    b = synth.dense_b(1024, 8, 0)
    c, w, _ = run_spmm(product, a, b, 8, 1)
    _, items, offsets = oracle.compress_reorder(a)
    assert np.array_equal(w.comp.cpu().numpy().view(np.uint32), items)
    assert np.array_equal(w.offs.cpu().numpy(), offsets)
    model, ref = oracle.spmm_model(a, b, 8, 1)
    assert_close(c, ref, "config1")
    # against the oracle's own fp16 result the difference is summation order only
    assert np.max(np.abs(c.astype(np.float32) - model.astype(np.float32))) <= 2.0 ** -8 * np.max(np.abs(ref))


@pytest.mark.parametrize("n", [8, 16, 32, 64, 128, 256])
@pytest.mark.parametrize("split_k", [1, 3])
def test_every_supported_n(product, oracle, torch_gpu, n, split_k):
    say(f"N sweep n={n} split_k={split_k}")
    a = synth.sparse_matrix(512, 1024, 0.8, 3)
    b = synth.dense_b(1024, n, 4)
    c, _, _ = run_spmm(product, a, b, n, split_k)
    _, ref = oracle.spmm_model(a, b, n, split_k)
    assert_close(c, ref, f"n={n} split_k={split_k}")


@pytest.mark.parametrize("reorder", [True, False])
@pytest.mark.parametrize("sparsity", [0.0, 0.3, 0.5, 0.7, 0.9, 0.99, 1.0])
def test_any_density(product, oracle, torch_gpu, sparsity, reorder):
    """Tiles denser than 50 % overflow the reference kernel's register budget; here any density works."""
    say(f"density sparsity={sparsity} reorder={reorder}")
    a = synth.sparse_matrix(256, 512, sparsity, 5)
    b = synth.dense_b(512, 16, 6)
    for split_k in (1, 2):
        c, _, _ = run_spmm(product, a, b, 16, split_k, reorder=reorder)
        _, ref = oracle.spmm_model(a, b, 16, split_k)
        if sparsity == 1.0:
            assert not c.any()
        else:
            assert_close(c, ref, f"sparsity={sparsity} split_k={split_k}")


def test_ragged_tiles_and_empty_slices(product, oracle, torch_gpu):
    """Empty tiles at the start, middle and end of a slice, one-vector tiles, a full tile, and more
    slices than k tiles."""
    say("ragged tiles")
    m, k = 256, 640
    a = synth.sparse_matrix(m, k, 0.8, 8)
    a[:128, 0:64] = 0          # first tile of tile row 0 empty
    a[:128, 256:384] = 0       # two empty tiles in the middle
    a[128:, 576:640] = 0       # last tile of tile row 1 empty
    a[128:, 64:128] = 0
    a[130, 70] = 1.5           # a single nonzero: one vector with three paddings
    a[:128, 448:512] = synth.sparse_matrix(128, 64, 0.0, 9)  # a full tile
    b = synth.dense_b(k, 16, 10)
    for split_k in (1, 2, 5, 10, 16):
        c, _, _ = run_spmm(product, a, b, 16, split_k)
        _, ref = oracle.spmm_model(a, b, 16, split_k)
        assert_close(c, ref, f"ragged split_k={split_k}")


# --- N = 64 with a multiple of eight row tiles: workgroups of eight waves sharing B through LDS ------------
def eight_row_tile_matrix(seed):
    """1024 x 640: eight row tiles (one workgroup of eight waves per K slice) whose waves meet very different
    slices: a tile row without any nonzero, one with a single nonzero, empty tiles at the start, in the middle
    and at the end of a row, a full tile, a row that is dense throughout."""
    m, k = 1024, 640
    a = synth.sparse_matrix(m, k, 0.8, seed)
    a[0:128, 0:64] = 0            # tile row 0: first tile empty
    a[0:128, 256:384] = 0         #             two empty tiles in the middle
    a[128:256, :] = 0             # tile row 1: nothing at all (its wave only attends the meetings)
    a[256:384, :] = 0
    a[300, 200] = -2.5            # tile row 2: one nonzero, one vector with three paddings
    a[384:512, 576:640] = 0       # tile row 3: last tile empty
    a[512:640, 448:512] = synth.sparse_matrix(128, 64, 0.0, seed + 1)   # tile row 4: a full tile
    a[640:768, :] = synth.sparse_matrix(128, k, 0.0, seed + 2)          # tile row 5: dense throughout
    a[768:896, 64:] = 0           # tile row 6: only its first tile holds anything
    return a


def test_eight_wave_workgroups_ragged_rows_and_empty_slices(product, oracle, torch_gpu, eight_row_tiles):
    say("N=64, eight row tiles per workgroup: ragged rows")
    assert product.lib().flashllm_hip_rows_per_workgroup(64, 1024, 3) == 8
    a = eight_row_tile_matrix(60)
    b = synth.dense_b(640, 64, 61)
    for split_k in (1, 2, 3, 5, 10, 16):   # windows of two k tiles: slices of 10, 5, 4 (and 2), 2, 1 and 0 k tiles
        c, _, _ = run_spmm(product, a, b, 64, split_k)
        _, ref = oracle.spmm_model(a, b, 64, split_k)
        assert not c[:, 128:256].any()
        assert_close(c, ref, f"eight-wave ragged split_k={split_k}")


@pytest.mark.parametrize("sparsity", [0.0, 0.5, 0.8, 0.95, 0.999, 1.0])
def test_eight_wave_workgroups_any_density(product, oracle, torch_gpu, sparsity, eight_row_tiles):
    say(f"N=64, eight row tiles per workgroup: sparsity={sparsity}")
    a = synth.sparse_matrix(1024, 768, sparsity, 62)
    b = synth.dense_b(768, 64, 63)
    for split_k in (1, 3, 4):
        c, _, _ = run_spmm(product, a, b, 64, split_k)
        _, ref = oracle.spmm_model(a, b, 64, split_k)
        if sparsity == 1.0:
            assert not c.any()
        else:
            assert_close(c, ref, f"eight-wave sparsity={sparsity} split_k={split_k}")


def test_eight_wave_workgroups_match_single_wave_workgroups_bit_for_bit(product, torch_gpu):
    """Where B comes from does not change a sum: with the library told to use one row tile per workgroup (every
    wave fetching its own B fragments) C and the slabs must be the same bits."""
    torch = torch_gpu
    say("N=64: eight-wave against one-wave workgroups")
    L = product.lib()
    b_h = synth.dense_b(640, 64, 65, dist="normal")
    for a in (eight_row_tile_matrix(64), synth.sparse_matrix(2048, 640, 0.8, 66, dist="normal", sigma=0.05)):
        m, k = a.shape
        w = product.SparseWeight(a)
        b = torch.from_numpy(b_h).cuda()
        for split_k in (1, 3, 7):
            got = []
            for cap in (8, 1):
                L.flashllm_hip_set_rows_per_workgroup(cap)
                try:
                    c = torch.full((64 * m,), float("nan"), dtype=torch.float16, device="cuda")
                    ws = torch.full((split_k * 64 * m,), float("nan"), dtype=torch.float16, device="cuda")
                    product.spmm_partials(w.comp, w.offs, b, c, m, 64, k, ws, split_k)   # plain slabs: the same layout either way
                    torch.cuda.synchronize()
                    got.append((c if split_k == 1 else ws).cpu().numpy().view(np.uint16).copy())
                finally:
                    L.flashllm_hip_set_rows_per_workgroup(0)
            assert np.array_equal(got[0], got[1]), f"m={m} split_k={split_k}"


# --- the four-wave kernel for wide B (N a multiple of 128) -------------------------------------------
@pytest.mark.parametrize("n", [128, 384])
@pytest.mark.parametrize("sparsity", [0.0, 0.5, 0.72, 0.8, 0.95, 0.999, 1.0])
def test_wide_b_any_density(product, oracle, torch_gpu, sparsity, n):
    """Tiles of up to 512 vectors are held in registers two rounds at a time (three when the matrix is denser
    than about a quarter); longer ones take further rounds straight from memory.  0 % and 50 % are all long
    tiles, 72 % mixes both kinds, 99.9 % is mostly empty tiles."""
    say(f"wide B density sparsity={sparsity} n={n}")
    a = synth.sparse_matrix(384, 1280, sparsity, 41)
    b = synth.dense_b(1280, n, 42)
    for split_k in (1, 3):
        c, _, _ = run_spmm(product, a, b, n, split_k)
        _, ref = oracle.spmm_model(a, b, n, split_k)
        if sparsity == 1.0:
            assert not c.any()
        else:
            assert_close(c, ref, f"wide sparsity={sparsity} n={n} split_k={split_k}")


def test_wide_b_ragged_tiles_and_empty_slices(product, oracle, torch_gpu):
    """The wide kernel always runs whole rounds of three tiles: slices of 1, 2, 3, 4 and 0 tiles, empty tiles at
    either end, a single-vector tile and a full tile."""
    say("wide B ragged tiles")
    m, k, n = 256, 640, 256
    a = synth.sparse_matrix(m, k, 0.8, 43)
    a[:128, 0:64] = 0
    a[:128, 256:384] = 0
    a[128:, 576:640] = 0
    a[128:, 64:128] = 0
    a[130, 70] = 1.5
    a[:128, 448:512] = synth.sparse_matrix(128, 64, 0.0, 44)
    b = synth.dense_b(k, n, 45)
    for split_k in (1, 2, 3, 5, 10, 16):
        c, _, _ = run_spmm(product, a, b, n, split_k)
        _, ref = oracle.spmm_model(a, b, n, split_k)
        assert_close(c, ref, f"wide ragged split_k={split_k}")


@pytest.mark.parametrize("n,sparsity", [(128, 0.8), (256, 0.8), (256, 0.6)])
def test_wide_b_matches_the_narrow_kernel_bit_for_bit(product, torch_gpu, n, sparsity):
    """Both kernels accumulate a slice's k tiles in order with the same MFMA, so their slabs are identical:
    the columns of a wide call equal 64-column calls on its column groups.  At 60 % sparsity the wide kernel
    holds three rounds of a tile in registers instead of two (its other instantiation)."""
    torch = torch_gpu
    say(f"wide B vs narrow kernel n={n} sparsity={sparsity}")
    m, k, s = 1024, 2048, 4
    a = synth.sparse_matrix(m, k, sparsity, 46, dist="normal", sigma=0.05)
    b_h = synth.dense_b(k, n, 47, dist="normal")
    wide, w, _ = run_spmm(product, a, b_h, n, s)
    b = torch.from_numpy(b_h).cuda()
    for part in range(n // 64):
        c = torch.empty(64 * m, dtype=torch.float16, device="cuda")
        ws = torch.empty(s * 64 * m, dtype=torch.float16, device="cuda")
        product.spmm_splitk(w.comp, w.offs, b[part * 64:(part + 1) * 64].contiguous(), c, m, 64, k, ws, s)
        torch.cuda.synchronize()
        assert np.array_equal(c.cpu().numpy().view(np.uint16), wide[part * 64:(part + 1) * 64].reshape(-1).view(np.uint16))


@pytest.mark.parametrize("n", [16, 64, 128])
def test_empty_matrix_with_a_four_byte_allocation(product, torch_gpu, n):
    """A matrix without nonzeros has no items; the reference's callers then allocate a single 4-byte element
    (kernel_benchmark/spmm_test.cu:258-260).  No kernel may count on more."""
    torch = torch_gpu
    say(f"empty matrix, one-element Compressed_A, n={n}")
    m, k = 1024, 1024
    a = np.zeros((m, k), dtype=np.float16)
    items, offsets = product.init_sparse_matrix_a(a)
    assert items.size == 0 and not offsets.any()
    comp = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert comp.numel() * comp.element_size() == 4
    offs = torch.from_numpy(offsets).cuda()
    b = torch.from_numpy(synth.dense_b(k, n, 48)).cuda()
    for split_k in (1, 3):
        c = torch.full((n * m,), float("nan"), dtype=torch.float16, device="cuda")
        ws = torch.full((split_k * n * m,), float("nan"), dtype=torch.float16, device="cuda")
        product.spmm_splitk(comp, offs, b, c, m, n, k, ws, split_k)
        torch.cuda.synchronize()
        assert not c.cpu().numpy().view(np.uint16).any()


def test_ones_matrix_subset_sums(product, oracle, torch_gpu):
    """The reference benchmark's data (A in {0,1}, B in fifths): small exact sums."""
    say("ones matrix")
    m, n, k = 256, 8, 256
    a = synth.sparse_matrix(m, k, 0.8, 3, dist="ones")
    b = (np.random.default_rng(0).integers(0, 5, size=(n, k)) / 4 - 0.5).astype(np.float16)  # quarters: exact in fp16/fp32
    c, _, _ = run_spmm(product, a, b, n, 1)
    want = (b.astype(np.float32) @ a.astype(np.float32).T).astype(np.float16)
    assert np.array_equal(c, want)


def test_scaled_permutation_exact(product, torch_gpu):
    say("permutation")
    k = m = 512
    perm = np.random.default_rng(1).permutation(k)
    a = np.zeros((m, k), dtype=np.float16)
    a[np.arange(m), perm] = 2.0
    b = synth.dense_b(k, 32, 5)
    for split_k in (1, 4):
        c, _, _ = run_spmm(product, a, b, 32, split_k)
        assert np.array_equal(c, b[:, perm] * np.float16(2.0))


def test_special_values_flow_through(product, oracle, torch_gpu):
    """-0 and NaN in A are dropped by the compressor, so C stays finite; Inf propagates."""
    say("special values")
    a = synth.sparse_matrix(128, 128, 0.8, 11)
    bits = a.view(np.uint16)
    bits[3, 5] = 0x7E00   # NaN: dropped
    bits[4, 6] = 0x8000   # -0: dropped
    b = np.abs(synth.dense_b(128, 8, 12)) + np.float16(0.5)
    c, _, _ = run_spmm(product, a, b, 8, 1)
    assert np.all(np.isfinite(c))
    dec = oracle.scatter(*oracle.compress_reorder(a)[1:], 128, 128).view(np.float16)
    _, ref = oracle.spmm_model(dec, b, 8, 1)
    assert_close(c, ref, "specials")
    bits[7, 9] = 0x7C00   # +Inf: kept
    c, _, _ = run_spmm(product, a, b, 8, 1)
    assert np.all(np.isinf(c[:, 7])) and np.all(np.isfinite(np.delete(c, 7, axis=1)))


def test_split_k_reduction_bit_exact(product, oracle, torch_gpu):
    torch = torch_gpu
    say("reduction kernel")
    rng = np.random.default_rng(2)
    # plain slabs; the last two shapes are outside the SpMM kernel's (M % 128, N) grid
    for m, n, s in [(128, 8, 2), (1024, 16, 7), (256, 64, 32), (384, 8, 5), (2048, 32, 9), (1024, 128, 3), (256, 256, 11),
                    (100, 8, 3), (128, 20, 6)]:
        ws_h = (rng.standard_normal((s, n * m)) * 3).astype(np.float16)
        ws = torch.from_numpy(ws_h).cuda()
        c = torch.zeros(n * m, dtype=torch.float16, device="cuda")
        product.splitk_reduce(c, ws, m, n, s)
        torch.cuda.synchronize()
        want = oracle.splitk_reduce(ws_h, n * m, s)
        assert np.array_equal(c.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_split_k_reduction_of_slabs_by_workgroup_bit_exact(product, oracle, torch_gpu):
    """The same sums when the slabs lie in the order the library's own two kernels use: random slabs are put
    into that order on the host (from the layout's description) and must reduce to the oracle's C."""
    torch = torch_gpu
    rng = np.random.default_rng(21)
    # 8 and 16 row tiles fill whole XCD rounds, 1 / 3 / 11 leave units beyond a multiple of eight
    for m, n, s in [(128, 8, 2), (1024, 16, 7), (256, 64, 32), (384, 8, 5), (2048, 32, 9), (1024, 128, 3), (256, 256, 11),
                    (1408, 16, 4), (1408, 64, 3), (1024, 64, 5), (512, 32, 3), (1536, 64, 2), (3072, 32, 4)]:
        say(f"reduction of pages m={m} n={n} s={s}")
        ws_h = (rng.standard_normal((s, n * m)) * 3).astype(np.float16)
        ws = torch.from_numpy(slab_pages(ws_h, m, n)).cuda()
        c = torch.full((n * m,), float("nan"), dtype=torch.float16, device="cuda")
        product.splitk_reduce(c, ws, m, n, s, slab_order=product.SLABS_BY_WORKGROUP)
        torch.cuda.synchronize()
        want = oracle.splitk_reduce(ws_h, n * m, s)
        assert np.array_equal(c.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_split_k_reduction_of_pages_of_eight_row_tile_workgroups_bit_exact(product, oracle, torch_gpu, eight_row_tiles):
    """The same for the pages N = 64 launches leave when their workgroups take eight row tiles each: one unit
    (1024 rows), three (units beyond whole XCD rounds), eight and nine."""
    torch = torch_gpu
    rng = np.random.default_rng(22)
    for m, s in [(1024, 5), (3072, 2), (8192, 3), (9216, 28)]:
        say(f"reduction of pages, eight row tiles per workgroup, m={m} s={s}")
        n = 64
        ws_h = (rng.standard_normal((s, n * m)) * 3).astype(np.float16)
        ws = torch.from_numpy(slab_pages(ws_h, m, n, rows=8)).cuda()
        c = torch.full((n * m,), float("nan"), dtype=torch.float16, device="cuda")
        product.splitk_reduce(c, ws, m, n, s, slab_order=product.SLABS_BY_WORKGROUP)
        torch.cuda.synchronize()
        want = oracle.splitk_reduce(ws_h, n * m, s)
        assert np.array_equal(c.cpu().numpy().view(np.uint16), want.view(np.uint16))


def test_workgroups_go_round_robin_over_the_xcds(product, torch_gpu):
    """The placement of slices and of the reduction's workgroups counts on workgroup w running on XCD w % 8.
    Results never depend on it (the reduction is a separate kernel), only where its loads hit."""
    say("xcd probe")
    ids = product.xcd_of_workgroups(2016)
    assert ids.max() < 8
    distinct = len(set(ids.tolist()))
    same_as_first_round = float(np.mean(ids == ids[np.arange(ids.size) % 8]))
    say(f"  {distinct} XCD ids; share of workgroups on the XCD of workgroup w % 8: {same_as_first_round:.3f}")
    assert distinct in (1, 2, 4, 8)  # whole GPU, or one of its partition modes


@pytest.mark.parametrize("m,n,k,s", [(512, 16, 1024, 4), (1152, 8, 512, 3), (1280, 64, 512, 2), (384, 128, 768, 3),
                                     (2048, 32, 1536, 5), (1536, 64, 448, 4)])
def test_partials_then_reduce_equals_api(product, oracle, torch_gpu, m, n, k, s):
    check_partials_then_reduce(product, oracle, torch_gpu, m, n, k, s, None)


@pytest.mark.parametrize("m,n,k,s", [(1024, 64, 1024, 3), (2048, 64, 1280, 5)])
def test_partials_then_reduce_equals_api_eight_row_tile_workgroups(product, oracle, torch_gpu, eight_row_tiles, m, n, k, s):
    check_partials_then_reduce(product, oracle, torch_gpu, m, n, k, s, 8)


def check_partials_then_reduce(product, oracle, torch_gpu, m, n, k, s, rows):
    """Both slab orders hold the same partial sums (each the oracle's product over its K slice), and the
    two halves called separately give the API's C in either order."""
    torch = torch_gpu
    say(f"partials + reduce m={m} n={n} k={k} s={s}")
    a = synth.sparse_matrix(m, k, 0.8, 13)
    b_h = synth.dense_b(k, n, 14)
    c_api, w, ws_api = run_spmm(product, a, b_h, n, s)
    b = torch.from_numpy(b_h).cuda()
    ws = torch.full((s * n * m,), float("nan"), dtype=torch.float16, device="cuda")
    c = torch.zeros(n * m, dtype=torch.float16, device="cuda")
    product.spmm_partials(w.comp, w.offs, b, c, m, n, k, ws, s)
    torch.cuda.synchronize()
    slabs = ws.cpu().numpy().reshape(s, n, m)
    # the API call left the same numbers, by workgroup
    assert np.array_equal(slabs.view(np.uint16), slabs_from_pages(ws_api.cpu().numpy(), s, m, n, rows).view(np.uint16))
    for i, (kb, ke) in enumerate(oracle.splitk_ranges(k, s)):
        _, ref = oracle.spmm_model(np.ascontiguousarray(a[:, kb * 64:ke * 64]), np.ascontiguousarray(b_h[:, kb * 64:ke * 64]), n, 1)
        assert_close(slabs[i], ref, f"slab {i}")
    product.splitk_reduce(c, ws, m, n, s)
    torch.cuda.synchronize()
    assert np.array_equal(c.cpu().numpy().view(np.uint16), c_api.reshape(-1).view(np.uint16))
    assert np.array_equal(c_api.reshape(-1).view(np.uint16), oracle.splitk_reduce(slabs.reshape(s, -1), n * m, s).view(np.uint16))
    # and the two halves in the library's own order
    ws2 = torch.full((s * n * m,), float("nan"), dtype=torch.float16, device="cuda")
    c2 = torch.full((n * m,), float("nan"), dtype=torch.float16, device="cuda")
    product.spmm_partials(w.comp, w.offs, b, c2, m, n, k, ws2, s, slab_order=product.SLABS_BY_WORKGROUP)
    product.splitk_reduce(c2, ws2, m, n, s, slab_order=product.SLABS_BY_WORKGROUP)
    torch.cuda.synchronize()
    assert np.array_equal(ws2.cpu().numpy().view(np.uint16), ws_api.cpu().numpy().view(np.uint16))
    assert np.array_equal(c2.cpu().numpy().view(np.uint16), c_api.reshape(-1).view(np.uint16))


def test_runs_on_a_side_stream_and_is_repeatable(product, oracle, torch_gpu):
    torch = torch_gpu
    say("side stream")
    m, n, k, s = 512, 16, 512, 2
    a = synth.sparse_matrix(m, k, 0.8, 15)
    b_h = synth.dense_b(k, n, 16)
    w = product.SparseWeight(a)
    b = torch.from_numpy(b_h).cuda()
    ws = torch.empty(s * n * m, dtype=torch.float16, device="cuda")
    outs = []
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    for _ in range(3):
        c = torch.empty(n * m, dtype=torch.float16, device="cuda")
        with torch.cuda.stream(stream):
            w.matmul(b, n, c=c, workspace=ws, split_k=s, stream=stream)
        stream.synchronize()
        outs.append(c.cpu().numpy())
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[1], outs[2])
    _, ref = oracle.spmm_model(a, b_h, n, s)
    assert_close(outs[0].reshape(n, m), ref, "side stream")


# --- BASELINE config 2: 9216 x 9216, 80 %, N = 16, Split_K in {1,2,4,8} -------------------------
def test_config2_skinny(product, oracle, torch_gpu):
    say("config2 generate")
    m = k = 9216
    a = synth.sparse_matrix(m, k, 0.8, 0)
    b = synth.dense_b(k, 16, 0)
    say("config2 oracle compress")
    _, items, offsets = oracle.compress_reorder(a)
    ref, _ = oracle.gemm_f32(a, b, 16)
    for split_k in (1, 2, 4, 8):
        say(f"config2 split_k={split_k}")
        c, w, _ = run_spmm(product, a, b, 16, split_k)
        if split_k == 1:
            assert np.array_equal(w.comp.cpu().numpy().view(np.uint32), items)
            assert np.array_equal(w.offs.cpu().numpy(), offsets)
        assert_close(c, ref, f"config2 split_k={split_k}")


# --- the headline shape: 36864 x 9216, 80 %, N(0, 0.02) weights, N(0,1) activations, N = 16 -----
def test_headline_shape(product, oracle, torch_gpu):
    m, k, n = 36864, 9216, 16
    say("headline generate")
    a = synth.sparse_matrix(m, k, 0.8, 0, dist="normal", sigma=0.02, threads=16)
    b = synth.dense_b(k, n, 0, dist="normal")
    say("headline reference gemm")
    ref, _ = oracle.gemm_f32(a, b, n)
    s = product.splitk_heuristic(m, n, k)
    for split_k in sorted({1, 3, s}):
        say(f"headline split_k={split_k}")
        c, w, _ = run_spmm(product, a, b, n, split_k)
        assert_close(c, ref, f"headline split_k={split_k}")
    say("headline round trip of the compressed stream")
    back = oracle.scatter(w.comp.cpu().numpy().view(np.uint32)[:w.nnz], w.offs.cpu().numpy(), m, k)
    bits = a.view(np.uint16)
    mag = bits & 0x7FFF
    assert np.array_equal(back, np.where((mag != 0) & (mag <= 0x7C00), bits, 0))
    # linearity in B (a size-independent property): A(b1 + b2) vs A b1 + A b2
    b2 = synth.dense_b(k, n, 1, dist="normal")
    bsum = (b.astype(np.float32) + b2.astype(np.float32)).astype(np.float16)
    c1, _, _ = run_spmm(product, a, b, n, s)
    c2, _, _ = run_spmm(product, a, b2, n, s)
    c12, _, _ = run_spmm(product, a, bsum, n, s)
    rel, _ = errors(c12, c1.astype(np.float32) + c2.astype(np.float32))
    assert rel <= 2e-2


# --- config 4 flavour: non-uniform rows, N = 32 --------------------------------------------------
def test_nonuniform_rows(product, oracle, torch_gpu):
    say("non-uniform rows")
    m, k, n = 3072, 3072, 32
    a = synth.sparse_matrix(m, k, 0.8, 2, dist="normal", row_beta=True)
    b = synth.dense_b(k, n, 3, dist="normal")
    ref, _ = oracle.gemm_f32(a, b, n)
    for split_k in (1, 6):
        c, _, _ = run_spmm(product, a, b, n, split_k)
        assert_close(c, ref, f"beta rows split_k={split_k}")


# --- config 5 flavour: the four linears of a decoder layer, chained --------------------------------
def test_decoder_layer_chain_eight_row_tile_workgroups(product, oracle, torch_gpu, eight_row_tiles):
    """64 tokens at hidden 1024 through the eight-wave workgroups of N = 64, the attention-output linear with B read
    in place at leading dimension 3072."""
    test_decoder_layer_chain(product, oracle, torch_gpu, 64, 1024)


@pytest.mark.parametrize("tokens,hidden", [(16, 512), (256, 512), (64, 1024)])
def test_decoder_layer_chain(product, oracle, torch_gpu, tokens, hidden):
    """QKV -> (first hidden rows) -> attention output -> FFN1 -> ReLU -> FFN2 on one stream with one
    workspace; every stage is checked against an fp32 product of the previous stage's fp16 output.
    tokens = 256 exercises the reference's fallback to Split_K = 1 (ft.patch:523, :1454); 64 tokens at hidden 1024 take
    the eight-wave workgroups of N = 64, the attention-output linear with B read in place at leading dimension 3072."""
    torch = torch_gpu
    say(f"decoder layer chain tokens={tokens} hidden={hidden}")
    shapes = [(3 * hidden, hidden), (hidden, hidden), (4 * hidden, hidden), (hidden, 4 * hidden)]
    dense = [synth.sparse_matrix(m, k, 0.8, 20 + i, dist="normal", sigma=0.05) for i, (m, k) in enumerate(shapes)]
    weights = [product.SparseWeight(a) for a in dense]
    layer = product.DecoderLayer(*weights)
    x_h = synth.dense_b(hidden, tokens, 30, dist="normal")
    x = torch.from_numpy(x_h).cuda()
    # with the optional contiguous copy of the attention-output linear's input, then without (the linear reads
    # qkv_out in place either way): every buffer must come out the same
    y, bufs = layer.forward(x, tokens, copy_attn_in=True)
    torch.cuda.synchronize()
    first = [b.clone() for b in bufs]
    for b in bufs:
        b.fill_(float("nan"))
    y, bufs = layer.forward(x, tokens, buffers=bufs)
    torch.cuda.synchronize()
    assert torch.isnan(bufs[1]).all()   # not written without copy_attn_in
    for i in (0, 2, 3, 4):
        assert torch.equal(bufs[i].view(torch.int16), first[i].view(torch.int16)), i
    qkv, attn_in, attn_out, ffn_mid, y = [b.cpu().numpy() for b in first]
    qkv = qkv.reshape(tokens, 3 * hidden)
    ref, _ = oracle.gemm_f32(dense[0], x_h, tokens)
    assert_close(qkv, ref, "qkv")
    attn_in = attn_in.reshape(tokens, hidden)
    assert np.array_equal(attn_in.view(np.uint16), np.ascontiguousarray(qkv[:, :hidden]).view(np.uint16))
    ref, _ = oracle.gemm_f32(dense[1], attn_in, tokens)
    attn_out = attn_out.reshape(tokens, hidden)
    assert_close(attn_out, ref, "attention output")
    ref, _ = oracle.gemm_f32(dense[2], attn_out, tokens)
    ffn_mid = ffn_mid.reshape(tokens, 4 * hidden)
    assert np.all(ffn_mid >= 0)
    assert_close(ffn_mid, np.maximum(ref, 0), "ffn1 + relu")
    ref, _ = oracle.gemm_f32(dense[3], ffn_mid, tokens)
    assert_close(y.reshape(tokens, hidden), ref, "ffn2")


def test_decoder_layer_rejects_shapes_that_do_not_chain(product, torch_gpu):
    torch = torch_gpu
    a = synth.sparse_matrix(256, 128, 0.8, 1)
    w = product.SparseWeight(a)
    layer = product.DecoderLayer(w, w, w, w)  # attention output expects k == hidden == 128 but ffn1.k != attn_out.m
    x = torch.zeros(128 * 16, dtype=torch.float16, device="cuda")
    with pytest.raises(product.HipError) as e:
        layer.forward(x, 16)
    assert e.value.code == 1


def test_seeded_random_shapes(product, oracle, torch_gpu):
    """Forty seeded draws of (M, K, N, Split_K, sparsity) over everything the API dispatches on, including row-tile
    counts that are no multiple of eight (units beyond whole XCD rounds), slices longer and shorter than the
    k tiles there are, and both kernels; each against the oracle's product on the same operands."""
    rng = np.random.default_rng(20240607)
    for case in range(40):
        m = 128 * int(rng.integers(1, 14))
        k = 64 * int(rng.integers(1, 25))
        n = int(rng.choice([8, 16, 32, 64, 128, 256]))
        split_k = int(rng.integers(1, min(9, k // 64) + 1))
        sparsity = float(rng.choice([0.5, 0.7, 0.8, 0.9, 0.97]))
        say(f"random case {case}: M={m} K={k} N={n} split_k={split_k} sparsity={sparsity}")
        a = synth.sparse_matrix(m, k, sparsity, 1000 + case)
        b = synth.dense_b(k, n, 2000 + case)
        c, _, _ = run_spmm(product, a, b, n, split_k)
        _, ref = oracle.spmm_model(a, b, n, split_k)
        assert_close(c, ref, f"case {case}")


def test_call_can_be_captured_in_a_graph_and_replayed(product, oracle, torch_gpu):
    """SpMM_SplitK_API allocates nothing and never waits for the host, so a caller may record it into a HIP graph.
    Replays, with other work and new contents of B between them, must each equal the eager result bit for bit."""
    torch = torch_gpu
    say("graph capture")
    m, n, k, s = 1024, 16, 2048, 5
    a = synth.sparse_matrix(m, k, 0.8, 31)
    w = product.SparseWeight(a)
    b = torch.zeros(n * k, dtype=torch.float16, device="cuda")
    c = torch.zeros(n * m, dtype=torch.float16, device="cuda")
    ws = torch.zeros(s * n * m, dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):   # one eager call first, as graph capture wants its kernels loaded already
        w.matmul(b, n, c=c, workspace=ws, split_k=s, stream=side)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        w.matmul(b, n, c=c, workspace=ws, split_k=s, stream=torch.cuda.current_stream())
    for rep in range(4):
        b_h = synth.dense_b(k, n, 40 + rep)
        b.copy_(torch.from_numpy(b_h).reshape(-1))
        ws.fill_(float("nan"))
        c.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = c.cpu().numpy().copy()
        eager = torch.full((n * m,), float("nan"), dtype=torch.float16, device="cuda")
        w.matmul(b, n, c=eager, workspace=ws, split_k=s)
        torch.cuda.synchronize()
        assert np.array_equal(got.view(np.uint16), eager.cpu().numpy().view(np.uint16)), f"replay {rep}"
        _, ref = oracle.spmm_model(a, b_h, n, s)
        assert_close(got.reshape(n, m), ref, f"replay {rep}")
