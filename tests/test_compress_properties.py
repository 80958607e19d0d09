"""Closed-form and cross-implementation checks of the Tiled-CSL compressors.

Independent numpy restatements of what the format fixes without reference to
any procedure (reference csrc/SpMM_API.cu:200-216 counting/padding, :349-359
TileOffsets, :439-474 scan order), plus oracle == product == Python
restatement on inputs nobody traced by hand.
"""
import numpy as np
import pytest

import py_restatement
import synth


def keeps(bits):
    mag = bits & 0x7FFF
    return (mag != 0) & (mag <= 0x7C00)


def tiles_of(a_bits):
    m, k = a_bits.shape
    return a_bits.reshape(m // 128, 128, k // 64, 64).transpose(0, 2, 1, 3).reshape(-1, 128, 64)


def closed_form_offsets(a_bits):
    nnz = keeps(tiles_of(a_bits)).reshape(-1, 128 * 64).sum(axis=1)
    vec = (nnz + 3) // 4
    off = np.concatenate([[0], np.cumsum(vec)])
    return np.concatenate([off, off[-1:]]).astype(np.int32)


def position_table():
    m = np.arange(128)[:, None]
    n = np.arange(64)[None, :]
    return (m * 64 + (n ^ ((m % 8) << 3))).astype(np.uint32)


def closed_form_noreorder(a_bits):
    """Scan order with the first `pad` dropped elements kept in place."""
    pos = position_table().reshape(-1)
    out = []
    for tile in tiles_of(a_bits):
        flat = tile.reshape(-1).astype(np.uint32)
        keep = keeps(flat)
        pad = (4 - int(keep.sum()) % 4) % 4
        dropped = np.flatnonzero(~keep)[:pad]
        keep[dropped] = True
        out.append((flat | (pos << 16))[keep])
    return np.concatenate(out) if out else np.zeros(0, np.uint32)


def special_values_matrix(seed, m=256, k=128):
    rng = np.random.default_rng(seed)
    a = synth.sparse_matrix(m, k, 0.7, seed).view(np.uint16).copy()
    specials = np.array([0x8000, 0x7E00, 0xFE00, 0x7C01, 0x0001, 0x8001, 0x7C00, 0xFC00, 0x03FF, 0x7BFF], dtype=np.uint16)
    idx = rng.integers(0, a.size, size=400)
    a.reshape(-1)[idx] = specials[rng.integers(0, specials.size, size=400)]
    return a


SHAPES = [(128, 64, 0.8), (128, 64, 0.0), (128, 64, 0.97), (256, 192, 0.5), (384, 128, 0.3), (1024, 1024, 0.8), (512, 640, 0.9)]


@pytest.mark.parametrize("m,k,sp", SHAPES)
def test_oracle_matches_closed_forms(oracle, m, k, sp):
    a = synth.sparse_matrix(m, k, sp, seed=m + k).view(np.uint16)
    n, items, offsets = oracle.compress_reorder(a)
    assert n == (m // 128) * (k // 64) + 2
    assert np.array_equal(offsets, closed_form_offsets(a))
    n2, items2, offsets2 = oracle.compress_noreorder(a)
    assert np.array_equal(offsets2, offsets)
    assert np.array_equal(items2, closed_form_noreorder(a))
    # reorder = a permutation of the kept items + padding items (value 0) at positions that hold a zero
    pos = position_table()
    t_bits = tiles_of(a)
    for t in range(t_bits.shape[0]):
        seg = items[offsets[t] * 4: offsets[t + 1] * 4]
        want = (t_bits[t].astype(np.uint32) | (pos << 16))[keeps(t_bits[t])]
        real = seg[(seg & 0xFFFF) != 0]
        pads = seg[(seg & 0xFFFF) == 0]
        assert np.array_equal(np.sort(real), np.sort(want))
        assert pads.size == (4 - want.size % 4) % 4
        dropped_positions = set(pos[~keeps(t_bits[t])].tolist())
        assert all(int(p >> 16) in dropped_positions for p in pads)
    # the scatter undoes it: kept values in place, everything else +0
    back = oracle.scatter(items, offsets, m, k)
    assert np.array_equal(back, np.where(keeps(a), a, 0))


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_special_values(oracle, product, seed):
    a = special_values_matrix(seed)
    n, items, offsets = oracle.compress_reorder(a)
    assert np.array_equal(offsets, closed_form_offsets(a))
    assert np.array_equal(oracle.scatter(items, offsets, *a.shape), np.where(keeps(a), a, 0))
    _, items2, offsets2 = oracle.compress_noreorder(a)
    assert np.array_equal(items2, closed_form_noreorder(a))
    p_items, p_offsets = product.init_sparse_matrix_a(a)
    assert np.array_equal(p_items, items) and np.array_equal(p_offsets, offsets)
    p_items2, p_offsets2 = product.init_sparse_matrix_a_noreorder(a)
    assert np.array_equal(p_items2, items2) and np.array_equal(p_offsets2, offsets2)
    py_items, py_offsets = py_restatement.compress_reorder(a)
    assert np.array_equal(py_items, items) and np.array_equal(py_offsets, offsets)


@pytest.mark.parametrize("m,k,sp,seed", [(128, 64, 0.8, 0), (128, 64, 0.2, 1), (128, 64, 0.995, 2), (256, 128, 0.6, 3), (128, 192, 0.9, 4)])
def test_three_implementations_agree(oracle, product, m, k, sp, seed):
    a = synth.sparse_matrix(m, k, sp, seed)
    _, items, offsets = oracle.compress_reorder(a)
    py_items, py_offsets = py_restatement.compress_reorder(a)
    assert np.array_equal(py_items, items) and np.array_equal(py_offsets, offsets)
    p_items, p_offsets = product.init_sparse_matrix_a(a)
    assert np.array_equal(p_items, items) and np.array_equal(p_offsets, offsets)


@pytest.mark.parametrize("m,k,sp,kw", [
    (1024, 1024, 0.8, {}),
    (2048, 1024, 0.7, {"dist": "normal"}),
    (1024, 2048, 0.9, {"dist": "normal"}),
    (1536, 768, 0.8, {"row_beta": True}),
    (512, 512, 0.0, {}),          # fully dense: 8192 items in every tile
    (512, 512, 0.3, {}),          # denser than the reference kernel's 50 % register budget
    (512, 512, 1.0, {}),          # nothing kept
    (256, 256, 0.8, {"dist": "ones"}),  # the reference's own test data: every nonzero is 1.0
])
def test_product_equals_oracle(oracle, product, m, k, sp, kw):
    a = synth.sparse_matrix(m, k, sp, seed=7, **kw)
    _, items, offsets = oracle.compress_reorder(a)
    for threads in (1, 5):
        p_items, p_offsets = product.init_sparse_matrix_a(a, threads=threads)
        assert np.array_equal(p_offsets, offsets)
        assert np.array_equal(p_items, items)
    _, items2, offsets2 = oracle.compress_noreorder(a)
    p_items2, p_offsets2 = product.init_sparse_matrix_a_noreorder(a, threads=3)
    assert np.array_equal(p_items2, items2) and np.array_equal(p_offsets2, offsets2)
    product.lib().flashllm_set_compress_threads(0)


def test_three_paddings_in_a_nearly_full_tile(oracle, product):
    """8189 nonzeros, the three zeros in one bank (bank 5): the emptiest bank is always the one that
    still has a zero, so all three padding items point at its first zero position, (0,10) -> 10.
    (A bank can only be chosen for padding while it holds fewer than 256 items, i.e. while it has a
    zero; the reference's assert at csrc/SpMM_API.cu:278 can therefore never fire.)"""
    a = np.full((128, 64), 0x3C00, dtype=np.uint16)
    a[0, 10] = a[0, 11] = a[8, 10] = 0
    n, items, offsets = oracle.compress_reorder(a)
    assert n == 3 and offsets[-1] == 2048
    pads = items[(items & 0xFFFF) == 0]
    assert [int(p) >> 16 for p in pads] == [10, 10, 10]
    p_items, _ = product.init_sparse_matrix_a(a)
    assert np.array_equal(p_items, items)
    py_items, _ = py_restatement.compress_reorder(a)
    assert np.array_equal(py_items, items)
    assert np.array_equal(oracle.scatter(items, offsets, 128, 64), a)


@pytest.mark.parametrize("m,k", [(100, 64), (128, 60), (0, 64), (128, 0), (127, 63)])
def test_bad_shapes(oracle, product, m, k):
    a = np.zeros((max(m, 1), max(k, 1)), dtype=np.uint16)[:m, :k]
    n, _, _ = oracle.compress_reorder(np.zeros((m, k), dtype=np.uint16))
    assert n == -1
    with pytest.raises(product.CompressError) as e:
        product.init_sparse_matrix_a(np.zeros((m, k), dtype=np.uint16))
    assert e.value.code == -1
    del a


def test_fp16_conversions_match_numpy(oracle):
    L = oracle.lib()
    halves = np.arange(65536, dtype=np.uint16)
    as_f32 = halves.view(np.float16).astype(np.float32)
    for h in range(0, 65536, 7):
        got = np.float32(L.oracle_half_to_float(h))
        assert got.tobytes() == as_f32[h].tobytes() or (np.isnan(got) and np.isnan(as_f32[h]))
        assert bool(L.oracle_nonzero(h)) == bool(np.abs(as_f32[h]) > 0)
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(3000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 3000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  2.0 ** -14, 2.0 ** -14 - 2.0 ** -25, 1.0009765625, 1.00048828125, 1.00146484375], dtype=np.float32),
    ])
    # exact ties between neighbouring halves
    h = rng.integers(0, 0x7BFF, 2000).astype(np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    vals = np.concatenate([vals, ((lo + hi) / 2).astype(np.float32)])
    want = vals.astype(np.float16).view(np.uint16)
    for v, w in zip(vals, want):
        assert L.oracle_float_to_half(float(v)) == w, (v, hex(w))
