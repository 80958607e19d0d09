"""The closed form the GPU-side compressor evaluates (flash-llm_amd/csrc/tiled_csl_device.hip), restated
in numpy and checked against the oracle's literal item-by-item drain on the CPU: an item at height h of
bank b is pop number  sum_b' max(fill[b'] - h, 0) + #{b' < b : fill[b'] >= h},  and the pop number maps
to one output index."""
import numpy as np
import pytest

ROWS, COLS, BANKS = 128, 64, 32


def keeps(bits):
    mag = bits & 0x7FFF
    return (mag != 0) & (mag <= 0x7C00)


def closed_form_tile(tile_bits):
    """tile_bits: (128, 64) uint16.  Returns the tile's packed items in output order."""
    m = np.arange(ROWS)[:, None]
    n = np.arange(COLS)[None, :]
    sw = n ^ ((m % 8) << 3)
    bank = sw >> 1
    pos = m * COLS + sw
    keep = keeps(tile_bits.astype(np.uint32))
    banks, heights, items = [], [], []
    fill = np.zeros(BANKS, dtype=np.int64)
    first_zero = np.full(BANKS, -1, dtype=np.int64)
    for b in range(BANKS):
        # scan order of the bank: row-major, its two columns of each row in ascending n
        mask = bank == b
        order = np.argsort((m * COLS + n)[mask], kind="stable")
        k = keep[mask][order]
        p = pos[mask][order]
        v = tile_bits[mask][order].astype(np.uint32)
        h = np.cumsum(k)
        banks += [b] * int(k.sum())
        heights += list(h[k])
        items += list(v[k] | (p[k].astype(np.uint32) << 16))
        fill[b] = int(k.sum())
        if (~k).any():
            first_zero[b] = int(p[~k][0])
    nnz = int(fill.sum())
    for _ in range((4 - nnz % 4) % 4):
        b = int(np.argmin(fill))  # lowest index on ties
        fill[b] += 1
        banks.append(b)
        heights.append(int(fill[b]))
        items.append(np.uint32(first_zero[b]) << np.uint32(16))
    count = int(fill.sum())
    out = np.zeros(count, dtype=np.uint32)
    vectors = count // 4
    rep, rem = vectors // BANKS, vectors % BANKS
    tail_items = rem * 4
    for b, h, item in zip(banks, heights, items):
        j = int(np.maximum(fill - h, 0).sum()) + int((fill[:b] >= h).sum())
        if j < tail_items:
            d = rep * 128 + (j % rem) * 4 + (3 - j // rem)
        else:
            q = j - tail_items
            w = rep * 4 - 1 - q // BANKS
            d = (w // 4) * 128 + (q % BANKS) * 4 + (w % 4)
        out[d] = item
    return out


def random_tile(rng, kind):
    t = np.zeros((ROWS, COLS), dtype=np.uint16)
    if kind == "uniform":
        keep = rng.random((ROWS, COLS)) < rng.choice([0.01, 0.05, 0.2, 0.5, 0.9, 1.0])
        t[keep] = rng.integers(1, 0x7C00, size=int(keep.sum()), dtype=np.uint16)
    elif kind == "few":
        c = int(rng.integers(0, 140))
        where = rng.choice(ROWS * COLS, size=c, replace=False)
        t.reshape(-1)[where] = rng.integers(1, 0x7C00, size=c, dtype=np.uint16)
    elif kind == "columns":  # a few very uneven banks
        for col in rng.choice(COLS, size=int(rng.integers(1, 6)), replace=False):
            rows = rng.choice(ROWS, size=int(rng.integers(1, ROWS + 1)), replace=False)
            t[rows, col] = rng.integers(1, 0x7C00, size=rows.size, dtype=np.uint16)
    elif kind == "specials":
        t[:] = rng.integers(0, 1 << 16, size=(ROWS, COLS), dtype=np.uint16)
        t[rng.random((ROWS, COLS)) < 0.6] = 0
        t[0, :4] = [0x8000, 0x7E00, 0x0001, 0xFC00]
    return t


@pytest.mark.parametrize("kind", ["uniform", "few", "columns", "specials"])
def test_closed_form_equals_the_sequential_drain(oracle, kind):
    rng = np.random.default_rng({"uniform": 1, "few": 2, "columns": 3, "specials": 4}[kind])
    for _ in range(12):
        tile = random_tile(rng, kind)
        _, want, offsets = oracle.compress_reorder(tile.view(np.float16))
        got = closed_form_tile(tile)
        assert got.size == want.size == int(offsets[-1]) * 4
        assert np.array_equal(got, want)
