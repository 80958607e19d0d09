"""Committed SHA-256 digests (tests/golden/digests.json, written by tests/golden/make_digests.py) of the
seeded synthetic inputs and of the Compressed_A / TileOffsets bytes: the generator, the oracle and the
product's host compressor must all still produce exactly these bytes."""
import hashlib
import json
import os

import pytest

import synth

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "digests.json")) as f:
    DIGESTS = json.load(f)


def sha(x):
    return hashlib.sha256(x.tobytes()).hexdigest()


@pytest.mark.parametrize("name", sorted(DIGESTS))
def test_bytes_match_committed_digests(oracle, product, name):
    d = DIGESTS[name]
    if d["dist"] == "normal":
        a = synth.sparse_matrix(d["M"], d["K"], d["sparsity"], d["seed"], dist="normal", sigma=0.02)
    else:
        a = synth.sparse_matrix(d["M"], d["K"], d["sparsity"], d["seed"])
    assert sha(a) == d["A_sha256"], "the synthetic generator changed"
    for variant, o_fn, p_fn in (("reorder", oracle.compress_reorder, product.init_sparse_matrix_a),
                                ("noreorder", oracle.compress_noreorder, product.init_sparse_matrix_a_noreorder)):
        want = d[variant]
        _, items, offsets = o_fn(a)
        assert items.size == want["nnz_padded"]
        assert sha(items) == want["Compressed_A_sha256"] and sha(offsets) == want["TileOffsets_sha256"], f"oracle {variant}"
        p_items, p_offsets = p_fn(a)
        assert sha(p_items) == want["Compressed_A_sha256"] and sha(p_offsets) == want["TileOffsets_sha256"], f"product {variant}"
