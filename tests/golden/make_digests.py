#!/usr/bin/env python3
"""Writes tests/golden/digests.json: SHA-256 of Compressed_A and TileOffsets as the CPU oracle emits
them for seeded synthetic matrices (the BASELINE plumbing shape and a few smaller ones).  The digests
are regression anchors for the generator + oracle + product trio across changes; what pins the
oracle to the reference's algorithm are the hand-traced cases in reorder_kat.py.

    python tests/golden/make_digests.py
"""
import hashlib
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for sub in ("flash-llm_amd", "oracle"):
    sys.path.insert(0, os.path.join(ROOT, sub))

import oracle  # noqa: E402
import synth  # noqa: E402

CASES = [
    # name, M, K, sparsity, seed, dist
    ("config1_1024x1024_s80_seed0", 1024, 1024, 0.8, 0, "uniform"),
    ("ffn_like_2048x1024_s70_seed1", 2048, 1024, 0.7, 1, "normal"),
    ("ffn_like_1024x2048_s90_seed2", 1024, 2048, 0.9, 2, "normal"),
    ("dense_256x128_s0_seed3", 256, 128, 0.0, 3, "uniform"),
    ("nearly_empty_256x256_s999_seed4", 256, 256, 0.999, 4, "uniform"),
]


def matrix(m, k, sparsity, seed, dist):
    if dist == "normal":
        return synth.sparse_matrix(m, k, sparsity, seed, dist="normal", sigma=0.02)
    return synth.sparse_matrix(m, k, sparsity, seed)


def digests():
    out = {}
    for name, m, k, sp, seed, dist in CASES:
        a = matrix(m, k, sp, seed, dist)
        entry = {"M": m, "K": k, "sparsity": sp, "seed": seed, "dist": dist,
                 "A_sha256": hashlib.sha256(a.tobytes()).hexdigest()}
        for variant, fn in (("reorder", oracle.compress_reorder), ("noreorder", oracle.compress_noreorder)):
            _, items, offsets = fn(a)
            entry[variant] = {"nnz_padded": int(items.size),
                              "Compressed_A_sha256": hashlib.sha256(items.tobytes()).hexdigest(),
                              "TileOffsets_sha256": hashlib.sha256(offsets.tobytes()).hexdigest()}
        out[name] = entry
    return out


if __name__ == "__main__":
    with open(os.path.join(HERE, "digests.json"), "w") as f:
        json.dump(digests(), f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", os.path.join(HERE, "digests.json"))
