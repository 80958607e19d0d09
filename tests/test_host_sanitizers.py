"""The host compressors and the .bin exporter under AddressSanitizer and UndefinedBehaviorSanitizer
(`make -C flash-llm_amd asan`, a host-only build of csrc/tiled_csl_compress.cpp and csrc/bin_export.cpp with the
driver tests/cxx/asan_compress.cpp): every known-answer tile, the special-value patterns, dense, empty and
ragged matrices go through both compressors (one and three worker threads) and the exporter; a sanitizer report
ends the driver with a non-zero code, and what it wrote is compared with the oracle's bytes."""
import os
import subprocess

import numpy as np
import pytest

import synth
from golden import reorder_kat as kat

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "cxx", "asan_compress.bin")


@pytest.fixture(scope="module")
def driver():
    sources = [os.path.join(ROOT, "tests", "cxx", "asan_compress.cpp"), os.path.join(ROOT, "flash-llm_amd", "csrc", "tiled_csl_compress.cpp"),
               os.path.join(ROOT, "flash-llm_amd", "csrc", "bin_export.cpp")]
    if not os.path.exists(EXE) or any(os.path.getmtime(EXE) < os.path.getmtime(s) for s in sources):
        r = subprocess.run(["make", "-C", os.path.join(ROOT, "flash-llm_amd"), "asan"], capture_output=True, text=True)
        assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    return EXE


def special_values():
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 1 << 16, size=(256, 128), dtype=np.uint16)
    bits = np.where(rng.random((256, 128)) < 0.3, bits, np.uint16(0))
    bits[0, :8] = [0x8000, 0x7E00, 0xFE00, 0x7C00, 0xFC00, 0x0001, 0x8001, 0x7C01]
    return bits.view(np.float16)


def one_column():
    a = np.zeros((128, 64), dtype=np.float16)
    a[:, 5] = 1.0   # 128 items in two banks: very uneven levels, padding in banks that hold nothing
    a[3, 9] = 2.0
    return a


MATRICES = {f"kat_{name}": (lambda name=name: kat.build_matrix(kat.CASES[name])) for name in sorted(kat.CASES)}
MATRICES.update({f"kat_noreorder_{name}": (lambda name=name: kat.build_matrix(kat.NOREORDER_CASES[name])) for name in sorted(kat.NOREORDER_CASES)})
MATRICES.update({
    "special_values": special_values,
    "one_column": one_column,
    "empty": lambda: np.zeros((256, 192), dtype=np.float16),
    "dense": lambda: synth.sparse_matrix(128, 128, 0.0, 5),
    "random_80": lambda: synth.sparse_matrix(384, 320, 0.8, 6),
    "random_999": lambda: synth.sparse_matrix(256, 256, 0.999, 7),
})


def read_stream(path):
    raw = np.fromfile(path, dtype=np.int32)
    n = int(raw[0])
    return raw[1:1 + n], raw[1 + n:].view(np.uint32)


@pytest.mark.parametrize("name", sorted(MATRICES))
def test_compressors_and_exporter_under_sanitizers(driver, oracle, tmp_path, name):
    a = np.ascontiguousarray(MATRICES[name]()).view(np.float16)
    m, k = a.shape
    dense = str(tmp_path / "dense.bin")
    a.tofile(dense)
    prefix = str(tmp_path / "out")
    r = subprocess.run([driver, dense, str(m), str(k), prefix], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, f"{name}: exit {r.returncode}\n{r.stdout[-1000:]}\n{r.stderr[-3000:]}"
    _, items, offsets = oracle.compress_reorder(a)
    got_offsets, got_items = read_stream(prefix + ".reorder.bin")
    assert np.array_equal(got_offsets, offsets) and np.array_equal(got_items, items)
    _, items_nr, offsets_nr = oracle.compress_noreorder(a)
    got_offsets, got_items = read_stream(prefix + ".noreorder.bin")
    assert np.array_equal(got_offsets, offsets_nr) and np.array_equal(got_items, items_nr)
    assert np.array_equal(np.fromfile(prefix + ".NZWeights.bin", dtype=np.uint32), items)
    assert np.array_equal(np.fromfile(prefix + ".TileOffsets.bin", dtype=np.int32), offsets)
    assert list(np.fromfile(prefix + ".OutputSizes.bin", dtype=np.int32)) == [items.size, offsets.size]
