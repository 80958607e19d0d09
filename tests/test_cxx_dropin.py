"""A C++ caller compiled against include/SpMM_API.h, the way the reference's kernel benchmark uses
SpMM_API.cuh: builds with hipcc, links libSpMM_API.so, compresses on the host (checked against the
oracle), and on a GPU runs SpMM_SplitK_API on a stream it created itself."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "flash-llm_amd")


@pytest.fixture(scope="module")
def dropin(product, tmp_path_factory):
    src = os.path.join(ROOT, "tests", "cxx", "dropin.cpp")
    prebuilt = os.path.join(ROOT, "tests", "cxx", "dropin.bin")  # what __graft_entry__.build() leaves
    if os.path.exists(prebuilt) and os.path.getmtime(prebuilt) >= os.path.getmtime(src):
        return prebuilt
    exe = str(tmp_path_factory.mktemp("cxx") / "dropin")
    cmd = ["/opt/rocm/bin/hipcc", "-O2", "--offload-arch=gfx950", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cxx", "dropin.cpp"), "-o", exe, "-L", PKG, "-lSpMM_API", f"-Wl,-rpath,{PKG}",
           "-Wno-unused-result"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    return exe


def test_cxx_caller_compresses_like_the_oracle(dropin, oracle, tmp_path):
    m, k = 384, 256
    out = str(tmp_path / "c.bin")
    subprocess.run([dropin, "compress", str(m), str(k), "75", out], check=True)
    raw = np.fromfile(out, dtype=np.uint8)
    n_off = int(raw[:4].view(np.int32)[0])
    offsets = raw[4:4 + 4 * n_off].view(np.int32)
    nnz = int(offsets[-1]) * 4
    items = raw[4 + 4 * n_off:4 + 4 * n_off + 4 * nnz].view(np.uint32)
    a = raw[4 + 4 * n_off + 4 * nnz:].view(np.uint16).reshape(m, k)
    n, o_items, o_offsets = oracle.compress_reorder(a)
    assert n == n_off and np.array_equal(offsets, o_offsets) and np.array_equal(items, o_items)


@pytest.mark.gpu
@pytest.mark.parametrize("n,split_k", [(16, 1), (16, 4), (64, 2)])
def test_cxx_caller_runs_spmm_on_its_own_stream(dropin, n, split_k):
    r = subprocess.run([dropin, "spmm", "512", "1024", str(n), "80", str(split_k)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "max_rel_err" in r.stdout
