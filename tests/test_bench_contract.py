"""bench.py's host-side contract, checked without a GPU: more than one GPU is refused with a message, the
algorithmic bytes are Compressed_A + TileOffsets + B once + C once, and the HBM traffic quoted in the JSON line comes
from the committed rocprofv3 summary of exactly the benchmarked workload (null for any other)."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_bench():
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr


def test_algorithmic_bytes_of_the_headline_workload():
    bench = load_bench()
    m, k, n, nnz = 36864, 9216, 16, 68012880
    tiles = (m // 128) * (k // 64)
    want = 4 * nnz + 4 * (tiles + 2) + 2 * k * n + 2 * m * n
    assert bench.algorithmic_bytes(nnz, m, n, k) == want == 273691976


def test_traffic_is_taken_from_the_profile_of_the_same_workload_only():
    bench = load_bench()
    traffic, source = bench.measured_traffic(36864, 9216, 16, 7, 68012880)
    assert source == os.path.join("profiles", "spmm_stream_kernel_36864x9216x16_s80.md")
    alg = bench.algorithmic_bytes(68012880, 36864, 16, 9216)
    assert alg <= traffic <= 1.10 * alg   # slabs instead of one C, a little re-reading of B and TileOffsets
    assert bench.measured_traffic(36864, 9216, 32, 7, 68012880) == (None, None)
    assert bench.measured_traffic(36864, 9216, 16, 8, 68012880) == (None, None)
