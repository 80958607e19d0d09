"""The spmm_test command line (the reference's kernel_benchmark/spmm_test.cu arguments and report
lines) runs on the GPU: a test of the tool (arguments, report layout, exit codes).  Parity of the
kernels is the business of test_gpu_spmm.py and test_gpu_baseline_configs.py; here the sparse results
only have to agree with the tool's own dense rocBLAS product to max|d|/max|C| <= 1e-2."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "flash-llm_amd", "kernel_benchmark", "spmm_test")

pytestmark = pytest.mark.gpu

LINE = re.compile(r"^(\S+)\s+->\s+Time/ms:\s+([\d.]+)\s+Performance/TFLOPs:\s+([\d.]+)\s+TotalError:\s+([\d.]+)", re.M)


@pytest.mark.parametrize("m,k,n,sparsity,split_k", [(1024, 1024, 16, 80, 4), (512, 2048, 64, 70, 0), (256, 512, 8, 90, 1)])
def test_spmm_test_reports_and_agrees_with_dense(m, k, n, sparsity, split_k):
    assert os.path.exists(EXE), "flash-llm_amd/kernel_benchmark/spmm_test is not built: make -C flash-llm_amd spmm_test"
    env = dict(os.environ, FLASHLLM_WARMUP="5", FLASHLLM_ITERS="20")
    r = subprocess.run([EXE, str(m), str(k), str(n), str(sparsity), str(split_k)], capture_output=True, text=True, timeout=120, env=env)
    print(r.stdout, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert f"M: {m} N: {n} K: {k} Pruning Rate: {sparsity}" in r.stdout
    rows = {name: (float(ms), float(tf), float(err)) for name, ms, tf, err in LINE.findall(r.stdout)}
    assert set(rows) == {"rocBLAS_TC", "FlashLLM_v1", "FlashLLM_v2"}
    rel = re.search(r"MaxRelError.*FlashLLM_v1 (\S+) FlashLLM_v2 (\S+)", r.stdout)
    assert rel, r.stdout
    assert float(rel.group(1)) <= 1e-2 and float(rel.group(2)) <= 1e-2
    for name in ("FlashLLM_v1", "FlashLLM_v2"):
        assert rows[name][0] > 0


def test_spmm_test_fails_on_an_unsupported_n():
    """N = 24 is not a width the API dispatches on (reference csrc/SpMM_API.cu:113-116): the tool must not
    print a time for a launch that never happened."""
    env = dict(os.environ, FLASHLLM_WARMUP="2", FLASHLLM_ITERS="5")
    r = subprocess.run([EXE, "256", "256", "24", "80", "1"], capture_output=True, text=True, timeout=120, env=env)
    assert r.returncode != 0, r.stdout
    assert "SpMM_SplitK_API returned" in r.stdout and "FlashLLM_v2" not in r.stdout


def test_spmm_test_rejects_bad_arguments():
    r = subprocess.run([EXE, "100", "64", "8", "80"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "Wrong Inputs" in r.stdout
