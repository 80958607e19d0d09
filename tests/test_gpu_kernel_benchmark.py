"""The spmm_test command line (the reference's kernel_benchmark/spmm_test.cu arguments and report
lines) runs on the GPU and its sparse results agree with the dense rocBLAS product."""
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
    # |C| is about sqrt(K * density / 3); fp16 rounding of each of the M*N outputs stays below 2^-10 of that,
    # plus the split-K partial roundings: a loose per-element bound of 1e-2 * typical magnitude
    typical = (k * (1 - sparsity / 100.0) / 3.0) ** 0.5
    for name in ("FlashLLM_v1", "FlashLLM_v2"):
        assert rows[name][2] <= 1e-2 * typical * m * n, (name, rows[name])
        assert rows[name][0] > 0


def test_spmm_test_rejects_bad_arguments():
    r = subprocess.run([EXE, "100", "64", "8", "80"], capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "Wrong Inputs" in r.stdout
