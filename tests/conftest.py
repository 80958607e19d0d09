import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for sub in ("flash-llm_amd", "oracle", "tests"):
    p = os.path.join(ROOT, sub)
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def product():
    """The shipped library through its ctypes binding; building is not a test's job."""
    import flashllm_spmm

    if not os.path.exists(flashllm_spmm.LIB_PATH):
        import subprocess

        subprocess.run(["make", "-C", os.path.join(ROOT, "flash-llm_amd")], check=True, capture_output=True)
    flashllm_spmm.lib()
    return flashllm_spmm


@pytest.fixture(scope="session")
def oracle():
    import oracle as o

    o.lib()
    return o
