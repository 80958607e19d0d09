"""The offline weight files, consumed on the GPU the way the reference's loaders consume them
(third_party/ft.patch:3744-3794): sizes from .OutputSizes.bin, then exactly that many items /
offsets from .NZWeights.bin / .TileOffsets.bin onto the device, then SpMM_SplitK_API.  Writer:
GenSparseMatrixBinFile (reference csrc/SpMM_API.cu:500-555)."""
import sys

import numpy as np
import pytest

import synth
from gpu_util import assert_close

pytestmark = pytest.mark.gpu


def load_and_multiply(product, names, m, k, b_host, n, split_k):
    import torch

    nnz, num_offsets = np.fromfile(names[2], dtype=np.int32).tolist()  # OutputSizes: NNZ, NumOffsets
    assert num_offsets == (m // 128) * (k // 64) + 2
    with open(names[0], "rb") as f:
        items = np.frombuffer(f.read(4 * nnz), dtype=np.int32)
    with open(names[1], "rb") as f:
        offsets = np.frombuffer(f.read(4 * num_offsets), dtype=np.int32)
    assert items.size == nnz and offsets.size == num_offsets
    # a fully sparse weight has no items: the callers allocate at least one element (kernel_benchmark/spmm_test.cu:258-259)
    comp = torch.zeros(max(nnz, 1), dtype=torch.int32, device="cuda")
    comp[:nnz] = torch.from_numpy(items.copy())
    offs = torch.from_numpy(offsets.copy()).cuda()
    b = torch.from_numpy(b_host).cuda()
    c = torch.full((n * m,), float("nan"), dtype=torch.float16, device="cuda")
    ws = torch.full((split_k * n * m,), float("nan"), dtype=torch.float16, device="cuda")
    product.spmm_splitk(comp, offs, b, c, m, n, k, ws, split_k)
    torch.cuda.synchronize()
    return c.cpu().numpy().reshape(n, m), nnz


@pytest.mark.parametrize("sparsity", [0.8, 1.0])
def test_bin_files_feed_the_kernel(product, oracle, tmp_path, sparsity):
    import torch

    assert torch.cuda.is_available()
    m = k = 1024
    n = 16
    print(f"bin files {m}x{k} sparsity={sparsity}", flush=True)
    sys.stdout.flush()
    a = synth.sparse_matrix(m, k, sparsity, 31)
    dense = tmp_path / "w.bin"
    a.tofile(dense)
    names = [str(tmp_path / f"w.{x}.bin") for x in ("NZWeights", "TileOffsets", "OutputSizes")]
    product.lib().GenSparseMatrixBinFile(str(dense).encode(), m, k, *[x.encode() for x in names])
    b = synth.dense_b(k, n, 32)
    for split_k in (1, 4):
        c, nnz = load_and_multiply(product, names, m, k, b, n, split_k)
        if sparsity == 1.0:
            assert nnz == 0 and not c.any()
        else:
            _, items, _ = oracle.compress_reorder(a)
            assert nnz == items.size
            ref, _ = oracle.gemm_f32(a, b, n)
            assert_close(c, ref, f"bin files split_k={split_k}")
