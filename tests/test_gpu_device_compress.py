"""GPU parity of the device-side Tiled-CSL compressor (flashllm_device_tile_offsets +
flashllm_device_compress, through the C ABI): Compressed_A and TileOffsets are compared bit for bit
with the CPU oracle's restatement of InitSparseMatrixA_API, and at the full headline size with the
product's host compressor (itself bit-exact against the oracle at the sizes the oracle finishes)."""
import sys

import numpy as np
import pytest

import synth

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def torch_gpu():
    import torch

    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


def device_compress(product, torch, a):
    a_dev = torch.from_numpy(np.ascontiguousarray(a).view(np.float16)).cuda()
    comp, offs = product.device_compress(a_dev)
    torch.cuda.synchronize()
    return comp.cpu().numpy().view(np.uint32), offs.cpu().numpy()


def check_against_oracle(product, oracle, torch, a, what):
    say("device compress:", what, a.shape)
    items, offsets = device_compress(product, torch, a)
    _, want_items, want_offsets = oracle.compress_reorder(a)
    assert np.array_equal(offsets, want_offsets), f"{what}: TileOffsets differ"
    assert items.shape == want_items.shape, f"{what}: {items.shape} vs {want_items.shape}"
    bad = np.flatnonzero(items != want_items)
    assert bad.size == 0, f"{what}: {bad.size} items differ, first at {bad[:4]}"
    assert product.device_compress_status() == 0, f"{what}: the encoder recorded an error"


def test_config1(product, oracle, torch_gpu):
    check_against_oracle(product, oracle, torch_gpu, synth.sparse_matrix(1024, 1024, 0.8, 0), "config1")


def test_config2(product, oracle, torch_gpu):
    check_against_oracle(product, oracle, torch_gpu, synth.sparse_matrix(9216, 9216, 0.8, 0), "config2")


@pytest.mark.parametrize("sparsity", [0.0, 0.3, 0.5, 0.9, 0.99, 0.999, 1.0])
def test_any_density(product, oracle, torch_gpu, sparsity):
    a = synth.sparse_matrix(384, 320, sparsity, 11)
    check_against_oracle(product, oracle, torch_gpu, a, f"sparsity {sparsity}")


def test_every_padding_count_and_short_tiles(product, oracle, torch_gpu):
    # one tile per case: 0..40 nonzeros (fewer vectors than banks: tail part only), around 128 and 256
    # items (main part only, main + tail), all four values of nnz % 4
    rng = np.random.default_rng(5)
    counts = list(range(0, 41)) + [124, 125, 126, 127, 128, 129, 130, 131, 253, 254, 255, 256, 257, 508, 512, 516, 8189, 8190, 8191, 8192]
    a = np.zeros((128 * len(counts), 64), dtype=np.float16)
    for i, c in enumerate(counts):
        flat = np.zeros(128 * 64, dtype=np.float16)
        where = rng.choice(128 * 64, size=c, replace=False)
        flat[where] = rng.uniform(0.5, 1.0, size=c).astype(np.float16)
        a[i * 128:(i + 1) * 128] = flat.reshape(128, 64)
    check_against_oracle(product, oracle, torch_gpu, a, "padding counts / short tiles")


def test_uneven_banks(product, oracle, torch_gpu):
    # nonzeros concentrated in a few columns (= a few LDS banks): the drain levels very uneven banks,
    # and padding lands in banks that hold nothing
    rng = np.random.default_rng(6)
    a = np.zeros((512, 256), dtype=np.float16)
    for t in range(16):
        r0, c0 = (t // 4) * 128, (t % 4) * 64
        cols = rng.choice(64, size=1 + t % 5, replace=False)
        for c in cols:
            rows = rng.choice(128, size=int(rng.integers(1, 129)), replace=False)
            a[r0 + rows, c0 + c] = rng.uniform(-1, 1, size=rows.size).astype(np.float16)
    check_against_oracle(product, oracle, torch_gpu, a, "uneven banks")


def test_special_values(product, oracle, torch_gpu):
    # -0 and NaN are dropped, subnormals and infinities are kept (the reference's float compare)
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 1 << 16, size=(256, 128), dtype=np.uint16)
    keep = rng.random((256, 128)) < 0.3
    bits = np.where(keep, bits, np.uint16(0))
    bits[0, :8] = [0x8000, 0x7E00, 0xFE00, 0x7C00, 0xFC00, 0x0001, 0x8001, 0x7C01]
    check_against_oracle(product, oracle, torch_gpu, bits.view(np.float16), "special values")


def test_headline_size_matches_host_compressor(product, torch_gpu):
    say("device compress: 36864x9216 against the host compressor")
    a = synth.sparse_matrix(36864, 9216, 0.8, 0, dist="normal", sigma=0.02, threads=16)
    items, offsets = device_compress(product, torch_gpu, a)
    want_items, want_offsets = product.init_sparse_matrix_a(a)
    assert np.array_equal(offsets, want_offsets)
    assert np.array_equal(items, want_items)


def test_spmm_on_device_compressed_weights(product, oracle, torch_gpu):
    # the device-compressed stream feeds the SpMM kernel directly
    from gpu_util import assert_close

    torch = torch_gpu
    m, k, n = 1024, 2048, 16
    a = synth.sparse_matrix(m, k, 0.8, 21)
    b = synth.dense_b(k, n, 22)
    comp, offs = product.device_compress(torch.from_numpy(a).cuda())
    b_dev = torch.from_numpy(b).cuda()
    c = torch.empty(n * m, dtype=torch.float16, device="cuda")
    ws = torch.empty(4 * n * m, dtype=torch.float16, device="cuda")
    product.spmm_splitk(comp, offs, b_dev, c, m, n, k, ws, 4)
    torch.cuda.synchronize()
    _, ref = oracle.spmm_model(a, b, n, 4)
    assert_close(c.cpu().numpy().reshape(n, m), ref, "spmm on device-compressed weights")


def test_status_reports_offsets_of_another_matrix(product, torch_gpu):
    """The encoder trusts TileOffsets for where a tile goes.  Given those of a different matrix it stays inside
    each tile's range, finishes normally, and says so through flashllm_device_compress_status; the word is
    cleared by reading it."""
    torch = torch_gpu
    say("device compress: status word")
    a = torch.from_numpy(synth.sparse_matrix(256, 128, 0.8, 31)).cuda()
    other = torch.from_numpy(synth.sparse_matrix(256, 128, 0.7, 32)).cuda()
    comp, offs = product.device_compress(a)
    assert product.device_compress_status() == 0
    _, offs_other = product.device_compress(other)
    assert product.device_compress_status() == 0
    out = torch.zeros(int(offs_other[-1].item()) * 4, dtype=torch.int32, device="cuda")
    rc = product.lib().flashllm_device_compress(None, a.data_ptr(), 256, 128, offs_other.data_ptr(), out.data_ptr())
    assert rc == 0
    assert product.device_compress_status() == product.ENCODE_OFFSETS
    assert product.device_compress_status() == 0
    # and the right offsets still give the right bytes afterwards
    again, _ = product.device_compress(a)
    assert torch.equal(again, comp) and product.device_compress_status() == 0


def test_rejects_bad_arguments(product, torch_gpu):
    torch = torch_gpu
    with pytest.raises(product.CompressError):
        product.device_compress(torch.zeros(100, 64, dtype=torch.float16, device="cuda"))
    with pytest.raises(product.CompressError):
        product.device_compress(torch.zeros(128, 96, dtype=torch.float16, device="cuda"))
    with pytest.raises(TypeError):
        product.device_compress(torch.zeros(128, 64, dtype=torch.float32, device="cuda"))
