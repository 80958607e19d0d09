"""GPU parity at the full workloads of the benchmark configurations: the FFN sweep (both shapes, three
sparsities, four batch widths), the hidden-12288 projections with Beta(2,8) row densities, and eight
chained decoder layers at hidden 9216.

Every product goes through the C ABI at the Split_K the library's heuristic picks and is compared with
the oracle's fp32-accumulated product on the same fp16 operands: max|C - ref| / max|ref| <= 1e-2 and
|C - ref| <= 1e-2*|ref| + 1e-2*rms(ref) element-wise.  The compressed stream of every matrix is
scattered back by the oracle and must reproduce the matrix bit for bit (-0 and NaN mapped to +0).
Shapes: the reference's benchmark grid (kernel_benchmark/benchmark.sh:13-31) and the four call sites
of a decoder layer (third_party/ft.patch:512-525, :615-633, :1247-1261, :1328-1340).
"""
import sys

import numpy as np
import pytest

import synth
from gpu_util import assert_close

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def torch_gpu():
    import torch

    assert torch.cuda.is_available(), "these tests need the GPU"
    return torch


def multiply(torch, w, b_host, n, split_k):
    """C (N, M) of the resident weight w times b_host, with poisoned output and workspace."""
    b = torch.from_numpy(np.ascontiguousarray(b_host)).cuda()
    c = torch.full((n * w.m,), float("nan"), dtype=torch.float16, device="cuda")
    ws = torch.full((max(split_k, 1) * n * w.m,), float("nan"), dtype=torch.float16, device="cuda")
    w.matmul(b, n, c=c, workspace=ws, split_k=split_k)
    torch.cuda.synchronize()
    return c.cpu().numpy().reshape(n, w.m)


def assert_round_trip(oracle, w, a):
    """scatter(Compressed_A) == A with -0 / NaN -> +0 (what the nonzero test of the format drops)."""
    back = oracle.scatter(w.comp.cpu().numpy().view(np.uint32)[:w.nnz], w.offs.cpu().numpy(), w.m, w.k)
    bits = a.view(np.uint16)
    mag = bits & 0x7FFF
    assert np.array_equal(back, np.where((mag != 0) & (mag <= 0x7C00), bits, 0))


# --- FFN-shaped sweep: 36864 x 9216 and 9216 x 36864, {70, 80, 90} %, N in {8, 16, 32, 64} ----------
@pytest.mark.parametrize("sparsity", [0.7, 0.8, 0.9])
@pytest.mark.parametrize("shape", [(36864, 9216), (9216, 36864)], ids=["up", "down"])
def test_ffn_sweep_full_size(product, oracle, torch_gpu, shape, sparsity):
    m, k = shape
    say(f"ffn sweep {m}x{k} sparsity={sparsity}: generate")
    a = synth.sparse_matrix(m, k, sparsity, int(sparsity * 10) + (m > k), dist="normal", sigma=0.02, threads=16)
    say("  compress + upload")
    w = product.SparseWeight(a)
    tiles = (m // 128) * (k // 64)
    assert w.num_offsets == tiles + 2
    say("  round trip of the compressed stream")
    assert_round_trip(oracle, w, a)
    # 128 and 256 (the kernel for wide B, beyond the configuration's own list) at 80 %, at the Split_K and the
    # several rounds of workgroups the heuristic gives them at full size
    for n in (8, 16, 32, 64) + ((128, 256) if sparsity == 0.8 else ()):
        s = product.splitk_heuristic(m, n, k)
        say(f"  N={n} split_k={s}")
        b = synth.dense_b(k, n, 100 + n, dist="normal")
        ref, _ = oracle.gemm_f32(a, b, n)
        c = multiply(torch_gpu, w, b, n, s)
        assert_close(c, ref, f"ffn {m}x{k} s={sparsity} N={n} split_k={s}")


# --- hidden 12288, row keep-ratio ~ Beta(2,8) rescaled to a 20 % mean, N = 32 -----------------------
@pytest.mark.parametrize("shape", [(36864, 12288), (12288, 12288), (49152, 12288), (12288, 49152)],
                         ids=["qkv", "out", "ffn1", "ffn2"])
def test_hidden12288_beta_rows_full_size(product, oracle, torch_gpu, shape):
    m, k = shape
    n = 32
    say(f"hidden12288 {m}x{k} beta rows: generate")
    a = synth.sparse_matrix(m, k, 0.8, 40 + (m // 12288) + 7 * (k // 12288), dist="normal", sigma=0.02, row_beta=True, threads=16)
    density = np.count_nonzero(a, axis=1) / k
    assert abs(density.mean() - 0.2) < 0.01 and density.max() > 0.5 and density.min() < 0.03  # really uneven rows
    say("  compress + upload")
    w = product.SparseWeight(a)
    say("  round trip of the compressed stream")
    assert_round_trip(oracle, w, a)
    b = synth.dense_b(k, n, 50, dist="normal")
    ref, _ = oracle.gemm_f32(a, b, n)
    s = product.splitk_heuristic(m, n, k)
    splits = [s, 1] if m == k else [s]  # Split_K = 1 as well for the smallest of the four
    for split_k in splits:
        say(f"  N={n} split_k={split_k}")
        c = multiply(torch_gpu, w, b, n, split_k)
        assert_close(c, ref, f"hidden12288 {m}x{k} split_k={split_k}")


# --- chained decoder-layer linears: hidden 9216, 16 tokens, 8 layers, seeds layer*4 + w -------------
def test_decoder_layers_hidden9216_eight_layers(product, oracle, torch_gpu):
    torch = torch_gpu
    hidden, tokens, layers = 9216, 16, 8
    shapes = [(3 * hidden, hidden), (hidden, hidden), (4 * hidden, hidden), (hidden, 4 * hidden)]
    x_h = synth.dense_b(hidden, tokens, 999, dist="normal")
    x = torch.from_numpy(x_h).cuda()
    bufs = ws = None
    comp_bytes = dense_bytes = 0
    for layer in range(layers):
        dense, weights = [], []
        for i, (m, k) in enumerate(shapes):
            say(f"layer {layer} weight {i} {m}x{k}: generate + compress")
            a = synth.sparse_matrix(m, k, 0.8, layer * 4 + i, dist="normal", sigma=0.02, threads=16)
            dense.append(a)
            weights.append(product.SparseWeight(a))
            comp_bytes += 4 * weights[-1].nnz + 4 * weights[-1].num_offsets
            dense_bytes += 2 * m * k
        lay = product.DecoderLayer(*weights)
        if ws is None:
            ws = torch.full((lay.workspace_halfs(tokens),), float("nan"), dtype=torch.float16, device="cuda")
        say(f"layer {layer}: run")
        y, bufs = lay.forward(x, tokens, buffers=bufs, workspace=ws)
        torch.cuda.synchronize()
        qkv, attn_in, attn_out, ffn_mid, y_h = [b.cpu().numpy() for b in bufs]
        say(f"layer {layer}: check")
        qkv = qkv.reshape(tokens, 3 * hidden)
        ref, _ = oracle.gemm_f32(dense[0], x_h, tokens)
        assert_close(qkv, ref, f"layer {layer} qkv")
        attn_in = np.ascontiguousarray(qkv[:, :hidden])   # read in place by the attention-output linear
        ref, _ = oracle.gemm_f32(dense[1], attn_in, tokens)
        attn_out = attn_out.reshape(tokens, hidden)
        assert_close(attn_out, ref, f"layer {layer} attention output")
        ref, _ = oracle.gemm_f32(dense[2], attn_out, tokens)
        ffn_mid = ffn_mid.reshape(tokens, 4 * hidden)
        assert np.all(ffn_mid >= 0)
        assert_close(ffn_mid, np.maximum(ref, 0), f"layer {layer} ffn1 + relu")
        ref, _ = oracle.gemm_f32(dense[3], ffn_mid, tokens)
        y_h = y_h.reshape(tokens, hidden)
        assert_close(y_h, ref, f"layer {layer} ffn2")
        assert np.all(np.isfinite(y_h)) and np.any(y_h != 0)
        # the next layer reads this layer's output
        x_h = y_h.copy()
        x = torch.from_numpy(x_h).cuda()
        del lay, weights, dense
    say(f"weights: {comp_bytes / 1e9:.2f} GB compressed vs {dense_bytes / 1e9:.2f} GB dense")
    assert comp_bytes < 0.45 * dense_bytes
