"""ctypes binding of libSpMM_API.so's plain-C entry points (include/flashllm_spmm.h).

Thin by design: every call goes straight into the shared library.  There is
no CPU fallback; if the library is missing, loading raises.  Device buffers
are torch tensors (torch is only the allocator and the stream provider).

The functions mirror the reference's API (build/SpMM_API.cuh:38-67):
init_sparse_matrix_a <-> InitSparseMatrixA_API, spmm_splitk <-> SpMM_SplitK_API,
gen_sparse_matrix_bin_file <-> GenSparseMatrixBinFile.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libSpMM_API.so")

_lib = None

_u16p = ctypes.POINTER(ctypes.c_uint16)
_u32p = ctypes.POINTER(ctypes.c_uint32)
_i32p = ctypes.POINTER(ctypes.c_int)
_vp = ctypes.c_void_p

class SparseWeightStruct(ctypes.Structure):
    """flashllm_sparse_weight"""
    _fields_ = [("nz_weights", ctypes.c_void_p), ("tile_offsets", ctypes.c_void_p),
                ("m", ctypes.c_int), ("k", ctypes.c_int), ("split_k", ctypes.c_int)]


class DecoderLayerStruct(ctypes.Structure):
    """flashllm_decoder_layer"""
    _fields_ = [("qkv", SparseWeightStruct), ("attn_out", SparseWeightStruct),
                ("ffn1", SparseWeightStruct), ("ffn2", SparseWeightStruct)]


# name -> (restype, argtypes); every symbol include/flashllm_spmm.h declares
SIGNATURES = {
    "flashllm_init_sparse_matrix_a": (ctypes.c_int, [_u16p, ctypes.c_int, ctypes.c_int, ctypes.POINTER(_u32p), ctypes.POINTER(_i32p)]),
    "flashllm_init_sparse_matrix_a_noreorder": (ctypes.c_int, [_u16p, ctypes.c_int, ctypes.c_int, ctypes.POINTER(_u32p), ctypes.POINTER(_i32p)]),
    "flashllm_free": (None, [_vp]),
    "flashllm_set_compress_threads": (None, [ctypes.c_int]),
    "flashllm_spmm_splitk": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, ctypes.c_int]),
    "flashllm_spmm_splitk_static": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "flashllm_spmm_partials": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, ctypes.c_int, ctypes.c_int]),
    "flashllm_splitk_reduce": (ctypes.c_int, [_vp, _vp, _vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "flashllm_device_tile_offsets": (ctypes.c_int, [_vp, _vp, ctypes.c_int, ctypes.c_int, _vp, ctypes.POINTER(ctypes.c_longlong)]),
    "flashllm_device_compress": (ctypes.c_int, [_vp, _vp, ctypes.c_int, ctypes.c_int, _vp, _vp]),
    "flashllm_device_compress_status": (ctypes.c_int, [_vp, ctypes.POINTER(ctypes.c_uint)]),
    "flashllm_splitk_heuristic": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "flashllm_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int, ctypes.c_int, ctypes.c_int]),
    "flashllm_decoder_layer_linears": (ctypes.c_int, [_vp, ctypes.POINTER(DecoderLayerStruct), _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, _vp]),
    "flashllm_gen_sparse_matrix_bin_file": (ctypes.c_int, [ctypes.c_char_p, ctypes.c_int, ctypes.c_int, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_char_p]),
    "GenSparseMatrixBinFile": (None, [ctypes.c_char_p, ctypes.c_int, ctypes.c_int, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_char_p]),
}


def lib():
    """Loads libSpMM_API.so once.  Raises OSError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError(f"{LIB_PATH} is not built: run `make -C {_HERE}` (or __graft_entry__.build())")
        # One HIP runtime per process: torch ships its own libamdhip64.so.7.  Loading it first makes
        # the dynamic loader resolve this library's libamdhip64.so.7 dependency to that same copy;
        # a second runtime in the process reports hipErrorNoDevice on its first launch.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


class CompressError(ValueError):
    def __init__(self, code):
        super().__init__(f"Tiled-CSL compression failed with code {code}")
        self.code = code


def _compress(fn_name, a, threads):
    a = np.ascontiguousarray(a)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    if a.dtype != np.uint16 or a.ndim != 2:
        raise TypeError("A must be a 2-D float16 (or uint16 bit pattern) array")
    m, k = a.shape
    L = lib()
    if threads is not None:
        L.flashllm_set_compress_threads(int(threads))
    comp = _u32p()
    offs = _i32p()
    n = getattr(L, fn_name)(a.ctypes.data_as(_u16p), m, k, ctypes.byref(comp), ctypes.byref(offs))
    if n < 0:
        raise CompressError(n)
    try:
        offsets = np.ctypeslib.as_array(offs, shape=(n,)).copy()
        nnz = int(offsets[n - 1]) * 4
        items = np.ctypeslib.as_array(comp, shape=(max(nnz, 1),))[:nnz].copy()
    finally:
        L.flashllm_free(comp)
        L.flashllm_free(offs)
    return items, offsets


def init_sparse_matrix_a(a, threads=None):
    """InitSparseMatrixA_API: (Compressed_A uint32[NNZ_padded], TileOffsets int32[tiles+2])."""
    return _compress("flashllm_init_sparse_matrix_a", a, threads)


def init_sparse_matrix_a_noreorder(a, threads=None):
    """InitSparseMatrixA_API_NoReorder."""
    return _compress("flashllm_init_sparse_matrix_a_noreorder", a, threads)


def splitk_heuristic(m, n, k):
    return lib().flashllm_splitk_heuristic(m, n, k)


def workspace_bytes(m, n, split_k):
    return lib().flashllm_workspace_bytes(m, n, split_k)


def gen_sparse_matrix_bin_file(dense, m, k, nz, offsets, sizes):
    rc = lib().flashllm_gen_sparse_matrix_bin_file(dense.encode(), m, k, nz.encode(), offsets.encode(), sizes.encode())
    if rc:
        raise CompressError(rc)


def xcd_of_workgroups(workgroups, stream=None):
    """XCD id of every workgroup of a launch of `workgroups` one-wave workgroups (numpy uint32 array).
    The SpMM kernel's placement counts on ids repeating with period 8 (round-robin hand-out)."""
    import torch

    out = torch.empty(workgroups, dtype=torch.int32, device="cuda")
    fn = lib().flashllm_hip_launch_xcd_probe
    fn.restype = ctypes.c_int
    fn.argtypes = [_vp, _vp, ctypes.c_int]
    rc = fn(_stream(stream), _ptr(out), workgroups)
    if rc:
        raise HipError(rc)
    torch.cuda.synchronize()
    return out.cpu().numpy().view(np.uint32) & 15


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _stream(stream):
    import torch

    s = stream if stream is not None else torch.cuda.current_stream()
    return ctypes.c_void_p(s.cuda_stream)


class HipError(RuntimeError):
    def __init__(self, code):
        super().__init__(f"libSpMM_API returned hipError_t {code}")
        self.code = code


def spmm_splitk(comp, offs, b, c, m, n, k, workspace, split_k, stream=None, a=None):
    """SpMM_SplitK_API on torch device tensors; asynchronous on `stream`
    (default: torch's current stream).  Raises HipError on a non-zero code."""
    rc = lib().flashllm_spmm_splitk(_stream(stream), _ptr(a), _ptr(comp), _ptr(offs), _ptr(b), _ptr(c), m, n, k, _ptr(workspace), split_k)
    if rc:
        raise HipError(rc)


STATIC_WORKSPACE_MAX_BYTES = 32 << 20


def spmm_splitk_static(comp, offs, b, c, m, n, k, split_k, stream=None):
    """flashllm_spmm_splitk_static: the slabs live in the library's own fixed device array."""
    rc = lib().flashllm_spmm_splitk_static(_stream(stream), None, _ptr(comp), _ptr(offs), _ptr(b), _ptr(c), m, n, k, split_k)
    if rc:
        raise HipError(rc)


SLABS_PLAIN = 0          # FLASHLLM_SLABS_PLAIN: slab s = M*N halfs at s*M*N, laid out like C
SLABS_BY_WORKGROUP = 1   # FLASHLLM_SLABS_BY_WORKGROUP: what spmm_splitk keeps between its two kernels


def spmm_partials(comp, offs, b, c, m, n, k, workspace, split_k, stream=None, slab_order=SLABS_PLAIN):
    rc = lib().flashllm_spmm_partials(_stream(stream), _ptr(comp), _ptr(offs), _ptr(b), _ptr(c), m, n, k, _ptr(workspace), split_k,
                                      slab_order)
    if rc:
        raise HipError(rc)


def splitk_reduce(c, workspace, m, n, split_k, stream=None, slab_order=SLABS_PLAIN):
    rc = lib().flashllm_splitk_reduce(_stream(stream), _ptr(c), _ptr(workspace), m, n, split_k, slab_order)
    if rc:
        raise HipError(rc)


def device_compress(a_dev, stream=None):
    """Tiled-CSL compression of a device-resident fp16 matrix (torch tensor M x K) on the GPU.
    Returns (Compressed_A int32 tensor[NNZ_padded], TileOffsets int32 tensor[tiles+2]), both on the
    device, with the bytes InitSparseMatrixA_API produces on the host."""
    import torch

    if a_dev.dim() != 2 or a_dev.dtype != torch.float16 or not a_dev.is_contiguous():
        raise TypeError("A must be a contiguous 2-D float16 device tensor")
    m, k = a_dev.shape
    if m <= 0 or k <= 0 or m % 128 or k % 64:
        raise CompressError(-1)
    offs = torch.empty((m // 128) * (k // 64) + 2, dtype=torch.int32, device=a_dev.device)
    nnz = ctypes.c_longlong(0)
    rc = lib().flashllm_device_tile_offsets(_stream(stream), _ptr(a_dev), m, k, _ptr(offs), ctypes.byref(nnz))
    if rc:
        raise CompressError(rc) if rc < 0 else HipError(rc)
    comp = torch.empty(max(int(nnz.value), 1), dtype=torch.int32, device=a_dev.device)
    rc = lib().flashllm_device_compress(_stream(stream), _ptr(a_dev), m, k, _ptr(offs), _ptr(comp))
    if rc:
        raise CompressError(rc) if rc < 0 else HipError(rc)
    return comp[: int(nnz.value)], offs


ENCODE_NO_ZERO, ENCODE_OFFSETS, ENCODE_RANGE = 1, 2, 4  # FLASHLLM_ENCODE_*


def device_compress_status(stream=None):
    """flashllm_device_compress_status: waits for the stream and returns (and clears) the FLASHLLM_ENCODE_* bits
    the device encoder has recorded on the current GPU; 0 = nothing wrong."""
    word = ctypes.c_uint(0)
    rc = lib().flashllm_device_compress_status(_stream(stream), ctypes.byref(word))
    if rc:
        raise HipError(rc)
    return int(word.value)


class SparseWeight:
    """A compressed weight resident on the GPU: what a caller keeps per linear
    layer (the reference's DenseWeight::NZWeights/TileOffsets/SplitK fields,
    third_party/ft.patch:456-462)."""

    def __init__(self, a_host, split_k=None, reorder=True, device="cuda"):
        import torch

        a_host = np.ascontiguousarray(a_host)
        self.m, self.k = a_host.shape
        fn = init_sparse_matrix_a if reorder else init_sparse_matrix_a_noreorder
        items, offsets = fn(a_host)
        self.nnz = items.size
        self.num_offsets = offsets.size
        if items.size == 0:  # fully sparse: keep one addressable element, as the reference's callers do
            items = np.zeros(1, dtype=np.uint32)
        self.comp = torch.from_numpy(items.view(np.int32)).to(device)
        self.offs = torch.from_numpy(offsets).to(device)
        self.split_k = split_k
        self.device = device

    def matmul(self, b, n, c=None, workspace=None, split_k=None, stream=None):
        """b: fp16 device tensor holding column-major K x N; returns column-major M x N."""
        import torch

        s = split_k or self.split_k or splitk_heuristic(self.m, n, self.k)
        if c is None:
            c = torch.empty(n * self.m, dtype=torch.float16, device=self.device)
        if s > 1 and workspace is None:
            workspace = torch.empty(s * n * self.m, dtype=torch.float16, device=self.device)
        spmm_splitk(self.comp, self.offs, b, c, self.m, n, self.k, workspace, s, stream=stream)
        return c

    def as_struct(self):
        return SparseWeightStruct(self.comp.data_ptr(), self.offs.data_ptr(), self.m, self.k, self.split_k or 0)


class DecoderLayer:
    """The four pruned linears of one decoder layer (QKV, attention output, FFN1, FFN2) on the GPU."""

    def __init__(self, qkv, attn_out, ffn1, ffn2):
        self.weights = (qkv, attn_out, ffn1, ffn2)
        self.struct = DecoderLayerStruct(*[w.as_struct() for w in self.weights])

    def workspace_halfs(self, tokens):
        need = 1
        for w in self.weights:
            s = w.split_k or splitk_heuristic(w.m, tokens, w.k)
            need = max(need, s * w.m * tokens)
        return need

    def forward(self, x, tokens, buffers=None, workspace=None, stream=None, copy_attn_in=False):
        """x: fp16 device tensor, column-major hidden x tokens.  Returns (y, buffers); buffers = [qkv_out, attn_in,
        attn_out, ffn_mid, y].  attn_in is only written with copy_attn_in=True: the attention-output linear reads
        the first hidden rows of qkv_out in place."""
        import torch

        qkv, o, f1, f2 = self.weights
        dev = x.device
        if buffers is None:
            buffers = [torch.empty(n * tokens, dtype=torch.float16, device=dev) for n in (qkv.m, o.k, o.m, f1.m, f2.m)]
        if workspace is None:
            workspace = torch.empty(self.workspace_halfs(tokens), dtype=torch.float16, device=dev)
        ptrs = [_ptr(b) for b in buffers]
        if not copy_attn_in:
            ptrs[1] = None
        rc = lib().flashllm_decoder_layer_linears(_stream(stream), ctypes.byref(self.struct), _ptr(x), *ptrs, tokens, _ptr(workspace))
        if rc:
            raise HipError(rc)
        return buffers[4], buffers
