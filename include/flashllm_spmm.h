/*
 * Plain-C ABI of libSpMM_API.so: the same hot path as SpMM_API.h with
 * nothing but pointers and ints in the signatures, for callers that bind
 * over an FFI.  Every function returns instead of exiting.
 */
#ifndef FLASHLLM_AMD_SPMM_C_H
#define FLASHLLM_AMD_SPMM_C_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Error codes of the host-side functions (negative return values). */
#define FLASHLLM_E_SHAPE (-1)   /* M % 128 != 0, K % 64 != 0 or not positive */
#define FLASHLLM_E_NOMEM (-2)   /* host allocation failed */
#define FLASHLLM_E_NOZERO (-3)  /* padding needed in a bank with no zero position (the reference asserts; unreachable:
                                   the emptiest bank always has one) */
#define FLASHLLM_E_ARG (-5)     /* null pointer */
#define FLASHLLM_E_IO (-6)      /* file could not be opened / short read */

/*
 * C twin of InitSparseMatrixA_API (reference csrc/SpMM_API.cu:163-360).
 * A_h: row-major M x K fp16 bit patterns on the host.  On success returns
 * (M/128)*(K/64)+2 and sets *Compressed_A / *TileOffsets to buffers that
 * must be released with flashllm_free.
 */
int flashllm_init_sparse_matrix_a(const uint16_t* A_h, int M, int K, uint32_t** Compressed_A, int** TileOffsets);

/* C twin of InitSparseMatrixA_API_NoReorder (reference csrc/SpMM_API.cu:363-489). */
int flashllm_init_sparse_matrix_a_noreorder(
    const uint16_t* A_h, int M, int K, uint32_t** Compressed_A, int** TileOffsets);

/* Releases a buffer returned by the two functions above (the reference's
 * callers use free(), kernel_benchmark/spmm_test.cu:268-269). */
void flashllm_free(void* p);

/* Worker threads the compressors use (tiles are independent); 0 = one per
 * host core, capped at 16.  The reference is single-threaded
 * (csrc/SpMM_API.cu:235-351); the bytes do not depend on this setting. */
void flashllm_set_compress_threads(int n);

/*
 * C twin of SpMM_SplitK_API (reference csrc/SpMM_API.cu:55-130).  stream is
 * a hipStream_t (NULL = the default stream); all other pointers are device
 * pointers.  Returns the hipError_t as an int (0 = success).
 */
int flashllm_spmm_splitk(void*       stream,
                         const void* A,
                         const void* Compressed_A,
                         const int*  TileOffsets,
                         const void* B,
                         void*       C,
                         int         M,
                         int         N,
                         int         K,
                         void*       Reduction_Workspace,
                         int         Split_K);

/*
 * flashllm_spmm_splitk without the Reduction_Workspace argument, for callers that cannot allocate
 * device memory and hold no workspace (code under stream capture, tight serving loops, harnesses
 * that forbid hipMalloc).  It has no counterpart in the reference.  The Split_K slabs go to a fixed
 * array of FLASHLLM_STATIC_WORKSPACE_MAX_BYTES that is part of the library's device image (every GPU
 * the library runs on holds one copy until the process ends); the call allocates and frees nothing.
 * Split_K * M * N * 2 bytes beyond that size are rejected with hipErrorInvalidValue (1) and a message
 * on stderr, before anything is launched.  All calls on one GPU share the array: calls that overlap
 * on one GPU (different streams or threads) race on the slabs; calls on one stream are ordered and safe.
 * Every slab is fully written before it is read, so nothing needs clearing between calls.
 * The first call on a GPU looks the array's address up (hipGetSymbolAddress) and keeps it; a caller that
 * records calls under stream capture should make one call outside the capture first.
 */
#define FLASHLLM_STATIC_WORKSPACE_MAX_BYTES (32u << 20)
int flashllm_spmm_splitk_static(void*       stream,
                                const void* A,
                                const void* Compressed_A,
                                const int*  TileOffsets,
                                const void* B,
                                void*       C,
                                int         M,
                                int         N,
                                int         K,
                                int         Split_K);

/*
 * Where the two halves below keep the Split_K partial products in
 * Reduction_Workspace (Split_K*M*N halfs either way):
 *  FLASHLLM_SLABS_PLAIN         slab s is M*N halfs at s*M*N, laid out like C:
 *                               the reference's workspace
 *                               (csrc/SpMM_Kernel.cuh:188-190, :293-303);
 *  FLASHLLM_SLABS_BY_WORKGROUP  the 128x16 blocks of partial sums as 4 KB
 *                               pages in the order of the SpMM launch's
 *                               workgroups, which keeps every page in the L2
 *                               of the one XCD that writes and sums it.  This
 *                               is what flashllm_spmm_splitk does between its
 *                               own two kernels; the contents mean something
 *                               only to flashllm_splitk_reduce with the same
 *                               M, N, Split_K.
 */
#define FLASHLLM_SLABS_PLAIN 0
#define FLASHLLM_SLABS_BY_WORKGROUP 1

/*
 * The first half of flashllm_spmm_splitk alone (reference
 * csrc/SpMM_API.cu:73-118): launches only the SpMM kernel and leaves the
 * Split_K fp16 slabs in Reduction_Workspace in the given order (or writes C
 * when Split_K == 1).  For callers that time the kernels separately or fuse
 * the reduction.
 */
int flashllm_spmm_partials(void*       stream,
                           const void* Compressed_A,
                           const int*  TileOffsets,
                           const void* B,
                           void*       C,
                           int         M,
                           int         N,
                           int         K,
                           void*       Reduction_Workspace,
                           int         Split_K,
                           int         Slab_Order);

/* The second half alone (reference csrc/Reduction_Kernel.cuh:24-45, launch
 * csrc/SpMM_API.cu:126-128): C[e] = rn16(sum_s float(slab s at e)), slabs
 * taken in order, for slabs stored in Slab_Order. */
int flashllm_splitk_reduce(void* stream, void* C, const void* Reduction_Workspace, int M, int N, int Split_K, int Slab_Order);

/*
 * Split_K recommended for one MI355X (256 CUs, wave64).  Takes the place of
 * the per-shape tables hand-tuned for A100 in the reference
 * (kernel_benchmark/benchmark.sh:13-15,
 * end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:20).
 */
int flashllm_splitk_heuristic(int M, int N, int K);

/*
 * Tiled-CSL compression on the GPU for a dense matrix that is already in
 * device memory: the bytes of flashllm_init_sparse_matrix_a (reference
 * InitSparseMatrixA_API, csrc/SpMM_API.cu:163-360, which runs on the host on
 * one thread), produced by one workgroup of four waves per 128x64 tile.  Two
 * calls, because the caller owns the output allocation:
 *
 *  flashllm_device_tile_offsets fills TileOffsets (device, (M/128)*(K/64)+2
 *  ints) and, when NNZ_padded is not NULL, waits for the stream and stores the
 *  number of packed items (TileOffsets[last]*4) there, so that the caller can
 *  allocate Compressed_A (4 bytes per item, 16-byte aligned);
 *
 *  flashllm_device_compress writes Compressed_A (device) from A and the
 *  TileOffsets of the first call, asynchronously on the stream.
 *
 * A: device pointer, row-major M x K halfs, 16-byte aligned; M % 128 == 0,
 * K % 64 == 0.  Returns 0, a negative FLASHLLM_E_* code or a positive
 * hipError_t value.  TileOffsets given to flashllm_device_compress must be
 * what flashllm_device_tile_offsets computed for this very A: the encoder
 * trusts them for where each tile goes.  With other offsets the contents of
 * Compressed_A are unspecified; the encoder still never writes outside
 * [TileOffsets[t], TileOffsets[t+1]) for tile t; the call is asynchronous, so
 * the mismatch is reported by flashllm_device_compress_status afterwards.
 */
int flashllm_device_tile_offsets(void* stream, const void* A, int M, int K, int* TileOffsets, long long* NNZ_padded);
int flashllm_device_compress(void* stream, const void* A, int M, int K, const int* TileOffsets, void* Compressed_A);

/*
 * What flashllm_device_compress found wrong, for callers that want the host compressor's error behaviour from the
 * asynchronous device one: waits for the stream, stores in *Status the bits recorded on the current GPU since the
 * last call of this function (0 = every tile was encoded as the host compressor would), and clears them.
 *  FLASHLLM_ENCODE_NO_ZERO  a padding item was needed in a bank without a zero position (the host compressor
 *                           returns FLASHLLM_E_NOZERO, the reference asserts, csrc/SpMM_API.cu:282);
 *  FLASHLLM_ENCODE_OFFSETS  TileOffsets did not belong to this matrix: some tile's range differs from its count
 *                           (items beyond the range were dropped, a longer range was left partly unwritten);
 *  FLASHLLM_ENCODE_RANGE    an item's computed place lay outside its tile (an internal error; the item was dropped).
 * Returns 0 or a hipError_t value.
 */
#define FLASHLLM_ENCODE_NO_ZERO 1u
#define FLASHLLM_ENCODE_OFFSETS 2u
#define FLASHLLM_ENCODE_RANGE 4u
int flashllm_device_compress_status(void* stream, unsigned int* Status);

/* Bytes the caller must provide as Reduction_Workspace (0 when Split_K == 1);
 * the contract of reference build/SpMM_API.cuh:33-36. */
size_t flashllm_workspace_bytes(int M, int N, int Split_K);

/*
 * One pruned linear layer resident on the GPU: the NZWeights / TileOffsets / SplitK fields the
 * reference adds to FasterTransformer's DenseWeight (third_party/ft.patch:456-462).
 * split_k == 0 asks for flashllm_splitk_heuristic at the given token count.
 */
typedef struct {
    const void* nz_weights;   /* device, Compressed_A */
    const int*  tile_offsets; /* device */
    int         m;            /* output features (rows of A) */
    int         k;            /* input features */
    int         split_k;
} flashllm_sparse_weight;

/* The four pruned weights of one decoder layer, in the reference's call order
 * (third_party/ft.patch:1247-1261 QKV, :1328-1340 attention output, :512-525 FFN1, :615-633 FFN2). */
typedef struct {
    flashllm_sparse_weight qkv, attn_out, ffn1, ffn2;
} flashllm_decoder_layer;

/*
 * Applies the four linears of one decoder layer back to back on `tokens` activations
 * (column-major, hidden x tokens fp16), all on `stream`, sharing one Reduction_Workspace as the
 * reference's cublasMMWrapper does (ft.patch:2761-2765, :2822-2847):
 *     qkv_out  = Wqkv * x                      (3*hidden x tokens)
 *     attn_out = Wo   * qkv_out[0:hidden, :]   (the attention itself is not part of this library:
 *                                               the first hidden rows stand in for its output)
 *     ffn_mid  = relu(W1 * attn_out)
 *     y        = W2   * ffn_mid
 * Like the reference's call sites, Split_K falls back to 1 when tokens > 128 (FFN, ft.patch:523)
 * or tokens > 64 (attention, ft.patch:1454).  The attention-output linear reads the first hidden rows
 * of every column of qkv_out in place (B with its columns qkv.m halfs apart).  attn_in may be NULL; when
 * it is not, it also receives those rows as a dense hidden x tokens matrix (a strided copy kernel).
 * Buffers: qkv_out qkv.m*tokens, attn_in / attn_out attn_out.k*tokens / attn_out.m*tokens,
 * ffn_mid ffn1.m*tokens, y ffn2.m*tokens halfs; workspace for the largest Split_K*M*tokens.
 * Returns a hipError_t as int (hipErrorInvalidValue when the shapes do not chain).
 */
int flashllm_decoder_layer_linears(void*                         stream,
                                   const flashllm_decoder_layer* layer,
                                   const void*                   x,
                                   void*                         qkv_out,
                                   void*                         attn_in,
                                   void*                         attn_out,
                                   void*                         ffn_mid,
                                   void*                         y,
                                   int                           tokens,
                                   void*                         Reduction_Workspace);

/* Six-argument file exporter (reference csrc/SpMM_API.cu:500-555) that
 * returns 0 or a FLASHLLM_E_* code instead of exiting. */
int flashllm_gen_sparse_matrix_bin_file(const char* DenseMatrixFileName,
                                        int         M,
                                        int         K,
                                        const char* NZWeightsFileName,
                                        const char* TileOffsetsFileName,
                                        const char* OutputSizesFileName);

/* Same symbol and signature as the reference's only extern "C" export
 * (csrc/SpMM_API.cu:500-505); exits on error like the reference. */
void GenSparseMatrixBinFile(char* DenseMatrixFileName,
                            int   M,
                            int   K,
                            char* NZWeightsFileName,
                            char* TileOffsetsFileName,
                            char* OutputSizesFileName);

#ifdef __cplusplus
}
#endif
#endif
