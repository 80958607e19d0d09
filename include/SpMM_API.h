/*
 * Source-level drop-in for the reference's build/SpMM_API.cuh on MI355X
 * (gfx950).  A caller that used to include SpMM_API.cuh includes this header
 * instead, recompiles with hipcc and links libSpMM_API.so; names, argument
 * order and argument meaning are unchanged, with hipStream_t / hipError_t in
 * place of the CUDA types (`half` is HIP's __half, `uint4` HIP's uint4).
 *
 * The plain-C entry points the library also exports for FFI callers (ctypes,
 * cgo, JNI ...) are declared in flashllm_spmm.h.
 */
#ifndef FLASHLLM_AMD_SPMM_API_H
#define FLASHLLM_AMD_SPMM_API_H

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

/*
 * C = A * B with A given in Tiled-CSL form.  Replaces SpMM_SplitK_API,
 * reference build/SpMM_API.cuh:38-48 (definition csrc/SpMM_API.cu:55-130).
 *
 *   stream               stream both kernels are enqueued on; no host sync.
 *   A                    unused (callers pass the dense copy or nullptr).
 *   Compressed_A         device, 16-byte aligned, packed nonzeros from
 *                        InitSparseMatrixA_API[_NoReorder]; for a matrix
 *                        without nonzeros (NNZ = 0) any allocation of one
 *                        element (4 bytes) will do, as the reference's
 *                        callers make (kernel_benchmark/spmm_test.cu:258-260).
 *   TileOffsets          device, (M/128)*(K/64)+2 ints from the same call.
 *   B                    device, column-major K x N (N columns of K halfs).
 *   C                    device, column-major M x N.
 *   M_Global             multiple of 128 (the reference needs 256).
 *   N_Global             8, 16, 32, 64, 128 or a multiple of 128; anything
 *                        else prints a message and returns hipErrorUnknown,
 *                        as the reference returns cudaErrorUnknown.  The
 *                        library is built for skinny B: measured on one
 *                        MI355X against the dense fp16 GEMM of the same
 *                        shape (36864 x 9216) the call is 2.5x faster at
 *                        N <= 16, 2.0x at N = 64, 1.1x-1.4x at N = 128
 *                        (70-90 % sparsity) and 0.74x-0.89x at N = 256:
 *                        callers should take their dense path above
 *                        N = 128.
 *   K_Global             multiple of 64.
 *   Reduction_Workspace  device, >= Split_K*M*N halfs; only touched when
 *                        Split_K > 1.  One workspace may serve every call
 *                        on one stream.
 *   Split_K              number of K slices (>= 1); slice s holds the
 *                        reference's k-tile range, is summed in fp32, stored
 *                        as an fp16 slab, and the slabs are added in fp32 by
 *                        a separate reduction kernel.
 * Returns hipSuccess, hipErrorInvalidValue for a bad shape / null pointer,
 * or the launch error.
 */
hipError_t SpMM_SplitK_API(hipStream_t  stream,
                           const half*  A,
                           const uint4* Compressed_A,
                           const int*   TileOffsets,
                           const half*  B,
                           half*        C,
                           const int    M_Global,
                           const int    N_Global,
                           const int    K_Global,
                           half*        Reduction_Workspace,
                           int          Split_K);

/*
 * Host-side Tiled-CSL compression with ahead-of-time bank reordering.
 * Replaces InitSparseMatrixA_API, reference build/SpMM_API.cuh:51
 * (definition csrc/SpMM_API.cu:163-360); output bytes are identical.
 * A_h is row-major M x K on the host; N is ignored, as in the reference.
 * *Compressed_A and *TileOffsets are malloc'd; the caller free()s them.
 * Returns the number of TileOffsets entries, (M/128)*(K/64)+2;
 * NNZ (padded) = (*TileOffsets)[ret-1]*4.  Where the reference asserts
 * (M%128, K%64, a padding item needed in a bank without a zero) this
 * returns a negative number and leaves the out-pointers NULL; on
 * out-of-memory it prints and exits like the reference.
 */
int InitSparseMatrixA_API(half* A_h, int M, int N, int K, uint32_t** Compressed_A, int** TileOffsets);

/* Same without reordering.  Replaces InitSparseMatrixA_API_NoReorder,
 * reference build/SpMM_API.cuh:53-58 (definition csrc/SpMM_API.cu:363-489). */
int InitSparseMatrixA_API_NoReorder(half* A_h, int M, int N, int K, uint32_t** Compressed_A, int** TileOffsets);

/*
 * Dense fp16 .bin -> .NZWeights.bin / .TileOffsets.bin / .OutputSizes.bin.
 * Replaces GenSparseMatrixBinFile as DEFINED and as called over ctypes
 * (six arguments: reference csrc/SpMM_API.cu:500-555, caller
 * end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:52-59); the
 * reference header's seven-argument declaration (build/SpMM_API.cuh:61-67)
 * has no definition.  Prints and exits on I/O errors like the reference.
 */
extern "C" void GenSparseMatrixBinFile(char* DenseMatrixFileName,
                                       int   M,
                                       int   K,
                                       char* NZWeightsFileName,
                                       char* TileOffsetsFileName,
                                       char* OutputSizesFileName);

#endif
