// The thin extern "C" HIP layer underneath the host API: one function per
// kernel launch, nothing but pointers and ints, no validation (the host API
// has checked the shapes these grids assume).
#ifndef FLASHLLM_AMD_SPMM_LAUNCH_H
#define FLASHLLM_AMD_SPMM_LAUNCH_H

#include "flashllm_spmm.h"

// size of the library-owned slab storage behind flashllm_hip_static_workspace: the limit the public header states
#define FLASHLLM_STATIC_WORKSPACE_BYTES FLASHLLM_STATIC_WORKSPACE_MAX_BYTES

#ifdef __cplusplus
extern "C" {
#endif

// *ptr = device address, on the current device, of the library's own fixed slab storage
// (FLASHLLM_STATIC_WORKSPACE_BYTES, 256-byte aligned).  Resolved once per device; allocates nothing.
int flashllm_hip_static_workspace(void** ptr);

// out: C when split_k == 1, else the slab workspace (split_k * M * N halfs).
// pages == 0: slab s is M*N halfs at s*M*N, laid out like C (for flashllm_hip_launch_reduce);
// pages != 0: each workgroup's 128 x 16 blocks of partial sums as 4 KB pages in workgroup order
// (for flashllm_hip_launch_reduce_pages; needs out 16-byte aligned).
// ldb: halfs between consecutive columns of B (>= K, a multiple of 8; K for a dense column-major B).
// Requires M % 128 == 0, K % 64 == 0, N in {8,16,32,64} or N % 64 == 0.
int flashllm_hip_launch_spmm(void*       stream,
                             const void* compressed_a,
                             const int*  tile_offsets,
                             const void* b,
                             int         ldb,
                             void*       out,
                             int         m,
                             int         n,
                             int         k,
                             int         split_k,
                             int         pages);

// Row tiles per workgroup of flashllm_hip_launch_spmm for n columns, m rows and split_k slices: 8 for n = 64
// when m / 128 is a multiple of 8 and (m / 1024) * split_k lies in 192 .. 256, otherwise 1.
// flashllm_hip_set_rows_per_workgroup is a measuring and testing aid, process-wide: 1 forces 1, 8 forces 8
// wherever m / 128 is a multiple of 8, anything else restores the rule.  The launch of the partial products and
// the reduction of its pages must see the same setting.
void flashllm_hip_set_rows_per_workgroup(int rows);
int  flashllm_hip_rows_per_workgroup(int n, int m, int split_k);

// The same product for wide B (n % 128 == 0) by workgroups of four waves that share each scattered tile.
int flashllm_hip_launch_spmm_group(void*       stream,
                                   const void* compressed_a,
                                   const int*  tile_offsets,
                                   const void* b,
                                   int         ldb,
                                   void*       out,
                                   int         m,
                                   int         n,
                                   int         k,
                                   int         split_k,
                                   int         pages);

// c[e] = rn16(sum_s float(ws[s*mn + e])), through max(., 0) first when relu != 0; requires mn % 4 == 0.
int flashllm_hip_launch_reduce(void* stream, void* c, const void* ws, long mn, int split_k, int relu);

// The same sums over the pages a launch with pages != 0 left for this (m, n, split_k): one workgroup per
// 128 x 16 block of C, on the XCD that stored the block's pages.  Requires M % 128 == 0, N as above, ws 16-byte
// and c 8-byte aligned.
int flashllm_hip_launch_reduce_pages(void* stream, void* c, const void* ws, int m, int n, int split_k, int relu);

// out[w] = id of the XCD workgroup w ran on, for a launch of `workgroups` one-wave workgroups shaped like the
// SpMM launches (a three-dimensional grid, eight wide, w counted x first, then y, then z): shows whether the
// round-robin hand-out in that order, which the placement above counts on, holds on this machine.
int flashllm_hip_launch_xcd_probe(void* stream, unsigned* out, int workgroups);

// x[i] = max(x[i], 0) over n halfs (n % 8 == 0): the activation between FFN1 and FFN2.
int flashllm_hip_launch_relu(void* stream, void* x, long n);

// dst[j*rows + i] = src[j*src_ld + i] for i < rows, j < cols (rows % 8 == 0, src_ld % 8 == 0).
int flashllm_hip_launch_take_rows(void* stream, void* dst, const void* src, int rows, int cols, int src_ld);

// offs[0..tiles+1] = TileOffsets of the device-resident dense matrix a (M x K halfs, 16-byte aligned,
// M % 128 == 0, K % 64 == 0): a count kernel and an in-place prefix sum.
int flashllm_hip_launch_tile_offsets(void* stream, const void* a, int m, int k, int* offs);

// out[offs[t]*4 ...] = the packed nonzeros of tile t in the reference's reordered layout.
int flashllm_hip_launch_encode(void* stream, const void* a, int m, int k, const int* offs, void* out);

// Waits for the stream, then *status = the FLASHLLM_ENCODE_* bits the encoder has recorded on the current device
// since they were last read, and clears them.
int flashllm_hip_encode_status(void* stream, unsigned int* status);

#ifdef __cplusplus
}
#endif
#endif
