// Host API: argument checks, Split_K policy and the two launches behind
// SpMM_SplitK_API (reference csrc/SpMM_API.cu:55-130), plus the C++ wrappers
// that keep the reference's compressor signatures (build/SpMM_API.cuh:51-58).
#include "SpMM_API.h"
#include "flashllm_spmm.h"
#include "spmm_launch.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>

namespace {

// The N values the reference dispatches on (csrc/SpMM_API.cu:79-118).
bool supported_n(int n)
{
    return n == 8 || n == 16 || n == 32 || n == 64 || (n > 0 && n % 128 == 0);
}

int check_shape(const void* comp, const int* offs, const void* b, const void* c, int m, int n, int k, const void* ws, int split_k)
{
    if (!comp || !offs || !b || !c)
        return hipErrorInvalidValue;
    if (m <= 0 || k <= 0 || m % 128 || k % 64 || split_k < 1)
        return hipErrorInvalidValue;
    if (!supported_n(n)) {
        std::printf("MM_Sparse_API Error: Unsupported N dimension %d!\n", n);
        return hipErrorUnknown;
    }
    if (split_k > 1 && !ws)
        return hipErrorInvalidValue;
    if (reinterpret_cast<uintptr_t>(comp) % 16 || reinterpret_cast<uintptr_t>(b) % 16 || reinterpret_cast<uintptr_t>(c) % 8
        || reinterpret_cast<uintptr_t>(ws) % 16)
        return hipErrorInvalidValue;
    return hipSuccess;
}

bool known_order(int slab_order)
{
    return slab_order == FLASHLLM_SLABS_PLAIN || slab_order == FLASHLLM_SLABS_BY_WORKGROUP;
}

int launch_partials(void* stream, const void* comp, const int* offs, const void* b, int ldb, void* c, int m, int n, int k, void* ws, int split_k, int slab_order)
{
    const int pages = slab_order == FLASHLLM_SLABS_BY_WORKGROUP;
    // wide B: four waves share every scattered tile; otherwise one wave per (row tile, slice, column group)
    if (n % 128 == 0)
        return flashllm_hip_launch_spmm_group(stream, comp, offs, b, ldb, split_k == 1 ? c : ws, m, n, k, split_k, pages);
    return flashllm_hip_launch_spmm(stream, comp, offs, b, ldb, split_k == 1 ? c : ws, m, n, k, split_k, pages);
}

// SpMM_SplitK_API with B's columns ldb halfs apart (the public entry points take a dense column-major B: ldb = K)
int spmm_splitk_ldb(void* stream, const void* comp, const int* offs, const void* b, int ldb, void* c, int m, int n, int k, void* ws, int split_k)
{
    int rc = check_shape(comp, offs, b, c, m, n, k, ws, split_k);
    if (rc)
        return rc;
    if (ldb < k || ldb % 8)
        return hipErrorInvalidValue;
    rc = launch_partials(stream, comp, offs, b, ldb, c, m, n, k, ws, split_k, FLASHLLM_SLABS_BY_WORKGROUP);
    if (rc || split_k == 1)
        return rc;
    return flashllm_hip_launch_reduce_pages(stream, c, ws, m, n, split_k, 0);
}

// The reduction behind launch_partials with the same slab_order.
int reduce_slabs(void* stream, void* c, const void* ws, int m, int n, int split_k, int relu, int slab_order)
{
    if (slab_order == FLASHLLM_SLABS_BY_WORKGROUP)
        return flashllm_hip_launch_reduce_pages(stream, c, ws, m, n, split_k, relu);
    return flashllm_hip_launch_reduce(stream, c, ws, static_cast<long>(m) * n, split_k, relu);
}

}  // namespace

extern "C" {

int flashllm_spmm_partials(void*       stream,
                           const void* comp,
                           const int*  offs,
                           const void* b,
                           void*       c,
                           int         m,
                           int         n,
                           int         k,
                           void*       ws,
                           int         split_k,
                           int         slab_order)
{
    const int bad = check_shape(comp, offs, b, c, m, n, k, ws, split_k);
    if (bad)
        return bad;
    if (!known_order(slab_order))
        return hipErrorInvalidValue;
    return launch_partials(stream, comp, offs, b, k, c, m, n, k, ws, split_k, slab_order);
}

int flashllm_splitk_reduce(void* stream, void* c, const void* ws, int m, int n, int split_k, int slab_order)
{
    if (!c || !ws || m <= 0 || n <= 0 || split_k < 1 || (static_cast<long>(m) * n) % 4 || !known_order(slab_order)
        || reinterpret_cast<uintptr_t>(c) % 8 || reinterpret_cast<uintptr_t>(ws) % 8)
        return hipErrorInvalidValue;
    // pages exist only for shapes the SpMM kernels take
    if (slab_order == FLASHLLM_SLABS_BY_WORKGROUP && (m % 128 || !supported_n(n) || reinterpret_cast<uintptr_t>(ws) % 16))
        return hipErrorInvalidValue;
    return reduce_slabs(stream, c, ws, m, n, split_k, 0, slab_order);
}

int flashllm_spmm_splitk(void*       stream,
                         const void* /*A: unused, as in the reference*/,
                         const void* comp,
                         const int*  offs,
                         const void* b,
                         void*       c,
                         int         m,
                         int         n,
                         int         k,
                         void*       ws,
                         int         split_k)
{
    // the workspace is this call's own business between its two kernels: slabs by workgroup
    int rc = flashllm_spmm_partials(stream, comp, offs, b, c, m, n, k, ws, split_k, FLASHLLM_SLABS_BY_WORKGROUP);
    if (rc || split_k == 1)
        return rc;
    return reduce_slabs(stream, c, ws, m, n, split_k, 0, FLASHLLM_SLABS_BY_WORKGROUP);
}

// SpMM_SplitK_API for callers that must not allocate and hold no workspace: the slabs go to the
// library's fixed device array.
int flashllm_spmm_splitk_static(void*       stream,
                                const void* a,
                                const void* comp,
                                const int*  offs,
                                const void* b,
                                void*       c,
                                int         m,
                                int         n,
                                int         k,
                                int         split_k)
{
    void* ws = nullptr;
    if (split_k > 1) {
        // sizes first: no launch and no symbol lookup for a call that cannot fit
        if (m <= 0 || n <= 0)
            return hipErrorInvalidValue;
        const size_t need = flashllm_workspace_bytes(m, n, split_k);
        if (need > FLASHLLM_STATIC_WORKSPACE_BYTES) {
            std::fprintf(stderr,
                         "flashllm_spmm_splitk_static: Split_K*M*N*2 = %zu bytes exceeds the library's fixed slab storage of %u bytes; "
                         "use a smaller Split_K or flashllm_spmm_splitk with a workspace of your own\n",
                         need, FLASHLLM_STATIC_WORKSPACE_BYTES);
            return hipErrorInvalidValue;
        }
        const int rc = flashllm_hip_static_workspace(&ws);
        if (rc)
            return rc;
    }
    return flashllm_spmm_splitk(stream, a, comp, offs, b, c, m, n, k, ws, split_k);
}

int flashllm_device_tile_offsets(void* stream, const void* a, int m, int k, int* offs, long long* nnz_padded)
{
    if (!a || !offs || (reinterpret_cast<uintptr_t>(a) & 15u))
        return FLASHLLM_E_ARG;
    if (m <= 0 || k <= 0 || m % 128 || k % 64)
        return FLASHLLM_E_SHAPE;
    int rc = flashllm_hip_launch_tile_offsets(stream, a, m, k, offs);
    if (rc || !nnz_padded)
        return rc;
    const size_t tiles   = static_cast<size_t>(m / 128) * (k / 64);
    int          vectors = 0;
    hipStream_t  s       = static_cast<hipStream_t>(stream);
    hipError_t   e       = hipMemcpyAsync(&vectors, offs + tiles, sizeof(int), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess)
        e = hipStreamSynchronize(s);
    if (e != hipSuccess)
        return static_cast<int>(e);
    *nnz_padded = 4LL * vectors;
    return 0;
}

int flashllm_device_compress(void* stream, const void* a, int m, int k, const int* offs, void* comp)
{
    if (!a || !offs || !comp || (reinterpret_cast<uintptr_t>(a) & 15u) || (reinterpret_cast<uintptr_t>(comp) & 15u))
        return FLASHLLM_E_ARG;
    if (m <= 0 || k <= 0 || m % 128 || k % 64)
        return FLASHLLM_E_SHAPE;
    return flashllm_hip_launch_encode(stream, a, m, k, offs, comp);
}

int flashllm_device_compress_status(void* stream, unsigned int* status)
{
    if (!status)
        return hipErrorInvalidValue;
    return flashllm_hip_encode_status(stream, status);
}

size_t flashllm_workspace_bytes(int m, int n, int split_k)
{
    if (split_k <= 1 || m <= 0 || n <= 0)
        return 0;
    return static_cast<size_t>(split_k) * m * n * sizeof(uint16_t);
}

// One wave streams one (row tile, K slice, column group); a CU holds eight of them (two per SIMD, what the
// registers allow at N >= 32), so 2048 fit at once and a grid beyond that runs a second, mostly empty round
// (36864x9216, N = 32: 56 us at 7 slices = 2016 waves, 74 us at 8).  Among the Split_K values of one round the
// time follows
//     longest slice (k tiles) x (2 + resident waves per CU)  +  Split_K x (0.5 + 0.5 x (N/16) x (M/36864)):
// a wave needs a fixed time per tile plus what its neighbours on the CU take from it (LDS and issue slots
// are shared), so more slices only help while they shorten the longest slice faster than they crowd the CU
// (12288x12288: 16 slices of 12 tiles beat 20 slices of which the last has 2); every slab costs a write and
// a read of M*N halfs and a step of the reduction.  Constants fitted to the whole-call times of the
// reference's twelve weight shapes (kernel_benchmark/benchmark.sh:13-14) x N in {8,16,32,64} at 80 %
// sparsity: mean 0.3 % and at most 4.6 % above the best Split_K of each case.
int flashllm_splitk_heuristic(int m, int n, int k)
{
    if (m <= 0 || k <= 0 || n <= 0 || m % 128 || k % 64)
        return 1;
    const int kt = k / 64;
    if (n % 128 == 0) {
        // Wide B goes to the four-wave kernel: a workgroup per (row tile, slice, 128 columns), up to three resident
        // per CU (768 at once), handed out as earlier ones finish, so more than one round is no loss by itself.
        // A tile costs a workgroup 1.4 / 1.8 times as long when two / three share the CU as when it has the CU to
        // itself; every slab costs a write and a read of M*N halfs.  Fitted to whole-call times of seven of the
        // reference's weight shapes at N = 128 / 256 and Split_K 1..12: mean 1.6 %, at most 10 % above the best.
        const long   units     = static_cast<long>(m / 128) * (n / 128);
        const double slab_cost = 2.75 * 4.0 * m * n / 5e6;
        int          best      = 1;
        double       best_cost = 1e30;
        for (int s = 1; s <= 32 && s <= kt; s++) {
            const long   wgs      = units * s;
            const long   per_cu   = (wgs + 255) / 256 < 3 ? (wgs + 255) / 256 : 3;
            const double rounds   = wgs > 768 ? std::pow(wgs / 768.0, 0.8) : 1.0;
            const int    longest  = (kt - 1) / s + 1;
            const double cost     = longest * (1.0 + 0.4 * (per_cu - 1)) * rounds + (s > 1 ? s * slab_cost : 0.0);
            if (cost < best_cost) {
                best_cost = cost;
                best      = s;
            }
        }
        return best;
    }
    const int    col_groups = n <= 64 ? 1 : n / 64;
    const long   units      = static_cast<long>(m / 128) * col_groups;
    const long   slots      = 256L * 8;
    int          best       = 1;
    double       best_cost  = 1e30;
    for (int s = 1; s <= 32 && s <= kt; s++) {  // workspace sizes in existing callers assume at most 32 slabs
        if (s > 1 && units * s > slots)
            break;
        // N = 64 with eight row tiles per workgroup (what the launch does for this Split_K when its workgroups
        // fill between three quarters and all of the CUs): the same form fitted to the same twelve shapes again,
        // mean 0.5 %, at most 5.7 % above the best.  Crowding costs less there (the waves of a CU no longer fetch
        // B eight times), so the pick is mostly the largest Split_K whose workgroups fit the 256 CUs.
        const bool   by_eight = flashllm_hip_rows_per_workgroup(n, m, s) == 8;
        const double fixed    = by_eight ? 4.0 : 2.0;
        const double crowding = by_eight ? 0.5 : 1.0;
        const double per_slab = by_eight ? 1.0 + 0.125 * (n / 16.0) * (m / 36864.0) : 0.5 + 0.5 * (n / 16.0) * (m / 36864.0);
        const int    longest  = (kt - 1) / s + 1;
        const double cost     = longest * (fixed + crowding * units * s / 256.0) + (s > 1 ? s * per_slab : 0.0);
        if (cost < best_cost) {
            best_cost = cost;
            best      = s;
        }
    }
    return best;
}

// The four pruned linears of a decoder layer, in the order and with the Split_K fallbacks of the
// reference's FasterTransformer call sites (third_party/ft.patch:512-525, :615-633, :1247-1261,
// :1328-1340, :1444-1456, :1508-1521).
int flashllm_decoder_layer_linears(void*                         stream,
                                   const flashllm_decoder_layer* layer,
                                   const void*                   x,
                                   void*                         qkv_out,
                                   void*                         attn_in,
                                   void*                         attn_out,
                                   void*                         ffn_mid,
                                   void*                         y,
                                   int                           tokens,
                                   void*                         ws)
{
    if (!layer || !x || !qkv_out || !attn_out || !ffn_mid || !y)
        return hipErrorInvalidValue;
    const flashllm_sparse_weight& q = layer->qkv;
    const flashllm_sparse_weight& o = layer->attn_out;
    const flashllm_sparse_weight& f1 = layer->ffn1;
    const flashllm_sparse_weight& f2 = layer->ffn2;
    const int hidden = q.k;
    if (o.k != hidden || q.m < hidden || f1.k != o.m || f2.k != f1.m || hidden % 8 || q.m % 8)
        return hipErrorInvalidValue;
    auto split = [&](const flashllm_sparse_weight& w, int limit) {
        if (tokens > limit)
            return 1;
        return w.split_k > 0 ? w.split_k : flashllm_splitk_heuristic(w.m, tokens, w.k);
    };
    auto linear = [&](const flashllm_sparse_weight& w, const void* in, int ld_in, void* out, int limit) {
        return spmm_splitk_ldb(stream, w.nz_weights, w.tile_offsets, in, ld_in, out, w.m, tokens, w.k, ws, split(w, limit));
    };
    int rc = linear(q, x, hidden, qkv_out, 64);
    if (rc)
        return rc;
    // The attention-output linear multiplies the first `hidden` rows of every column of qkv_out: it reads them
    // where they are (columns q.m halfs apart).  A caller that also wants them contiguous passes attn_in.
    if (attn_in) {
        rc = flashllm_hip_launch_take_rows(stream, attn_in, qkv_out, hidden, tokens, q.m);
        if (rc)
            return rc;
    }
    rc = linear(o, qkv_out, q.m, attn_out, 64);
    if (rc)
        return rc;
    // FFN1 with the ReLU folded into its reduction when there is one
    const int s1 = split(f1, 128);
    rc = flashllm_spmm_partials(stream, f1.nz_weights, f1.tile_offsets, attn_out, ffn_mid, f1.m, tokens, f1.k, ws, s1, FLASHLLM_SLABS_BY_WORKGROUP);
    if (rc)
        return rc;
    rc = s1 > 1 ? reduce_slabs(stream, ffn_mid, ws, f1.m, tokens, s1, 1, FLASHLLM_SLABS_BY_WORKGROUP)
                : flashllm_hip_launch_relu(stream, ffn_mid, static_cast<long>(f1.m) * tokens);
    if (rc)
        return rc;
    return linear(f2, ffn_mid, f2.k, y, 128);
}

}  // extern "C"

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
                           int          Split_K)
{
    return static_cast<hipError_t>(flashllm_spmm_splitk(
        stream, A, Compressed_A, TileOffsets, B, C, M_Global, N_Global, K_Global, Reduction_Workspace, Split_K));
}

namespace {
int init_or_exit(int rc)
{
    if (rc == FLASHLLM_E_NOMEM) {
        std::printf("InitSparseMatrixA: Error in malloc memory from host memory!\n");
        std::exit(-1);
    }
    if (rc < 0)
        std::fprintf(stderr, "InitSparseMatrixA: rejected (code %d): M must be a multiple of 128 and K of 64\n", rc);
    return rc;
}
}  // namespace

int InitSparseMatrixA_API(half* A_h, int M, int /*N*/, int K, uint32_t** Compressed_A, int** TileOffsets)
{
    return init_or_exit(
        flashllm_init_sparse_matrix_a(reinterpret_cast<const uint16_t*>(A_h), M, K, Compressed_A, TileOffsets));
}

int InitSparseMatrixA_API_NoReorder(half* A_h, int M, int /*N*/, int K, uint32_t** Compressed_A, int** TileOffsets)
{
    return init_or_exit(flashllm_init_sparse_matrix_a_noreorder(
        reinterpret_cast<const uint16_t*>(A_h), M, K, Compressed_A, TileOffsets));
}
