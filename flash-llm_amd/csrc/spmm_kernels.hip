// gfx950 kernels of the Flash-LLM hot path and their launch functions.
//
// spmm_stream_kernel: load-as-sparse / compute-as-dense, redesigned around a
// single wave64 per workgroup (the reference uses four cooperating 32-lane
// warps and two barriers per k tile, csrc/SpMM_Kernel.cuh:179-386):
//
//   * A wave owns one 128-row tile row of A, one K slice and one group of
//     output columns.  The slice's packed nonzeros are one contiguous range
//     of Compressed_A (tiles of a tile row are stored back to back), so the
//     wave streams it as 1 KB chunks (64 lanes x 16 B, coalesced, aligned)
//     through a ring of DEPTH register slots that is always DEPTH chunks
//     ahead, whatever the tile boundaries are.
//   * Each chunk is scattered into the wave's private 128x64 fp16 tile in LDS
//     at the position stored in the item (the format's XOR-swizzled layout,
//     reference csrc/SpMM_API.cu:252-261).  When the running vector index
//     passes TileOffsets[t+1] the tile is complete: the wave reads it back as
//     16 ds_read_b128 MFMA operands (the swizzle makes every group of eight
//     lanes hit 32 distinct banks), issues v_mfma_f32_16x16x32_f16 against B
//     fragments taken straight from global/L2 (column-major B already is the
//     MFMA operand layout: 8 consecutive k per lane), and clears the tile.
//   * One wave, in-order LDS: no barrier anywhere.  Any tile density works,
//     empty tiles and empty slices included.
//
// splitk_reduce_kernel: the separate reduction over fp16 slabs
// (reference csrc/Reduction_Kernel.cuh:24-45), 16 bytes per lane per slab.
#include "spmm_launch.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

using half8   = _Float16 __attribute__((ext_vector_type(8)));
using half4   = _Float16 __attribute__((ext_vector_type(4)));
using floatx4 = float __attribute__((ext_vector_type(4)));

constexpr int kTileRows  = 128;
constexpr int kTileCols  = 64;
constexpr int kTileHalfs = kTileRows * kTileCols;
constexpr int kLanes     = 64;

__device__ __forceinline__ void clear_tile(uint16_t* tile, int lane)
{
    const uint4 zero = {0u, 0u, 0u, 0u};
    uint4*      t    = reinterpret_cast<uint4*>(tile);
#pragma unroll
    for (int i = 0; i < kTileHalfs * 2 / 16 / kLanes; i++)
        t[i * kLanes + lane] = zero;
}

// low 16 bits: fp16 value; high 16 bits: position in the swizzled tile.
__device__ __forceinline__ void scatter_item(uint16_t* tile, uint32_t item)
{
    tile[(item >> 16) & (kTileHalfs - 1)] = static_cast<uint16_t>(item);
}

template<int NB, int DEPTH>
__global__ __launch_bounds__(kLanes) void spmm_stream_kernel(const uint4* __restrict__ comp,
                                                            const int* __restrict__ offs,
                                                            const _Float16* __restrict__ B,
                                                            _Float16* __restrict__ out,
                                                            int M,
                                                            int N,
                                                            int K,
                                                            int split_k)
{
    __shared__ __attribute__((aligned(16))) uint16_t tile[kTileHalfs];

    const int lane    = threadIdx.x;
    const int r16     = lane & 15;  // row inside a 16-row block / output column
    const int g       = lane >> 4;  // which 8-wide k chunk of a 32-wide k step
    const int kt      = K / kTileCols;
    const int slice   = blockIdx.x % split_k;
    const int rowtile = blockIdx.x / split_k;
    const int col0    = blockIdx.y * (16 * NB);

    // the reference's slicing (csrc/SpMM_Kernel.cuh:196-204), clamped to K
    const int avg = (kt - 1) / split_k + 1;
    int       kb  = slice * avg;
    kb            = kb < kt ? kb : kt;
    int ke        = kb + avg;
    ke            = ke < kt ? ke : kt;

    floatx4 acc[NB][8];
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int rb = 0; rb < 8; rb++)
            acc[nb][rb] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int* toff = offs + static_cast<size_t>(rowtile) * kt;
    const int  vbeg = toff[kb];
    const int  vend = toff[ke];

    if (vend > vbeg) {
        // operand addresses: row r16 of a row block, 16-byte chunk (ks*4+g) ^ (row%8)
        const int       a_off0 = r16 * (kTileCols * 2) + ((g ^ (r16 & 7)) << 4);
        const int       a_off1 = a_off0 ^ 64;
        const _Float16* bptr[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            int n = col0 + nb * 16 + r16;
            n     = n < N ? n : N - 1;  // N == 8: lanes 8..15 compute columns nobody stores
            bptr[nb] = B + static_cast<size_t>(n) * K + g * 8;
        }

        clear_tile(tile, lane);

        const int cbase   = vbeg & ~(kLanes - 1);
        const int nchunks = (vend - cbase + kLanes - 1) / kLanes;
        const int vlast   = vend - 1;
        uint4     ring[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; d++) {
            int v   = cbase + d * kLanes + lane;
            v       = v < vlast ? v : vlast;
            ring[d] = comp[v];
        }

        int   t       = kb;
        int   tile_lo = vbeg;
        int   tile_hi = toff[t + 1];
        half8 bfrag[2][NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            bfrag[0][nb] = *reinterpret_cast<const half8*>(bptr[nb] + t * kTileCols);
            bfrag[1][nb] = *reinterpret_cast<const half8*>(bptr[nb] + t * kTileCols + 32);
        }

        bool done = false;
        for (int c0 = 0; c0 < nchunks && !done; c0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; d++) {
                const int c = c0 + d;
                if (c >= nchunks || done)
                    break;
                const uint4 cur = ring[d];
                {
                    int v   = cbase + (c + DEPTH) * kLanes + lane;
                    v       = v < vlast ? v : vlast;
                    ring[d] = comp[v];
                }
                const int vb = cbase + c * kLanes;
                const int v  = vb + lane;
                for (;;) {
                    const int hi = tile_hi < vb + kLanes ? tile_hi : vb + kLanes;
                    if (v >= tile_lo && v < hi) {
                        scatter_item(tile, cur.x);
                        scatter_item(tile, cur.y);
                        scatter_item(tile, cur.z);
                        scatter_item(tile, cur.w);
                    }
                    if (tile_hi > vb + kLanes)
                        break;  // the tile continues in the next chunk
                    if (tile_hi > tile_lo) {
                        const char* base = reinterpret_cast<const char*>(tile);
#pragma unroll
                        for (int ks = 0; ks < 2; ks++)
#pragma unroll
                            for (int rb = 0; rb < 8; rb++) {
                                const half8 a = *reinterpret_cast<const half8*>(
                                    base + rb * (16 * kTileCols * 2) + (ks ? a_off1 : a_off0));
#pragma unroll
                                for (int nb = 0; nb < NB; nb++)
                                    acc[nb][rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                        a, bfrag[ks][nb], acc[nb][rb], 0, 0, 0);
                            }
                        clear_tile(tile, lane);
                    }
                    t++;
                    if (t >= ke) {
                        done = true;
                        break;
                    }
#pragma unroll
                    for (int nb = 0; nb < NB; nb++) {
                        bfrag[0][nb] = *reinterpret_cast<const half8*>(bptr[nb] + t * kTileCols);
                        bfrag[1][nb] = *reinterpret_cast<const half8*>(bptr[nb] + t * kTileCols + 32);
                    }
                    tile_lo = tile_hi;
                    tile_hi = toff[t + 1];
                }
            }
        }
    }

    // D layout of the 16x16 MFMA: lane holds column r16, rows 4*g .. 4*g+3.
    _Float16* o = out + static_cast<size_t>(slice) * M * N + static_cast<size_t>(rowtile) * kTileRows + g * 4;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        const int n = col0 + nb * 16 + r16;
        if (n < N) {
#pragma unroll
            for (int rb = 0; rb < 8; rb++) {
                half4 h;
                h[0] = static_cast<_Float16>(acc[nb][rb][0]);
                h[1] = static_cast<_Float16>(acc[nb][rb][1]);
                h[2] = static_cast<_Float16>(acc[nb][rb][2]);
                h[3] = static_cast<_Float16>(acc[nb][rb][3]);
                *reinterpret_cast<half4*>(o + static_cast<size_t>(n) * M + rb * 16) = h;
            }
        }
    }
}

__device__ __forceinline__ void add_slab(float (&s)[8], const uint4 v)
{
    const half8 h = __builtin_bit_cast(half8, v);
#pragma unroll
    for (int j = 0; j < 8; j++)
        s[j] += static_cast<float>(h[j]);
}

__global__ __launch_bounds__(256) void splitk_reduce_kernel(uint4* __restrict__ c,
                                                           const uint4* __restrict__ ws,
                                                           long n8,
                                                           int  split_k)
{
    const long i = static_cast<long>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n8)
        return;
    float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    int   k    = 0;
    for (; k + 4 <= split_k; k += 4) {
        const uint4 v0 = ws[(k + 0) * n8 + i];
        const uint4 v1 = ws[(k + 1) * n8 + i];
        const uint4 v2 = ws[(k + 2) * n8 + i];
        const uint4 v3 = ws[(k + 3) * n8 + i];
        add_slab(s, v0);
        add_slab(s, v1);
        add_slab(s, v2);
        add_slab(s, v3);
    }
    for (; k < split_k; k++)
        add_slab(s, ws[k * n8 + i]);
    half8 h;
#pragma unroll
    for (int j = 0; j < 8; j++)
        h[j] = static_cast<_Float16>(s[j]);
    c[i] = __builtin_bit_cast(uint4, h);
}

template<int NB, int DEPTH>
int launch_spmm(hipStream_t stream, const void* comp, const int* offs, const void* b, void* out, int m, int n, int k, int split_k, int col_groups)
{
    const dim3 grid(static_cast<unsigned>(m / kTileRows) * split_k, col_groups, 1);
    hipLaunchKernelGGL((spmm_stream_kernel<NB, DEPTH>),
                       grid,
                       dim3(kLanes),
                       0,
                       stream,
                       static_cast<const uint4*>(comp),
                       offs,
                       static_cast<const _Float16*>(b),
                       static_cast<_Float16*>(out),
                       m,
                       n,
                       k,
                       split_k);
    return static_cast<int>(hipGetLastError());
}

}  // namespace

extern "C" int flashllm_hip_launch_spmm(
    void* stream, const void* comp, const int* offs, const void* b, void* out, int m, int n, int k, int split_k)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (n <= 16)
        return launch_spmm<1, 8>(s, comp, offs, b, out, m, n, k, split_k, 1);
    if (n == 32)
        return launch_spmm<2, 8>(s, comp, offs, b, out, m, n, k, split_k, 1);
    return launch_spmm<4, 8>(s, comp, offs, b, out, m, n, k, split_k, n / 64);
}

extern "C" int flashllm_hip_launch_reduce(void* stream, void* c, const void* ws, long mn, int split_k)
{
    const long n8 = mn / 8;
    hipLaunchKernelGGL(splitk_reduce_kernel,
                       dim3(static_cast<unsigned>((n8 + 255) / 256)),
                       dim3(256),
                       0,
                       static_cast<hipStream_t>(stream),
                       static_cast<uint4*>(c),
                       static_cast<const uint4*>(ws),
                       n8,
                       split_k);
    return static_cast<int>(hipGetLastError());
}
