// Tiled-CSL compression on the GPU, for weights that are already device-resident.
//
// Produces the bytes of the reference's host-side InitSparseMatrixA_API
// (csrc/SpMM_API.cu:163-360).  Its per-tile procedure is sequential (bucket the
// nonzeros by LDS bank, pad, then pop the fullest bank item by item,
// csrc/SpMM_API.cu:248-346), but its result has a closed form that every item
// can evaluate on its own:
//
//   * An item's height h in its bank is 1 + the number of nonzeros before it in
//     the bank's scan order (row-major over the tile; a bank owns two adjacent
//     columns of every row).  Padding items sit on top.
//   * "Pop the fullest bank, lowest index on ties" removes items in order of
//     (height descending, bank ascending), so the item (bank b, height h) is
//     pop number  j = sum_b' max(fill[b'] - h, 0) + #{b' < b : fill[b'] >= h}.
//   * The drain's tail-then-main fill and its last-in-first-out write-out
//     (csrc/SpMM_API.cu:306-346) map j to one output index.
//
// One workgroup of four waves per 128x64 tile: the tile is laid out bank-major
// in LDS, each wave takes eight banks, bank fills and first-zero positions
// come from 64-lane ballots, and each nonzero writes itself to its final
// place.  Three kernels: vectors per tile, an in-place prefix sum
// (TileOffsets), the encoder.
#include "spmm_launch.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

constexpr int kTileRows = 128;
constexpr int kTileCols = 64;
constexpr int kBanks    = 32;
constexpr int kPerBank  = kTileRows * kTileCols / kBanks;  // 256 positions of a tile map to one bank
constexpr int kLanes    = 64;
constexpr int kMaxFill  = kPerBank + 3;  // at most three padding items

// What the encoder found wrong since the word was last read (FLASHLLM_ENCODE_* bits), one word per GPU.  The host
// compressor returns an error in these cases; a kernel cannot, so it records them here and carries on.
__device__ unsigned int g_encode_status;

__device__ __forceinline__ void report(unsigned int what)
{
    atomicOr(&g_encode_status, what);
}

// |x| > 0 in the reference's float compare (csrc/SpMM_API.cu:183): drops +0, -0 and NaN.
__device__ __forceinline__ bool keeps(uint32_t h)
{
    const uint32_t mag = h & 0x7fffu;
    return mag != 0 && mag <= 0x7c00u;
}

__device__ __forceinline__ int lanes_below(uint64_t mask)
{
    return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0));
}

__device__ __forceinline__ const uint16_t* tile_base(const uint16_t* a, int k, int tiles_per_row, int t)
{
    const int ti = t / tiles_per_row, tj = t % tiles_per_row;
    return a + static_cast<size_t>(ti) * kTileRows * k + static_cast<size_t>(tj) * kTileCols;
}

// offs[t + 1] = 16-byte vectors of tile t (nonzeros rounded up to a multiple of four, over four)
__global__ __launch_bounds__(kLanes) void count_tiles_kernel(const uint16_t* __restrict__ a, int k, int tiles_per_row, int* __restrict__ offs)
{
    const int       t    = blockIdx.x;
    const int       lane = threadIdx.x;
    const uint16_t* base = tile_base(a, k, tiles_per_row, t);
    int             n    = 0;
#pragma unroll 4
    for (int it = 0; it < kTileRows / 8; it++) {
        const int   m = it * 8 + (lane >> 3);
        const uint4 v = *reinterpret_cast<const uint4*>(base + static_cast<size_t>(m) * k + (lane & 7) * 8);
        n += keeps(v.x & 0xffffu) + keeps(v.x >> 16) + keeps(v.y & 0xffffu) + keeps(v.y >> 16) + keeps(v.z & 0xffffu) +
             keeps(v.z >> 16) + keeps(v.w & 0xffffu) + keeps(v.w >> 16);
    }
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1)
        n += __shfl_xor(n, s);
    if (lane == 0)
        offs[t + 1] = (n + 3) / 4;
}

// in place: offs[0] = 0, offs[t + 1] = sum of the counts up to tile t, offs[tiles + 1] = offs[tiles].
// One workgroup; every thread sums a contiguous run of tiles, the 1024 run totals are scanned once.
__global__ __launch_bounds__(1024) void scan_offsets_kernel(int* __restrict__ offs, int tiles)
{
    __shared__ int part[1024];
    const int      tid = threadIdx.x;
    const int      run = (tiles + 1023) / 1024;
    const int      lo  = tid * run < tiles ? tid * run : tiles;
    const int      hi  = lo + run < tiles ? lo + run : tiles;
    int            sum = 0;
    for (int i = lo; i < hi; i++)
        sum += offs[i + 1];
    part[tid] = sum;
    __syncthreads();
    for (int s = 1; s < 1024; s <<= 1) {
        const int add = tid >= s ? part[tid - s] : 0;
        __syncthreads();
        part[tid] += add;
        __syncthreads();
    }
    int acc = part[tid] - sum;  // total of the runs before this one
    for (int i = lo; i < hi; i++) {
        acc += offs[i + 1];
        offs[i + 1] = acc;
    }
    if (tid == 1023) {
        offs[0]         = 0;
        offs[tiles + 1] = part[1023];
    }
}

// One workgroup of four waves per tile; wave w owns banks 8w .. 8w+7.
constexpr int kEncodeWaves  = 4;
constexpr int kBanksPerWave = kBanks / kEncodeWaves;

__global__ __launch_bounds__(kLanes* kEncodeWaves) void encode_tiles_kernel(const uint16_t* __restrict__ a,
                                                                            int k,
                                                                            int tiles_per_row,
                                                                            const int* __restrict__ offs,
                                                                            uint32_t* __restrict__ out)
{
    __shared__ __attribute__((aligned(16))) uint16_t vals[kBanks][kPerBank];  // bank-major: [bank][2*row + (column & 1)]
    __shared__ int                                   fill_s[kBanks];
    __shared__ int                                   first_zero_s[kBanks];    // in-tile position of the bank's first zero, -1: none
    __shared__ int                                   pad_s[3][3];             // bank, height, position of each padding item
    __shared__ int                                   npad_s;
    __shared__ int                                   above[kMaxFill + 2];     // items higher than h, over all banks
    __shared__ uint32_t                              reach[kMaxFill + 2];     // banks holding at least h items
    __shared__ uint16_t                              tail_dest[4 * kBanks];   // output index of the first 4*rem pops

    const int       t    = blockIdx.x;
    const int       tid  = threadIdx.x;
    const int       lane = tid & (kLanes - 1);
    const int       wave = tid >> 6;
    const uint16_t* base = tile_base(a, k, tiles_per_row, t);

    // Element (m, n) lives at swizzled column sw = n ^ ((m % 8) << 3) (csrc/SpMM_API.cu:252-256): the
    // 8-column chunk c of row m becomes chunk c ^ (m % 8), order inside the chunk unchanged, so the four
    // 32-bit words of a thread's 16 bytes are the four banks (c ^ (m % 8)) * 4 + w at in-bank index 2m, 2m+1.
#pragma unroll
    for (int it = 0; it < kTileRows / 32; it++) {
        const int   m  = it * 32 + (tid >> 3);
        const uint4 v  = *reinterpret_cast<const uint4*>(base + static_cast<size_t>(m) * k + (tid & 7) * 8);
        const int   b0 = ((tid & 7) ^ (m & 7)) * 4;
        *reinterpret_cast<uint32_t*>(&vals[b0 + 0][2 * m]) = v.x;
        *reinterpret_cast<uint32_t*>(&vals[b0 + 1][2 * m]) = v.y;
        *reinterpret_cast<uint32_t*>(&vals[b0 + 2][2 * m]) = v.z;
        *reinterpret_cast<uint32_t*>(&vals[b0 + 3][2 * m]) = v.w;
    }
    __syncthreads();

    // fill and first zero (in scan order) of this wave's banks
    for (int bi = 0; bi < kBanksPerWave; bi++) {
        const int b   = wave * kBanksPerWave + bi;
        int       cnt = 0, fz = -1;
#pragma unroll
        for (int q = 0; q < kPerBank / kLanes; q++) {
            const uint64_t mask = __builtin_amdgcn_ballot_w64(keeps(vals[b][q * kLanes + lane]));
            cnt += __builtin_popcountll(mask);
            if (fz < 0 && ~mask != 0)
                fz = q * kLanes + __builtin_ctzll(~mask);
        }
        if (lane == 0) {
            fill_s[b]       = cnt;
            first_zero_s[b] = fz < 0 ? -1 : (fz >> 1) * kTileCols + 2 * b + (fz & 1);
        }
    }
    __syncthreads();

    // Padding to a multiple of four: each padding item goes on top of the emptiest bank (lowest index
    // on ties) at that bank's first zero position, value 0 (csrc/SpMM_API.cu:274-287).  Wave 0 decides.
    if (wave == 0) {
        int fill = lane < kBanks ? fill_s[lane] : 0;
        int nnz  = fill;
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1)
            nnz += __shfl_xor(nnz, s);
        const int pad = (4 - nnz % 4) % 4;
        for (int p = 0; p < pad; p++) {
            int key = lane < kBanks ? (fill << 5) | lane : 0x7fffffff;
#pragma unroll
            for (int s = 32; s >= 1; s >>= 1) {
                const int other = __shfl_xor(key, s);
                key             = other < key ? other : key;
            }
            const int b = key & 31;
            if (lane == b) {
                const int fz = first_zero_s[b];
                pad_s[p][0]  = b;
                pad_s[p][1]  = fill + 1;
                pad_s[p][2]  = fz < 0 ? 0 : fz;  // the emptiest bank holds fewer than 256 items, so it has a zero
                if (fz < 0)
                    report(FLASHLLM_ENCODE_NO_ZERO);
                fill++;
            }
        }
        if (lane < kBanks)
            fill_s[lane] = fill;
        if (lane == 0)
            npad_s = pad;
    }
    __syncthreads();

    int count = 0, top = 0;
    for (int b = 0; b < kBanks; b++) {
        const int f = fill_s[b];
        count += f;
        top = f > top ? f : top;
    }
    const int vectors    = count / 4;
    const int rep        = vectors / kBanks, rem = vectors % kBanks;
    const int tail_items = rem * 4;

    for (int h = tid; h <= top + 1; h += kLanes * kEncodeWaves) {
        int      g = 0;
        uint32_t r = 0;
        for (int b = 0; b < kBanks; b++) {
            const int f = fill_s[b];
            g += f > h ? f - h : 0;
            r |= f >= h ? 1u << b : 0u;
        }
        above[h] = g;
        reach[h] = r;
    }
    // the first 4*rem pops are drained first, lane-major per pass; each lane is written back to front
    if (tid < tail_items)
        tail_dest[tid] = static_cast<uint16_t>(rep * 4 * kBanks + (tid % rem) * 4 + (3 - tid / rem));
    __syncthreads();

    uint32_t* out_tile = out + static_cast<size_t>(offs[t]) * 4;
    // Never write outside this tile's range of Compressed_A, whatever TileOffsets says: with offsets that were
    // not computed from this very matrix the output is meaningless, but it stays inside the caller's buffer.
    const int room = (offs[t + 1] - offs[t]) * 4;
    const int full = count;
    if (room != full && tid == 0)
        report(FLASHLLM_ENCODE_OFFSETS);
    count = count < room ? count : room;
    auto      emit     = [&](int b, int h, uint32_t item) {
        const int j = above[h] + __builtin_popcount(reach[h] & ((1u << b) - 1u));
        int       d;
        if (j < tail_items) {
            d = tail_dest[j];
        }
        else {
            const int q    = j - tail_items;
            const int pass = q / kBanks, ln = q % kBanks;  // pass = r*4 + v in fill order
            const int w    = rep * 4 - 1 - pass;           // its place in emission order
            d              = (w / 4) * (4 * kBanks) + ln * 4 + (w % 4);
        }
        if (d >= 0 && d < count)
            out_tile[d] = item;
        if (d < 0 || d >= full)  // cannot happen while the closed form above is right
            report(FLASHLLM_ENCODE_RANGE);
    };

    for (int bi = 0; bi < kBanksPerWave; bi++) {
        const int b     = wave * kBanksPerWave + bi;
        int       below = 0;
#pragma unroll
        for (int q = 0; q < kPerBank / kLanes; q++) {
            const int      i    = q * kLanes + lane;
            const uint32_t v    = vals[b][i];
            const bool     keep = keeps(v);
            const uint64_t mask = __builtin_amdgcn_ballot_w64(keep);
            if (keep) {
                const int      h   = below + lanes_below(mask) + 1;
                const uint32_t pos = static_cast<uint32_t>((i >> 1) * kTileCols + 2 * b + (i & 1));
                emit(b, h, v | (pos << 16));
            }
            below += __builtin_popcountll(mask);
        }
    }
    if (tid < npad_s)
        emit(pad_s[tid][0], pad_s[tid][1], static_cast<uint32_t>(pad_s[tid][2]) << 16);
}

}  // namespace

extern "C" int flashllm_hip_launch_tile_offsets(void* stream, const void* a, int m, int k, int* offs)
{
    const int   tiles_per_row = k / kTileCols;
    const int   tiles         = (m / kTileRows) * tiles_per_row;
    hipStream_t s             = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(count_tiles_kernel, dim3(tiles), dim3(kLanes), 0, s, static_cast<const uint16_t*>(a), k, tiles_per_row, offs);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return static_cast<int>(e);
    hipLaunchKernelGGL(scan_offsets_kernel, dim3(1), dim3(1024), 0, s, offs, tiles);
    return static_cast<int>(hipGetLastError());
}

extern "C" int flashllm_hip_encode_status(void* stream, unsigned int* status)
{
    hipStream_t   s = static_cast<hipStream_t>(stream);
    unsigned int* word = nullptr;
    hipError_t    e = hipGetSymbolAddress(reinterpret_cast<void**>(&word), HIP_SYMBOL(g_encode_status));
    if (e == hipSuccess)
        e = hipStreamSynchronize(s);
    if (e == hipSuccess)
        e = hipMemcpy(status, word, sizeof(unsigned int), hipMemcpyDeviceToHost);
    const unsigned int zero = 0;
    if (e == hipSuccess && *status)
        e = hipMemcpy(word, &zero, sizeof(unsigned int), hipMemcpyHostToDevice);
    return static_cast<int>(e);
}

extern "C" int flashllm_hip_launch_encode(void* stream, const void* a, int m, int k, const int* offs, void* out)
{
    const int tiles_per_row = k / kTileCols;
    const int tiles         = (m / kTileRows) * tiles_per_row;
    hipLaunchKernelGGL(encode_tiles_kernel,
                       dim3(tiles),
                       dim3(kLanes * kEncodeWaves),
                       0,
                       static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(a),
                       k,
                       tiles_per_row,
                       offs,
                       static_cast<uint32_t*>(out));
    return static_cast<int>(hipGetLastError());
}
