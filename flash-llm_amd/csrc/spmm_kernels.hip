// gfx950 kernels of the Flash-LLM hot path and their launch functions.
//
// spmm_stream_kernel: load-as-sparse / compute-as-dense, redesigned around a
// single wave64 per workgroup (the reference uses four cooperating 32-lane
// warps and two barriers per k tile, csrc/SpMM_Kernel.cuh:179-386):
//
//   * A wave owns one 128-row tile row of A, one K slice and one group of
//     output columns.  The slice's packed nonzeros are one contiguous range
//     of Compressed_A (tiles of a tile row are stored back to back), so the
//     wave streams it as 1 KB chunks (64 lanes x 16 B, coalesced, aligned,
//     non-temporal) through a ring of DEPTH register slots that stays DEPTH
//     chunks ahead, whatever the tile boundaries are.
//   * Each chunk is scattered into the wave's private 128x64 fp16 tile in LDS
//     at the position stored in the item (the format's XOR-swizzled layout,
//     reference csrc/SpMM_API.cu:252-261).  When the running vector index
//     passes TileOffsets[t+1] the tile is complete: the wave takes it out of
//     LDS as 16 MFMA operands of 16 bytes per lane with ds_wrxchg2_rtn_b64,
//     which returns the operand and leaves zeros behind in one LDS instruction
//     (the swizzle makes every group of eight lanes hit 32 distinct banks), so
//     the tile is empty again for the next one without a separate clearing
//     pass, and issues v_mfma_f32_16x16x32_f16 against the B fragments of that
//     k tile (column-major B already is the MFMA operand layout: 8 consecutive
//     k per lane).  Any number of tiles may end inside one chunk (empty tiles,
//     tiles of a single vector).
//   * One wave, in-order LDS: no barrier anywhere.
//   * For N = 64 the same wave program runs eight to a workgroup, one row tile each over the same K slice, and
//     the workgroup stages B in LDS once for all eight (see the kernel's own comment); the waves meet at one
//     barrier per two k tiles and are otherwise as independent as before.
//
// Waiting for memory.  Every path through a ring stage issues exactly one
// ring load, so the compiler's wait before a slot is used is the exact
// vmcnt(DEPTH-1).  The B fragments of a k tile (column-major B already is the
// MFMA operand layout, 16 bytes per lane per fragment) are loaded straight
// into registers when the tile is opened and first used when it completes;
// the compiler places those waits as well.  Staging B through LDS instead
// (global_load_lds_dwordx4) measured the same at N <= 32 and slower at
// N = 64, where its 8 KB per wave cost two resident waves per CU.
// The operand exchanges are inline assembly (the compiler has no 16-byte LDS
// exchange) and carry their own lgkmcnt(0) inside the same statement.
//
// Placement.  The GPU has eight accelerator dies (XCDs), each with its own L2, and hands the
// workgroups of a launch to them round-robin in launch order: workgroup w runs on XCD w % 8.  The
// SpMM kernels therefore give the Split_K slices of one (row tile, column group) unit to workgroups
// eight apart, and each XCD a contiguous block of units: the partial sums of a unit all land in one L2.
//
// splitk_reduce_pages_kernel: the separate reduction (reference csrc/Reduction_Kernel.cuh:24-45) over
// slabs stored by workgroup (store_pages below), one workgroup per 128 x 16 block of C on the XCD that
// stored the block's pages, 16 bytes per lane per slice, eight slices in flight.  Where a workgroup runs
// only decides where its loads hit; the sums do not depend on it.
// splitk_reduce_kernel: the same sums over plain slabs (slab s = M*N halfs laid out like C), the
// reference's workspace layout.
#include "spmm_launch.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>

namespace {

using half8   = _Float16 __attribute__((ext_vector_type(8)));
using half4   = _Float16 __attribute__((ext_vector_type(4)));
using floatx4 = float __attribute__((ext_vector_type(4)));
using uintx4  = uint32_t __attribute__((ext_vector_type(4)));

constexpr int kTileRows  = 128;
constexpr int kTileCols  = 64;
constexpr int kTileHalfs = kTileRows * kTileCols;
constexpr int kLanes     = 64;
constexpr int kNoTile    = 0x7fffffff;
constexpr int kXcds      = 8;  // accelerator dies of an MI355X, each with its own L2

// Workgroup w of a launch <-> (unit, part), part in [0, parts): the parts of one unit go to workgroups kXcds
// apart (one XCD under round-robin hand-out), XCD x takes the units x*per_xcd .. (x+1)*per_xcd-1 with
// per_xcd = units / kXcds:  w = ((unit % per_xcd)*parts + part)*kXcds + unit / per_xcd;  the units beyond a
// multiple of kXcds are laid out plainly behind them, w = unit*parts + part.
// The launches are three-dimensional grids (kXcds, parts, layers), whose workgroups the dispatcher hands out in
// the order x fastest, then y, then z, so that w = x + kXcds*(y + parts*z) and unit and part fall out of the
// workgroup's coordinates without a division: layer z < per_xcd holds unit x*per_xcd + z, part y.  One more
// layer holds the units beyond a multiple of kXcds (and a few workgroups that find nothing to do).
struct Place {
    int      unit, part;
    unsigned w;      // position in the launch order described above
    bool     valid;  // false: a workgroup of the last layer beyond the last unit
};

__device__ __forceinline__ Place place_of_workgroup(unsigned units, unsigned parts)
{
    const unsigned per_xcd = units / kXcds;
    Place          p;
    if (blockIdx.z < per_xcd) {
        p.unit  = static_cast<int>(blockIdx.x * per_xcd + blockIdx.z);
        p.part  = static_cast<int>(blockIdx.y);
        p.w     = blockIdx.x + kXcds * (blockIdx.y + parts * blockIdx.z);
        p.valid = true;
    }
    else {
        const unsigned i = blockIdx.x + kXcds * blockIdx.y;
        p.unit           = static_cast<int>(per_xcd * kXcds + i / parts);
        p.part           = static_cast<int>(i % parts);
        p.w              = per_xcd * kXcds * parts + i;
        p.valid          = static_cast<unsigned>(p.unit) < units;
    }
    return p;
}

inline dim3 grid_of(unsigned units, unsigned parts)
{
    return dim3(kXcds, parts, units / kXcds + (units % kXcds ? 1 : 0));
}

// Slab storage by workgroup ("pages").  A page is one 128-row x 16-column block of partial sums (4 KB; 128 x 8
// and 2 KB when N == 8), kept in the order the matrix cores leave it in registers: 16-byte piece
// q*(4*cols) + g*cols + r16 holds rows 32q + 4g .. +3 and 32q + 16 + 4g .. +3 of column r16.  Page b of
// workgroup w (its position in the launch order above) of a launch of G workgroups is page b*G + w of the workspace.  Under round-robin hand-out the
// XCD that writes and later sums a page is (page index) % 8 whenever G is a multiple of 8, whatever the shape
// of the product: a workspace shared by the linears of a layer keeps every line in one L2, where stores to
// lines already present stay readable for the reduction kernel (stores that miss go to memory and do not).
template<int NBLK>
__device__ __forceinline__ void store_pages(_Float16* ws, const floatx4 (&acc)[NBLK][8], int first_page, int N, int lane, unsigned w, unsigned launch)
{
    const int    cols  = N < 16 ? 8 : 16;
    const int    r16   = lane & 15, g = lane >> 4;
    const size_t pitch = static_cast<size_t>(launch) * (cols * 16);  // uint4 between consecutive pages of a workgroup
    uint4*       page  = reinterpret_cast<uint4*>(ws) + (static_cast<size_t>(first_page) * launch + w) * (cols * 16);
    if (r16 >= cols)
        return;
#pragma unroll
    for (int nb = 0; nb < NBLK; nb++) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            half8 h;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                h[e]     = static_cast<_Float16>(acc[nb][2 * q][e]);
                h[4 + e] = static_cast<_Float16>(acc[nb][2 * q + 1][e]);
            }
            page[nb * pitch + q * (4 * cols) + g * cols + r16] = __builtin_bit_cast(uint4, h);
        }
    }
}

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

__device__ __forceinline__ void scatter_vector(uint16_t* tile, const uint4& v)
{
    scatter_item(tile, v.x);
    scatter_item(tile, v.y);
    scatter_item(tile, v.z);
    scatter_item(tile, v.w);
}

// streaming load of one 16-byte vector: the weights are read once, keep them out of the caches' way
__device__ __forceinline__ uint4 load_stream(const uint4* p)
{
    const uintx4 x = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(p));
    return uint4{x[0], x[1], x[2], x[3]};
}

__device__ __forceinline__ uint32_t lds_offset(const void* p)
{
    return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((const __attribute__((address_space(3))) void*)(p)));
}

// Takes eight 16-byte operands out of LDS (one per 16-row block, at addr[0..7]) and leaves zeros behind:
// ds_wrxchg2_rtn_b64 returns the operand and stores the zeros in one LDS instruction.  The compiler does not
// track the LDS returns of inline assembly, so the exchanges and the wait for them sit in ONE statement, with
// early-clobber outputs: no register of a[] can be read, moved or spilled while its exchange is in flight.
using uintx2 = uint32_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void take_8_and_wait(uintx4 (&a)[8], const uint32_t (&addr)[8])
{
    const uintx2 zero = {0u, 0u};
    asm volatile(
        "ds_wrxchg2_rtn_b64 %0, %8, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %1, %9, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %2, %10, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %3, %11, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %4, %12, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %5, %13, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %6, %14, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %7, %15, %16, %16 offset1:1\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(a[0]), "=&v"(a[1]), "=&v"(a[2]), "=&v"(a[3]), "=&v"(a[4]), "=&v"(a[5]), "=&v"(a[6]), "=&v"(a[7])
        : "v"(addr[0]), "v"(addr[1]), "v"(addr[2]), "v"(addr[3]), "v"(addr[4]), "v"(addr[5]), "v"(addr[6]), "v"(addr[7]), "v"(zero)
        : "memory");
}

// Sixteen operands (both 32-wide k steps): all sixteen exchanges are issued back to back, then one wait.
// Two statements, because one statement takes at most thirty operands: the first issues eight exchanges,
// the second, directly behind it, the other eight and the wait, and carries the first eight as in/out
// operands so that they cannot be used before that wait.
__device__ __forceinline__ void take_16_and_wait(uintx4 (&a0)[8], uintx4 (&a1)[8], const uint32_t (&addr0)[8], const uint32_t (&addr1)[8])
{
    const uintx2 zero = {0u, 0u};
    asm volatile(
        "ds_wrxchg2_rtn_b64 %0, %8, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %1, %9, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %2, %10, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %3, %11, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %4, %12, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %5, %13, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %6, %14, %16, %16 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %7, %15, %16, %16 offset1:1"
        : "=&v"(a0[0]), "=&v"(a0[1]), "=&v"(a0[2]), "=&v"(a0[3]), "=&v"(a0[4]), "=&v"(a0[5]), "=&v"(a0[6]), "=&v"(a0[7])
        : "v"(addr0[0]), "v"(addr0[1]), "v"(addr0[2]), "v"(addr0[3]), "v"(addr0[4]), "v"(addr0[5]), "v"(addr0[6]), "v"(addr0[7]), "v"(zero)
        : "memory");
    asm volatile(
        "ds_wrxchg2_rtn_b64 %0, %16, %24, %24 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %1, %17, %24, %24 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %2, %18, %24, %24 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %3, %19, %24, %24 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %4, %20, %24, %24 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %5, %21, %24, %24 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %6, %22, %24, %24 offset1:1\n\t"
        "ds_wrxchg2_rtn_b64 %7, %23, %24, %24 offset1:1\n\t"
        "s_waitcnt lgkmcnt(0)"
        : "=&v"(a1[0]), "=&v"(a1[1]), "=&v"(a1[2]), "=&v"(a1[3]), "=&v"(a1[4]), "=&v"(a1[5]), "=&v"(a1[6]), "=&v"(a1[7]),
          "+v"(a0[0]), "+v"(a0[1]), "+v"(a0[2]), "+v"(a0[3]), "+v"(a0[4]), "+v"(a0[5]), "+v"(a0[6]), "+v"(a0[7])
        : "v"(addr1[0]), "v"(addr1[1]), "v"(addr1[2]), "v"(addr1[3]), "v"(addr1[4]), "v"(addr1[5]), "v"(addr1[6]), "v"(addr1[7]), "v"(zero)
        : "memory");
}

// One 1 KB piece of B (eight columns x the 64 k of a k tile, i.e. eight whole 128-byte lines) from global memory
// straight into LDS, without passing through registers: lane l delivers its 16 bytes at lds + 16*l.  The wave's
// vector-memory counter counts it like any load; the compiler does not know of it.
__device__ __forceinline__ void load_to_lds_16(const void* src, uint32_t lds)
{
    uint32_t saved;
    asm volatile(
        "s_mov_b32 %0, m0\n\t"
        "s_mov_b32 m0, %2\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, off\n\t"
        "s_mov_b32 m0, %0"
        : "=&s"(saved)
        : "v"(src), "s"(lds)
        : "memory");
}

// NB: 16-column blocks per wave (1 for N <= 16, 2 for N = 32, 4 for N >= 64).
// DEPTH: ring slots = 1 KB chunks in flight per wave.
// W: waves per workgroup.  W == 1: a wave is a workgroup and fetches its own B fragments from L2.
//
// W > 1 (N = 32 and 64, where the 2*NB fragment loads per tile and wave are what holds the one-wave form back):
// the W waves of a workgroup take the SAME K slice of W consecutive row tiles, so they need the same B, and B
// is staged in LDS once per workgroup, as the reference stages one B tile per thread block for all of its
// warps (csrc/MatMulUtilities.cuh:39-75).  Every wave keeps its private tile and its own stream and runs
// freely; the waves meet once per window of G k tiles:
//   * the window's B (G k tiles x 16*NB columns x 128 bytes) is fetched as whole 128-byte lines by
//     load_to_lds_16, each wave two of the window's 1 KB pieces; piece (l % 8) ^ (l / 8) of a line goes to
//     slot l % 8 of its column, so the operand reads below are free of bank conflicts;
//   * two windows of LDS alternate.  Before a wave reads the first fragment of window w it makes sure its own
//     pieces of w have landed (they were requested a whole window earlier: after DEPTH younger ring loads the
//     ring's own waits have already covered them, otherwise it drains) and meets the others at a barrier;
//     past the barrier everybody has finished reading window w-1, whose LDS then receives window w+1;
//   * a tile's fragments are 2*NB plain 16-byte LDS reads issued with the operand exchanges.
// A wave without nonzeros in the slice, or beyond the last row tile, still fetches its pieces and attends
// every barrier.
template<int NB, int DEPTH, int W, int G>
__global__ __launch_bounds__(kLanes* W) void spmm_stream_kernel(const uint4* __restrict__ comp,
                                                                const int* __restrict__ offs,
                                                                const _Float16* __restrict__ B,
                                                                int ldb,
                                                                _Float16* __restrict__ out,
                                                                int M,
                                                                int N,
                                                                int K,
                                                                int split_k,
                                                                int col_groups,
                                                                int pages,
                                                                unsigned units)
{
    constexpr int kBTile  = NB * 2048;                     // bytes of B per k tile in LDS: 16*NB columns x 128
    constexpr int kBBytes = W > 1 ? 2 * G * kBTile : 0;    // two windows
    constexpr int kPieces = W > 1 ? G * 2 * NB / W : 0;    // 1 KB pieces of a window each wave fetches
    static_assert(W == 1 || (G * 2 * NB) % W == 0, "the pieces of a window must divide among the waves");
    static_assert((G & (G - 1)) == 0, "G must be a power of two");
    // the windows of B first (the LDS address of a direct load travels in M0 and stays small), then the waves' tiles
    __shared__ __attribute__((aligned(16))) unsigned char lds[kBBytes + W * kTileHalfs * 2];

    const int lane = threadIdx.x & (kLanes - 1);
    const int wave = W > 1 ? __builtin_amdgcn_readfirstlane(threadIdx.x / kLanes) : 0;
    uint16_t* const tile = reinterpret_cast<uint16_t*>(lds + kBBytes) + wave * kTileHalfs;
    const int r16  = lane & 15;  // row inside a 16-row block / output column
    const int g    = lane >> 4;  // which 8-wide k chunk of a 32-wide k step
    const int kt   = K / kTileCols;
    // W == 1: unit = (row tile, column group), column group fastest: the column groups of a row tile read the
    // same weights and meet in one L2.  W > 1: unit = W consecutive row tiles, all 16*NB columns.
    const Place place = place_of_workgroup(units, split_k);
    if (!place.valid)
        return;
    const int  unit = place.unit, slice = place.part;
    const int  rowtile   = W > 1 ? unit * W + wave : unit / col_groups;
    const int  col0      = W > 1 ? 0 : (unit % col_groups) * (16 * NB);
    const bool have_rows = W == 1 || rowtile < M / kTileRows;
    // HW_ID.wave_id: which of the SIMD's wave slots this wave sits in (bit 0 tells the two apart)
    const int wave_slot = __builtin_amdgcn_s_getreg(4 | (0 << 6) | (3 << 11)) & 1;

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

    const int* toff = offs + static_cast<size_t>(have_rows ? rowtile : 0) * kt;
    const int  vbeg = toff[kb];
    const int  vend = have_rows ? toff[ke] : vbeg;

    // ---- the shared B windows (W > 1 only) ----
    const uint32_t bwin_lds = lds_offset(&lds[0]);
    int            since    = 0;  // ring loads this wave has issued since it last requested pieces of B
    // this wave's pieces of window w: piece j is k tile j / (2*NB) of the window, columns 8*(j % (2*NB)) .. +7
    auto fetch_window = [&](int w) {
#pragma unroll
        for (int i = 0; i < kPieces; i++) {
            const int j  = wave * kPieces + i;
            int       tk = kb + w * G + j / (2 * NB);
            tk           = tk < ke ? tk : ke - 1;  // past the slice's end: any valid lines, nobody reads them
            const int c  = 8 * (j % (2 * NB)) + (lane >> 3);
            load_to_lds_16(B + static_cast<size_t>(c) * ldb + tk * kTileCols + (((lane & 7) ^ (lane >> 3)) << 3),
                           bwin_lds + (w & 1) * (G * kBTile) + j * 1024);
        }
        since = 0;
    };
    // before the first read of window w
    auto open_window = [&](int w) {
        // At most DEPTH loads still in flight: with DEPTH ring loads younger than this wave's pieces of window w
        // those have landed (loads complete in order); the ring itself is rarely touched by this wait, a slot is
        // only refilled after the wait for its previous contents.  With fewer younger loads: drain.
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DEPTH) : "memory");
        if (since < DEPTH)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        asm volatile("s_barrier" ::: "memory");
        if (kb + (w + 1) * G < ke)
            fetch_window(w + 1);
    };
    if constexpr (W > 1) {
        if (kb < ke)
            fetch_window(0);
    }

    if (vend > vbeg) {
        // operand addresses: row r16 of a row block, 16-byte chunk (ks*4+g) ^ (row%8)
        const int       a_off0 = r16 * (kTileCols * 2) + ((g ^ (r16 & 7)) << 4);
        const int       a_off1 = a_off0 ^ 64;
        const _Float16* bptr[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            int n    = col0 + nb * 16 + r16;
            n        = n < N ? n : N - 1;  // N == 8: lanes 8..15 compute columns nobody stores
            bptr[nb] = B + static_cast<size_t>(n) * ldb + g * 8;
        }
        const uint32_t tile_lds = lds_offset(tile);
        uint32_t       a_addr0[8], a_addr1[8];  // LDS byte addresses of this lane's operands: k step 0 / 1 of row block rb
#pragma unroll
        for (int rb = 0; rb < 8; rb++) {
            a_addr0[rb] = tile_lds + rb * (16 * kTileCols * 2) + a_off0;
            a_addr1[rb] = tile_lds + rb * (16 * kTileCols * 2) + a_off1;
        }
        half8          bfrag[2][NB];  // B fragments of the open tile (W == 1) / of the tile being multiplied
        auto           load_b = [&](int t) {
#pragma unroll
            for (int ks = 0; ks < 2; ks++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    bfrag[ks][nb] = *reinterpret_cast<const half8*>(bptr[nb] + t * kTileCols + ks * 32);
        };
        // W > 1: the fragments of k step ks of tile t out of its window: column 16*nb + r16 holds piece
        // (4*ks + g) at slot (4*ks + g) ^ (r16 % 8), the same offsets as an operand of A inside a row block
        auto read_b = [&](int t, int ks) {
            const int            i    = t - kb;
            const unsigned char* base = lds + ((i / G) & 1) * (G * kBTile) + (i % G) * kBTile + (ks ? a_off1 : a_off0);
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
                bfrag[ks][nb] = *reinterpret_cast<const half8*>(base + nb * 2048);
        };

        clear_tile(tile, lane);

        const int cbase   = vbeg & ~(kLanes - 1);
        const int nchunks = (vend - cbase + kLanes - 1) / kLanes;
        const int vlast   = vend - 1;
        uint4     ring[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; d++)
            ring[d] = uint4{0u, 0u, 0u, 0u};

        int t = kb, tile_lo = vbeg, tile_hi = toff[kb + 1], next_hi = toff[kb + 2];
        if constexpr (W == 1)
            load_b(t);

        // Chunks -DEPTH .. -1 only fill the ring: none of their lanes reaches tile_lo, and a tile can
        // only "end" there when it is empty.
        for (int c0 = -DEPTH; c0 < nchunks; c0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; d++) {
                const int v  = cbase + (c0 + d) * kLanes + lane;  // this lane's vector
                const int ve = cbase + (c0 + d + 1) * kLanes;     // end of the chunk
                {
                    const uint4 cur = ring[d];
                    if (v >= tile_lo && v < tile_hi)
                        scatter_vector(tile, cur);
                    while (tile_hi <= ve) {  // a tile ends inside, or exactly at the end of, this chunk
                        if constexpr (W > 1) {
                            if (((t - kb) & (G - 1)) == 0)
                                open_window((t - kb) / G);
                        }
                        if (tile_hi > tile_lo) {
                            // NB <= 2: all 16 operands in one batch.  NB == 4: one 32-wide k step at a time, which
                            // keeps the kernel within 256 VGPRs (two waves per SIMD).
                            if constexpr (NB >= 4) {
#pragma unroll
                                for (int ks = 0; ks < 2; ks++) {
                                    uintx4 a[8];
                                    if constexpr (W > 1)
                                        read_b(t, ks);
                                    take_8_and_wait(a, ks ? a_addr1 : a_addr0);
#pragma unroll
                                    for (int rb = 0; rb < 8; rb++)
#pragma unroll
                                        for (int nb = 0; nb < NB; nb++)
                                            acc[nb][rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                                __builtin_bit_cast(half8, a[rb]), bfrag[ks][nb], acc[nb][rb], 0, 0, 0);
                                }
                            }
                            else {
                                uintx4 a0[8], a1[8];
                                if constexpr (W > 1) {
                                    read_b(t, 0);
                                    read_b(t, 1);
                                }
                                take_16_and_wait(a0, a1, a_addr0, a_addr1);
#pragma unroll
                                for (int rb = 0; rb < 8; rb++)
#pragma unroll
                                    for (int nb = 0; nb < NB; nb++)
                                        acc[nb][rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                            __builtin_bit_cast(half8, a0[rb]), bfrag[0][nb], acc[nb][rb], 0, 0, 0);
#pragma unroll
                                for (int rb = 0; rb < 8; rb++)
#pragma unroll
                                    for (int nb = 0; nb < NB; nb++)
                                        acc[nb][rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                            __builtin_bit_cast(half8, a1[rb]), bfrag[1][nb], acc[nb][rb], 0, 0, 0);
                            }
                        }
                        t++;
                        tile_lo = tile_hi;
                        // The SIMD's arbiter serves its older wave first, which leaves the younger of the two
                        // resident waves about 17 % slower; taking turns at raised priority, one tile each,
                        // evens their finishing times.  The tile counters of the two waves are not in step:
                        // the younger wave's raised level is the higher one, so it wins when both are raised
                        // as the older one wins when neither is.
                        if ((t ^ wave_slot) & 1) {
                            if (wave_slot)
                                __builtin_amdgcn_s_setprio(2);
                            else
                                __builtin_amdgcn_s_setprio(1);
                        }
                        else
                            __builtin_amdgcn_s_setprio(0);
                        if (t < ke) {
                            if constexpr (W == 1)
                                load_b(t);
                            tile_hi = next_hi;
                            next_hi = toff[t + 2];
                            if (v >= tile_lo && v < tile_hi)  // the rest of this chunk opens the next tile
                                scatter_vector(tile, cur);
                        }
                        else {  // nothing left: the remaining stages are no-ops
                            tile_lo = kNoTile;
                            tile_hi = kNoTile;
                        }
                    }
                }
                {
                    int vn  = v + DEPTH * kLanes;
                    vn      = vn < vlast ? vn : vlast;
                    ring[d] = load_stream(comp + vn);
                    if constexpr (W > 1)
                        since++;
                }
            }
        }
    }
    else if constexpr (W > 1) {
        // nothing to multiply: this wave's part in the windows remains
        for (int w = 0; w * G < ke - kb; w++)
            open_window(w);
    }

    if (!have_rows)
        return;
    // D layout of the 16x16 MFMA: lane holds column r16, rows 4*g .. 4*g+3 of each 16-row block.
    if (pages) {  // a workgroup's pages: wave by wave, NB each
        store_pages<NB>(out, acc, wave * NB, N, lane, place.w, units * split_k);
        return;
    }
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

// ------------------------------------------------------------------------------------------------
// spmm_group_kernel: the kernel for wide B (N a multiple of 128).  The one-wave kernel above pays the whole
// cost of a tile (scatter, take it out of LDS, clear it) once per 64 output columns; here four waves share it,
// as the reference's four warps share one A tile for its wide-N configurations (csrc/SpMM_API.cu:97-112).
// A workgroup of four waves owns (row tile, K slice, group of 4*16*NBW columns):
//   * all four stream and scatter: round r of a tile gives wave w the 64 vectors (r*4 + w)*64 .. of the
//     tile's range of Compressed_A; the vectors of the next kAhead tiles are in flight per wave;
//   * each wave multiplies the whole tile by its own 16*NBW columns: 16 plain 16-byte operand reads
//     (no clearing: the tile has four readers), 16*NBW MFMAs; its B operands are fetched a tile ahead as
//     whole 128-byte lines and turned into the MFMA layout through LDS (stage_b);
//   * three tile buffers rotate, so one barrier per tile is enough: in step t a wave reads tile t from one
//     buffer (complete since the previous barrier), scatters its part of tile t+1 into the second and clears
//     its quarter of the third (read by everybody before the previous barrier).
// Every step issues the same number of global loads in the same order (R stream loads and 2*NBW loads of B
// lines, addresses clamped instead of skipped) and every round has all three steps, so the waits the compiler
// places are exact counts that never drain the stream, and the accumulators stay where they are (with early
// exits from the unrolled round the register allocation more than doubled).  A tile with more than R*256
// vectors takes its remaining rounds on a slow path.
constexpr int kGroupWaves   = 4;
constexpr int kGroupThreads = kGroupWaves * kLanes;
constexpr int kAhead        = 3;  // tiles of the stream in flight per wave = the three buffers' rotation

template<int NBW, int R>
__device__ __forceinline__ void spmm_group_body(uint16_t (&tiles)[3][kTileHalfs],
                                                const uint4* __restrict__ comp,
                                                const int* __restrict__ toff,
                                                const _Float16* __restrict__ B,
                                                int ldb,
                                                _Float16* __restrict__ o,
                                                int M,
                                                int N,
                                                int K,
                                                int kb,
                                                int ke,
                                                int col0,
                                                int vmax,
                                                int pages,
                                                unsigned w,
                                                unsigned launch)
{
    const int lane = threadIdx.x & (kLanes - 1);
    const int wave = threadIdx.x / kLanes;

    floatx4 acc[NBW][8];
#pragma unroll
    for (int nb = 0; nb < NBW; nb++)
#pragma unroll
        for (int rb = 0; rb < 8; rb++)
            acc[nb][rb] = floatx4{0.f, 0.f, 0.f, 0.f};

    // B is fetched whole 128-byte lines at a time: load i of a tile takes the 64 k of columns col0 + 8i .. + 7,
    // eight lanes per column.  (A load of 16 columns x 64 bytes, which is what the MFMA operand layout asks
    // for, takes twice the requests for the same bytes and measured slower.)  Lane l fetches 16-byte piece
    // (l % 8) ^ (l / 8) of its column, so that the staging below reads back without bank conflicts.
    const _Float16* bptr = B + static_cast<size_t>(col0 + (lane >> 3)) * ldb + (((lane & 7) ^ (lane >> 3)) << 3);
    // operand of this lane inside a 16-row block: row r16 = lane % 16, 16-byte chunk (ks*4 + lane/16) ^ (row%8)
    const int a_off0 = (lane & 15) * (kTileCols * 2) + (((lane >> 4) ^ (lane & 7)) << 4);
    const int a_off1 = a_off0 ^ 64;

    uint4 ring[kAhead][R];  // ring[p][r]: this wave's vectors of round r of the tile in slot p
    int   slot_lo[kAhead], slot_n[kAhead];
    uintx4 braw[2 * NBW];  // braw[i]: columns col0 + 8i .. + 7 of B for the next tile, as loaded
    half8  bfrag[2][NBW];  // the MFMA B operands of the current tile

    auto tile_range = [&](int t, int& lo, int& n) {  // tiles at or beyond ke are empty
        const int a = t < ke ? t : ke, b = t + 1 < ke ? t + 1 : ke;
        lo          = toff[a];
        n           = toff[b] - lo;
    };
    int  ahead_lo, ahead_n;  // range of the tile the next request is for, fetched one request earlier
    auto request = [&](auto pp, int t) {  // this wave's R loads of tile t into slot p, always issued
        constexpr int p = decltype(pp)::value;
        slot_lo[p]      = ahead_lo;
        slot_n[p]       = ahead_n;
        tile_range(t + 1, ahead_lo, ahead_n);  // requests go tile by tile, so the next one is for t + 1
#pragma unroll
        for (int r = 0; r < R; r++) {
            int v      = slot_lo[p] + (r * kGroupWaves + wave) * kLanes + lane;
            v          = v < vmax ? v : vmax;
            ring[p][r] = load_stream(comp + v);
        }
    };
    auto load_b = [&](int t) {  // always issued: past the end the last tile's lines are fetched again
        const int tc = t < ke ? t : ke - 1;
#pragma unroll
        for (int i = 0; i < 2 * NBW; i++)
            braw[i] = *reinterpret_cast<const uintx4*>(bptr + static_cast<size_t>(i) * 8 * ldb + tc * kTileCols);
    };
    // The lines go to LDS as they are (lane l -> piece l of load i, i.e. column 8i + l/8 at 128 bytes per
    // column) and are read back at once in the operand layout of the MFMA: lane (r16, g) takes piece
    // (4*ks + g) ^ (r16 % 8) of column 16*nb + r16.  The 4 KB this needs are the wave's own quarter of the
    // tile buffer it is about to clear (nobody else touches that quarter between two meetings).  One wave,
    // in-order LDS: no barrier between write, read and the clearing that follows.
    // blank: a tile past the slice's end multiplies by zeros, whatever B holds
    auto stage_b = [&](uint16_t* buf, bool blank) {
        uintx4* mine = reinterpret_cast<uintx4*>(buf) + wave * (kTileHalfs * 2 / 16 / kGroupWaves);
        static_assert(2 * NBW * kLanes <= kTileHalfs * 2 / 16 / kGroupWaves, "a wave's B lines must fit its quarter of a tile buffer");
#pragma unroll
        for (int i = 0; i < 2 * NBW; i++)
            mine[i * kLanes + lane] = blank ? uintx4{0u, 0u, 0u, 0u} : braw[i];
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int nb = 0; nb < NBW; nb++)
                bfrag[ks][nb] = __builtin_bit_cast(half8, mine[(nb * 16 + (lane & 15)) * 8 + ((ks * 4 + (lane >> 4)) ^ (lane & 7))]);
    };
    auto scatter_slot = [&](auto pp, uint16_t* buf) {
        constexpr int p = decltype(pp)::value;
#pragma unroll
        for (int r = 0; r < R; r++)
            if ((r * kGroupWaves + wave) * kLanes + lane < slot_n[p])
                scatter_vector(buf, ring[p][r]);
        // a tile longer than R rounds: the rest straight from memory
        for (int r = R; r * kGroupThreads < slot_n[p]; r++) {
            const int i = (r * kGroupWaves + wave) * kLanes + lane;
            if (i < slot_n[p])
                scatter_vector(buf, load_stream(comp + slot_lo[p] + i));
        }
    };
    auto clear_quarter = [&](uint16_t* buf) {
        uint4 zero = {0u, 0u, 0u, 0u};
        asm volatile("" : "+v"(zero.x), "+v"(zero.y), "+v"(zero.z), "+v"(zero.w));  // made here, not kept in registers round the loop
        uint4* q = reinterpret_cast<uint4*>(buf) + wave * (kTileHalfs * 2 / 16 / kGroupWaves);
#pragma unroll
        for (int i = 0; i < kTileHalfs * 2 / 16 / kGroupThreads; i++)
            q[i * kLanes + lane] = zero;
    };
    constexpr int kAtOnce = 8;
    auto          multiply = [&](const half8 (&bf)[2][NBW], const uint16_t* buf) {
        const char* base = reinterpret_cast<const char*>(buf);
#pragma unroll
        for (int ks = 0; ks < 2; ks++)
#pragma unroll
            for (int part = 0; part < 8 / kAtOnce; part++) {  // a few row blocks at a time keeps the operand registers few
                half8 a[kAtOnce];
#pragma unroll
                for (int i = 0; i < kAtOnce; i++)
                    a[i] = *reinterpret_cast<const half8*>(base + (part * kAtOnce + i) * (16 * kTileCols * 2) + (ks ? a_off1 : a_off0));
#pragma unroll
                for (int i = 0; i < kAtOnce; i++)
#pragma unroll
                    for (int nb = 0; nb < NBW; nb++)
                        // in place (the accumulator is an in/out operand): left to itself the compiler gives the
                        // unrolled steps accumulators of their own and runs out of registers moving between them
                        asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[nb][part * kAtOnce + i]) : "v"(a[i]), "v"(bf[ks][nb]));
            }
    };
    // all LDS traffic of this wave has landed, then everybody meets: nothing here waits for global memory
    auto meet = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // prologue: request kAhead tiles, clear the buffers, scatter the first tile
    tile_range(kb, ahead_lo, ahead_n);
    request(std::integral_constant<int, 0>{}, kb + 0);
    request(std::integral_constant<int, 1>{}, kb + 1);
    request(std::integral_constant<int, 2>{}, kb + 2);
    load_b(kb);
    clear_quarter(tiles[0]);
    clear_quarter(tiles[1]);
    meet();
    scatter_slot(std::integral_constant<int, 0>{}, tiles[0]);
    request(std::integral_constant<int, 0>{}, kb + kAhead);
    clear_quarter(tiles[2]);
    meet();

    // step j of a round of three: tile t sits in buffer j and came from slot j; its B lines were requested a
    // step ago and go through LDS first.  The MFMAs (their A operands have been complete since the last
    // meeting) run while the wave requests the next tile's B lines and scatters the next tile.
    // Rounds are always whole: a step past the slice's end finds an empty (all-zero) buffer, scatters nothing,
    // and multiplies zeros by zeros (its fragments are blanked, so that an Inf or NaN in B cannot leak in).
    auto step = [&](auto jj, int t) {
        constexpr int j = decltype(jj)::value, next = (j + 1) % kAhead;
        stage_b(tiles[(j + 2) % 3], t >= ke);
        multiply(bfrag, tiles[j]);
        load_b(t + 1);
        scatter_slot(std::integral_constant<int, next>{}, tiles[next]);  // tile t + 1 (empty past the end)
        request(std::integral_constant<int, next>{}, t + 1 + kAhead);
        clear_quarter(tiles[(j + 2) % 3]);
        meet();
    };
    for (int t = kb; t < ke; t += kAhead) {
        step(std::integral_constant<int, 0>{}, t);
        step(std::integral_constant<int, 1>{}, t + 1);
        step(std::integral_constant<int, 2>{}, t + 2);
    }

    // the MFMAs came from inline assembly, where the compiler does not pad for the matrix core's write-back
    // latency: give the last ones time before the accumulators are read
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    // D layout of the 16x16 MFMA: lane holds column r16, rows 4*g .. 4*g+3 of each 16-row block.  The lane's
    // coordinates are derived afresh (through an opaque statement) so that nothing is carried round the loop for this.
    int lane_again = threadIdx.x & (kLanes - 1);
    asm volatile("" : "+v"(lane_again));
    if (pages) {  // o is the workspace itself here; this wave's NBW pages follow those of the waves before it
        store_pages<NBW>(o, acc, static_cast<int>(threadIdx.x / kLanes) * NBW, N, lane_again, w, launch);
        return;
    }
    const int r16 = lane_again & 15, g = lane_again >> 4;
#pragma unroll
    for (int nb = 0; nb < NBW; nb++) {
        const int n = col0 + nb * 16 + r16;
        if (n < N) {
#pragma unroll
            for (int rb = 0; rb < 8; rb++) {
                half4 h;
                h[0] = static_cast<_Float16>(acc[nb][rb][0]);
                h[1] = static_cast<_Float16>(acc[nb][rb][1]);
                h[2] = static_cast<_Float16>(acc[nb][rb][2]);
                h[3] = static_cast<_Float16>(acc[nb][rb][3]);
                *reinterpret_cast<half4*>(o + static_cast<size_t>(n) * M + g * 4 + rb * 16) = h;
            }
        }
    }
}

template<int NBW>
__global__ __launch_bounds__(kGroupThreads, 3) void spmm_group_kernel(const uint4* __restrict__ comp,
                                                                  const int* __restrict__ offs,
                                                                  const _Float16* __restrict__ B,
                                                                  int ldb,
                                                                  _Float16* __restrict__ out,
                                                                  int M,
                                                                  int N,
                                                                  int K,
                                                                  int split_k,
                                                                  int col_groups,
                                                                  int pages,
                                                                  unsigned units)
{
    __shared__ __attribute__((aligned(16))) uint16_t tiles[3][kTileHalfs];
    const int   kt    = K / kTileCols;
    const Place place = place_of_workgroup(units, split_k);
    if (!place.valid)
        return;
    const int unit = place.unit, slice = place.part;
    const int rowtile = unit / col_groups;
    const int col0    = (unit % col_groups) * (kGroupWaves * 16 * NBW) + (threadIdx.x / kLanes) * (16 * NBW);
    // the reference's slicing (csrc/SpMM_Kernel.cuh:196-204), clamped to K
    const int avg = (kt - 1) / split_k + 1;
    int       kb  = slice * avg;
    kb            = kb < kt ? kb : kt;
    int ke        = kb + avg;
    ke            = ke < kt ? ke : kt;
    const int* toff = offs + static_cast<size_t>(rowtile) * kt;
    _Float16*  o    = pages ? out : out + static_cast<size_t>(slice) * M * N + static_cast<size_t>(rowtile) * kTileRows;
    // last vector any load of this slice may touch (clamped loads re-read it)
    int vmax = toff[ke] - 1;
    vmax     = vmax > 0 ? vmax : 0;
    // rounds held in registers per tile: two cover 512 vectors (8 KB, tiles up to a quarter full), three 768
    const int whole = offs[static_cast<size_t>(M / kTileRows) * kt];  // vectors in the matrix
    // An empty matrix has no vector 0: its callers allocate one 4-byte element (reference
    // kernel_benchmark/spmm_test.cu:258-260).  The always-issued loads then read the first 16 bytes of B
    // instead (always there, 16-byte aligned); nothing of them is scattered, every tile has zero vectors.
    if (whole == 0)
        comp = reinterpret_cast<const uint4*>(B);
    if (whole <= 440LL * (M / kTileRows) * kt)
        spmm_group_body<NBW, 2>(tiles, comp, toff, B, ldb, o, M, N, K, kb, ke, col0, vmax, pages, place.w, units * split_k);
    else
        spmm_group_body<NBW, 3>(tiles, comp, toff, B, ldb, o, M, N, K, kb, ke, col0, vmax, pages, place.w, units * split_k);
}

__device__ __forceinline__ void add_slab(float (&s)[4], const uint2 v)
{
    const half4 h = __builtin_bit_cast(half4, v);
#pragma unroll
    for (int j = 0; j < 4; j++)
        s[j] += static_cast<float>(h[j]);
}

// C[e] = rn16(sum over slabs, in slab order, of float(ws[s*MN + e])).  Eight bytes per lane and up to
// eight slabs in flight per lane: the slabs are small (M*N halfs), so the kernel is latency bound and
// wants many independent loads rather than wide ones.
// RELU: the sums go through max(x, 0) before rounding (the activation after FFN1, saving a pass over C)
template<bool RELU>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(uint2* __restrict__ c,
                                                           const uint2* __restrict__ ws,
                                                           long n4,
                                                           int  split_k)
{
    const long i = static_cast<long>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n4)
        return;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    int   k    = 0;
    for (; k + 8 <= split_k; k += 8) {
        uint2 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++)
            v[j] = ws[(k + j) * n4 + i];
#pragma unroll
        for (int j = 0; j < 8; j++)
            add_slab(s, v[j]);
    }
    if (k + 4 <= split_k) {
        uint2 v[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
            v[j] = ws[(k + j) * n4 + i];
#pragma unroll
        for (int j = 0; j < 4; j++)
            add_slab(s, v[j]);
        k += 4;
    }
    {
        uint2 v[3];
        const int left = split_k - k;  // 0..3
#pragma unroll
        for (int j = 0; j < 3; j++)
            if (j < left)
                v[j] = ws[(k + j) * n4 + i];
#pragma unroll
        for (int j = 0; j < 3; j++)
            if (j < left)
                add_slab(s, v[j]);
    }
    half4 h;
#pragma unroll
    for (int j = 0; j < 4; j++)
        h[j] = static_cast<_Float16>(RELU && !(s[j] > 0.f) ? 0.f : s[j]);
    c[i] = __builtin_bit_cast(uint2, h);
}

// The same sums over slabs stored by workgroup (store_pages), one workgroup per 128-row x 16-column block of C.
// pages_per_unit: pages one workgroup of the SpMM launch stores (its NB, or 4*NBW in the four-wave kernel);
// spmm_grid: workgroups of that launch.  The workgroup order mirrors the SpMM kernel's, so a block is summed
// on the XCD that stored its pages.  Thread t takes 16-byte piece t of each slice's page.
template<bool RELU>
__global__ __launch_bounds__(256) void splitk_reduce_pages_kernel(_Float16* __restrict__ c,
                                                                 const uint4* __restrict__ ws,
                                                                 int M,
                                                                 int N,
                                                                 int split_k,
                                                                 int pages_per_unit,
                                                                 int rows_per_unit,
                                                                 int col_groups,
                                                                 unsigned units)
{
    const int cols = N < 16 ? 8 : 16;
    const int t    = threadIdx.x;
    if (t >= cols * 16)  // N == 8: half a block
        return;
    const Place place = place_of_workgroup(units, pages_per_unit);
    if (!place.valid)
        return;
    const int      unit = place.unit, sub = place.part;
    const unsigned spmm_grid = units * split_k;
    const uint4* first = ws + static_cast<size_t>(sub) * spmm_grid * (cols * 16) + t;
    // the SpMM launch's workgroup of (unit, slice) is base_w + slice*step_w (the launch order above is linear in
    // the part); for a unit of the XCDs' own blocks its two coordinates are this workgroup's x and z
    const bool     own    = blockIdx.z < units / kXcds;
    const unsigned base_w = own ? blockIdx.z * split_k * kXcds + blockIdx.x : static_cast<unsigned>(unit) * split_k;
    const unsigned step_w = own ? kXcds : 1;
    float          s[8]   = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < split_k; k0 += 8) {
        uint4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (k0 + j < split_k)
                v[j] = first[static_cast<size_t>(base_w + (k0 + j) * step_w) * (cols * 16)];
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (k0 + j < split_k) {
                const half8 h = __builtin_bit_cast(half8, v[j]);
#pragma unroll
                for (int e = 0; e < 8; e++)
                    s[e] += static_cast<float>(h[e]);
            }
    }
    half4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        lo[e] = static_cast<_Float16>(RELU && !(s[e] > 0.f) ? 0.f : s[e]);
        hi[e] = static_cast<_Float16>(RELU && !(s[4 + e] > 0.f) ? 0.f : s[4 + e]);
    }
    // piece t = q*(4*cols) + g*cols + r16: rows 32q + 4g .. +3 and 16 further on, column r16 of the block
    // a unit's pages: rows_per_unit row tiles, one after the other, each with the unit's 16-column blocks in order
    const int lg = N < 16 ? 3 : 4;  // cols = 1 << lg
    const int q = t >> (lg + 2), g = (t >> lg) & 3, r16 = t & (cols - 1);
    const int blocks  = pages_per_unit / rows_per_unit;
    const int n       = ((unit % col_groups) * blocks + sub % blocks) * 16 + r16;
    const int rowtile = (unit / col_groups) * rows_per_unit + sub / blocks;
    _Float16* o = c + static_cast<size_t>(n) * M + static_cast<size_t>(rowtile) * kTileRows + q * 32 + g * 4;
    *reinterpret_cast<half4*>(o)      = lo;
    *reinterpret_cast<half4*>(o + 16) = hi;
}

// out[w] = id of the XCD that workgroup w of this launch ran on, w = x + 8*(y + 3*z) in a grid (8, 3, layers):
// the order in which the launches above count on their workgroups being handed out
__global__ __launch_bounds__(kLanes) void xcd_probe_kernel(unsigned* __restrict__ out, unsigned workgroups)
{
    const unsigned w = blockIdx.x + kXcds * (blockIdx.y + 3 * blockIdx.z);
    if (threadIdx.x == 0 && w < workgroups)
        out[w] = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11));  // XCC_ID, bits 3:0
}

__global__ __launch_bounds__(256) void relu_kernel(uint4* __restrict__ x, long n8)
{
    const long i = static_cast<long>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n8)
        return;
    half8 h = __builtin_bit_cast(half8, x[i]);
#pragma unroll
    for (int j = 0; j < 8; j++)
        h[j] = h[j] > static_cast<_Float16>(0) ? h[j] : static_cast<_Float16>(0);  // NaN -> 0 like max(x, 0)
    x[i] = __builtin_bit_cast(uint4, h);
}

__global__ __launch_bounds__(256) void take_rows_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, int rows8, int cols, int ld8)
{
    const long i = static_cast<long>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= static_cast<long>(rows8) * cols)
        return;
    const int j = static_cast<int>(i / rows8), r = static_cast<int>(i % rows8);
    dst[i] = src[static_cast<long>(j) * ld8 + r];
}

template<int NB, int DEPTH, int W, int G>
int launch_spmm(hipStream_t stream, const void* comp, const int* offs, const void* b, int ldb, void* out, int m, int n, int k, int split_k, int col_groups, int pages)
{
    const unsigned units = (static_cast<unsigned>(m / kTileRows) + W - 1) / W * col_groups;
    hipLaunchKernelGGL((spmm_stream_kernel<NB, DEPTH, W, G>),
                       grid_of(units, split_k),
                       dim3(kLanes * W),
                       0,
                       stream,
                       static_cast<const uint4*>(comp),
                       offs,
                       static_cast<const _Float16*>(b),
                       ldb,
                       static_cast<_Float16*>(out),
                       m,
                       n,
                       k,
                       split_k,
                       col_groups,
                       pages,
                       units);
    return static_cast<int>(hipGetLastError());
}

// Row tiles per workgroup of the launch for B of n columns, A of m rows and split_k slices: 8 (a CU's eight waves
// share each staged window of B) for n = 64 when the row tiles come in whole groups of eight (the slabs of whole
// workgroups then fill Split_K*M*N halfs exactly, and the callers' workspaces hold no more) and the launch's
// workgroups, each of which fills a CU, number between 192 and 256: one round on at least three quarters of the
// 256 CUs.  Otherwise 1: fewer, larger workgroups would leave CUs idle (7168 x 7168 at its best Split_K: 23.8 us
// with one row tile per workgroup, 29.6 us with eight), more would run in two rounds.
// Measured at 36864 x 9216, 80 %: n = 64 62-64 us against 73.6 with one row tile per workgroup; n = 32 52.4
// against 51.7 (the four fragment loads a tile costs there are no more than the meeting and the LDS reads that
// replace them), and workgroups of four row tiles meeting at every tile gain nothing at n = 64 (72.9 us).
// g_rows_override (a measuring and testing aid): 1 forces 1, 8 forces 8 wherever the row tiles allow it.
std::atomic<int> g_rows_override{0};

int rows_per_workgroup(int n, int m, int split_k)
{
    const int forced = g_rows_override.load(std::memory_order_relaxed);
    const int tiles  = m / kTileRows;
    if (n != 64 || forced == 1 || tiles % 8)
        return 1;
    if (forced == 8)
        return 8;
    const long workgroups = static_cast<long>(tiles / 8) * split_k;
    return workgroups >= 192 && workgroups <= 256 ? 8 : 1;
}

constexpr int      kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

}  // namespace

// Library-owned slab storage for callers that cannot provide (or allocate) a Reduction_Workspace: a fixed
// array in the code object's own device memory, one copy per GPU the library runs on, held until the
// process ends.  In host code the array's name is only a handle: the device address comes from
// hipGetSymbolAddress, once per device, and that pointer is what kernels receive.
static __device__ __align__(256) unsigned char scratch[FLASHLLM_STATIC_WORKSPACE_BYTES];

extern "C" int flashllm_hip_static_workspace(void** ptr)
{
    int        dev = -1;
    hipError_t e   = hipGetDevice(&dev);
    if (e != hipSuccess)
        return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices)
        return static_cast<int>(hipErrorInvalidDevice);
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {  // first call on this device (two threads racing here resolve the same address)
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess)
            return static_cast<int>(e);
        if (!p)
            return static_cast<int>(hipErrorInvalidSymbol);
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *ptr = p;
    return 0;
}

// pages != 0 (Split_K > 1 only): the slabs go to the workspace by workgroup, for flashllm_hip_launch_reduce_pages
extern "C" int flashllm_hip_launch_spmm(
    void* stream, const void* comp, const int* offs, const void* b, int ldb, void* out, int m, int n, int k, int split_k, int pages)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    pages         = pages && split_k > 1;
    if (n <= 16)
        return launch_spmm<1, 8, 1, 1>(s, comp, offs, b, ldb, out, m, n, k, split_k, 1, pages);
    if (n == 32)
        return launch_spmm<2, 8, 1, 1>(s, comp, offs, b, ldb, out, m, n, k, split_k, 1, pages);
    if (rows_per_workgroup(n, m, split_k) == 8)
        return launch_spmm<4, 8, 8, 2>(s, comp, offs, b, ldb, out, m, n, k, split_k, 1, pages);
    return launch_spmm<4, 6, 1, 1>(s, comp, offs, b, ldb, out, m, n, k, split_k, n / 64, pages);
}

extern "C" void flashllm_hip_set_rows_per_workgroup(int rows)
{
    g_rows_override.store(rows, std::memory_order_relaxed);
}

extern "C" int flashllm_hip_rows_per_workgroup(int n, int m, int split_k)
{
    return rows_per_workgroup(n, m, split_k);
}

extern "C" int flashllm_hip_launch_spmm_group(
    void* stream, const void* comp, const int* offs, const void* b, int ldb, void* out, int m, int n, int k, int split_k, int pages)
{
    // 128 columns per workgroup (four waves x 32); requires n % 128 == 0
    const unsigned units = static_cast<unsigned>(m / kTileRows) * (n / 128);
    hipLaunchKernelGGL(spmm_group_kernel<2>, grid_of(units, split_k), dim3(kGroupThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(comp), offs, static_cast<const _Float16*>(b), ldb, static_cast<_Float16*>(out),
                       m, n, k, split_k, n / 128, pages && split_k > 1, units);
    return static_cast<int>(hipGetLastError());
}

extern "C" int flashllm_hip_launch_reduce(void* stream, void* c, const void* ws, long mn, int split_k, int relu)
{
    const long     n4 = mn / 4;
    const dim3     grid(static_cast<unsigned>((n4 + 255) / 256));
    hipStream_t    s  = static_cast<hipStream_t>(stream);
    uint2*         cp = static_cast<uint2*>(c);
    const uint2*   wp = static_cast<const uint2*>(ws);
    if (relu)
        hipLaunchKernelGGL(splitk_reduce_kernel<true>, grid, dim3(256), 0, s, cp, wp, n4, split_k);
    else
        hipLaunchKernelGGL(splitk_reduce_kernel<false>, grid, dim3(256), 0, s, cp, wp, n4, split_k);
    return static_cast<int>(hipGetLastError());
}

extern "C" int flashllm_hip_launch_reduce_pages(void* stream, void* c, const void* ws, int m, int n, int split_k, int relu)
{
    // the units of the SpMM launch for this N: `rows` row tiles x 16*blocks columns (a wave's columns in
    // spmm_stream_kernel, a workgroup's 128 in spmm_group_kernel)
    const bool     group      = n % 128 == 0;
    const int      rows       = group ? 1 : rows_per_workgroup(n, m, split_k);
    const int      blocks     = group ? 8 : (n <= 16 ? 1 : (n == 32 ? 2 : 4));
    const int      col_groups = group ? n / 128 : (n <= 64 ? 1 : n / 64);
    const unsigned units      = (static_cast<unsigned>(m / kTileRows) + rows - 1) / rows * col_groups;
    const int      pages_per_unit = blocks * rows;
    const dim3     grid = grid_of(units, pages_per_unit);
    hipStream_t    s  = static_cast<hipStream_t>(stream);
    _Float16*      cp = static_cast<_Float16*>(c);
    const uint4*   wp = static_cast<const uint4*>(ws);
    if (relu)
        hipLaunchKernelGGL(splitk_reduce_pages_kernel<true>, grid, dim3(256), 0, s, cp, wp, m, n, split_k, pages_per_unit, rows, col_groups, units);
    else
        hipLaunchKernelGGL(splitk_reduce_pages_kernel<false>, grid, dim3(256), 0, s, cp, wp, m, n, split_k, pages_per_unit, rows, col_groups, units);
    return static_cast<int>(hipGetLastError());
}

extern "C" int flashllm_hip_launch_xcd_probe(void* stream, unsigned* out, int workgroups)
{
    if (workgroups <= 0)
        return static_cast<int>(hipErrorInvalidValue);
    const dim3 grid(kXcds, 3, (static_cast<unsigned>(workgroups) + 3 * kXcds - 1) / (3 * kXcds));
    hipLaunchKernelGGL(xcd_probe_kernel, grid, dim3(kLanes), 0, static_cast<hipStream_t>(stream), out, static_cast<unsigned>(workgroups));
    return static_cast<int>(hipGetLastError());
}

extern "C" int flashllm_hip_launch_relu(void* stream, void* x, long n)
{
    const long n8 = n / 8;
    hipLaunchKernelGGL(relu_kernel, dim3(static_cast<unsigned>((n8 + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<uint4*>(x), n8);
    return static_cast<int>(hipGetLastError());
}

extern "C" int flashllm_hip_launch_take_rows(void* stream, void* dst, const void* src, int rows, int cols, int src_ld)
{
    const long n8 = static_cast<long>(rows / 8) * cols;
    hipLaunchKernelGGL(take_rows_kernel, dim3(static_cast<unsigned>((n8 + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<uint4*>(dst), static_cast<const uint4*>(src),
                       rows / 8, cols, src_ld / 8);
    return static_cast<int>(hipGetLastError());
}
