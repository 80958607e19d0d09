// Host-side Tiled-CSL compression: dense row-major fp16 -> packed nonzeros
// (fp16 bits | 16-bit in-tile LDS position) + per-tile vector offsets.
//
// Produces the bytes of the reference's InitSparseMatrixA_API
// (csrc/SpMM_API.cu:163-360) and InitSparseMatrixA_API_NoReorder
// (csrc/SpMM_API.cu:363-489) by a different route:
//   * tiles are independent, so they are counted and encoded by a pool of
//     threads, with a prefix sum over the padded counts in between;
//   * the reference's "pop the fullest bank" (a 32-way scan per item,
//     csrc/SpMM_API.cu:145-156) becomes a bit-mask per fill level: the fullest
//     bank with the lowest index is ctz(mask[level]);
//   * its two-stage fill-then-LIFO write-out (csrc/SpMM_API.cu:306-346)
//     becomes one closed-form destination index per pop.
#include "flashllm_spmm.h"

#include <atomic>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

namespace {

constexpr int kTileRows = 128;
constexpr int kTileCols = 64;
constexpr int kBanks    = 32;
constexpr int kVec      = 4;
constexpr int kPerBank  = kTileRows * kTileCols / kBanks;  // 256 positions map to one bank
constexpr int kBankCap  = kPerBank + kVec;                 // + at most 3 padding items

std::atomic<int> g_threads{0};

// |x| > 0 in the reference's float compare: drops +0, -0 and NaN.
inline bool keeps(uint16_t h)
{
    const uint16_t mag = h & 0x7fffu;
    return mag != 0 && mag <= 0x7c00u;
}

inline int count_tile(const uint16_t* tile, size_t ld)
{
    int nnz = 0;
    for (int m = 0; m < kTileRows; m++) {
        const uint16_t* row = tile + m * ld;
        for (int n = 0; n < kTileCols; n++)
            nnz += keeps(row[n]);
    }
    return nnz;
}

// Encodes one tile with the bank reordering.  Returns false when a padding
// item is needed in a bank that has no zero position.
bool encode_tile_reorder(const uint16_t* tile, size_t ld, int pad, uint32_t* out)
{
    uint32_t bank[kBanks][kBankCap];
    int      fill[kBanks];
    int      first_zero[kBanks];
    for (int b = 0; b < kBanks; b++) {
        fill[b]       = 0;
        first_zero[b] = -1;
    }
    for (int m = 0; m < kTileRows; m++) {
        const uint16_t* row  = tile + m * ld;
        const int       flip = (m & 7) << 3;
        for (int n = 0; n < kTileCols; n++) {
            const int      sw  = n ^ flip;
            const int      b   = sw >> 1;
            const uint32_t pos = static_cast<uint32_t>(m * kTileCols + sw);
            const uint16_t v   = row[n];
            if (keeps(v))
                bank[b][fill[b]++] = v | (pos << 16);
            else if (first_zero[b] < 0)
                first_zero[b] = static_cast<int>(pos);
        }
    }
    for (int p = 0; p < pad; p++) {
        int b = 0;
        for (int i = 1; i < kBanks; i++)
            if (fill[i] < fill[b])
                b = i;
        if (first_zero[b] < 0)
            return false;
        bank[b][fill[b]++] = static_cast<uint32_t>(first_zero[b]) << 16;
    }
    int count = 0, top = 0;
    // level[s] = set of banks currently holding exactly s items
    uint32_t level[kBankCap + 1];
    std::memset(level, 0, sizeof(level));
    for (int b = 0; b < kBanks; b++) {
        level[fill[b]] |= 1u << b;
        count += fill[b];
        if (fill[b] > top)
            top = fill[b];
    }
    const int vectors = count / kVec;
    const int rep = vectors / kBanks, rem = vectors % kBanks;
    const int tail_items = rem * kVec;
    uint32_t* tail_out   = out + static_cast<size_t>(rep) * kVec * kBanks;
    for (int j = 0; j < count; j++) {
        const int      b    = __builtin_ctz(level[top]);
        const uint32_t item = bank[b][--fill[b]];
        level[top] &= ~(1u << b);
        level[top - 1] |= 1u << b;
        if (level[top] == 0)
            top--;
        if (j < tail_items) {
            // drained first, lane-major per pass; each lane is emitted back to front
            const int pass = j / rem, lane = j % rem;
            tail_out[lane * kVec + (kVec - 1 - pass)] = item;
        }
        else {
            const int q    = j - tail_items;
            const int pass = q / kBanks, lane = q % kBanks;  // pass = r*4 + v in fill order
            const int w    = rep * kVec - 1 - pass;          // its place in emission order
            out[(w / kVec) * (kVec * kBanks) + lane * kVec + (w % kVec)] = item;
        }
    }
    return true;
}

void encode_tile_scan(const uint16_t* tile, size_t ld, int pad, uint32_t* out)
{
    for (int m = 0; m < kTileRows; m++) {
        const uint16_t* row  = tile + m * ld;
        const int       flip = (m & 7) << 3;
        for (int n = 0; n < kTileCols; n++) {
            const uint16_t v = row[n];
            bool           k = keeps(v);
            if (!k && pad > 0) {
                pad--;
                k = true;
            }
            if (k)
                *out++ = v | (static_cast<uint32_t>(m * kTileCols + (n ^ flip)) << 16);
        }
    }
}

int worker_count(size_t tiles)
{
    int n = g_threads.load();
    if (n <= 0) {
        n = static_cast<int>(std::thread::hardware_concurrency());
        if (n > 16)
            n = 16;
    }
    if (n < 1)
        n = 1;
    if (static_cast<size_t>(n) > tiles)
        n = static_cast<int>(tiles);
    return n < 1 ? 1 : n;
}

template<typename F>
void for_each_tile(size_t tiles, F&& body)
{
    const int workers = worker_count(tiles);
    if (workers <= 1) {
        for (size_t t = 0; t < tiles; t++)
            body(t);
        return;
    }
    std::atomic<size_t>      next{0};
    std::vector<std::thread> pool;
    auto                     run = [&]() {
        constexpr size_t grab = 16;
        for (;;) {
            const size_t lo = next.fetch_add(grab);
            if (lo >= tiles)
                return;
            const size_t hi = lo + grab < tiles ? lo + grab : tiles;
            for (size_t t = lo; t < hi; t++)
                body(t);
        }
    };
    // a thread that cannot be created is simply left out: the others (at least this one) drain the tiles
    try {
        pool.reserve(workers);
        for (int w = 1; w < workers; w++)
            pool.emplace_back(run);
    }
    catch (...) {
    }
    run();
    for (auto& th : pool)
        th.join();
}

int compress(const uint16_t* A, int M, int K, uint32_t** comp_out, int** offs_out, bool reorder)
{
    if (!comp_out || !offs_out)
        return FLASHLLM_E_ARG;
    *comp_out = nullptr;
    *offs_out = nullptr;
    if (!A)
        return FLASHLLM_E_ARG;
    if (M <= 0 || K <= 0 || M % kTileRows || K % kTileCols)
        return FLASHLLM_E_SHAPE;
    const size_t tr = M / kTileRows, tc = K / kTileCols, tiles = tr * tc;
    const size_t ld = static_cast<size_t>(K);
    int*         offs = static_cast<int*>(std::malloc(sizeof(int) * (tiles + 2)));
    if (!offs)
        return FLASHLLM_E_NOMEM;
    // pass 1: nonzeros per tile (kept in offs[t+1] until the prefix sum)
    for_each_tile(tiles, [&](size_t t) {
        const uint16_t* tile = A + (t / tc) * kTileRows * ld + (t % tc) * kTileCols;
        offs[t + 1]          = count_tile(tile, ld);
    });
    uint8_t* pad = static_cast<uint8_t*>(std::malloc(tiles));
    if (!pad) {
        std::free(offs);
        return FLASHLLM_E_NOMEM;
    }
    long long running = 0;  // in items
    offs[0]           = 0;
    for (size_t t = 0; t < tiles; t++) {
        const int nnz = offs[t + 1];
        pad[t]        = static_cast<uint8_t>((kVec - nnz % kVec) % kVec);
        running += nnz + pad[t];
        offs[t + 1] = static_cast<int>(running / kVec);
    }
    offs[tiles + 1] = static_cast<int>(running / kVec);  // the trailing empty tile
    if (running / kVec > INT_MAX) {  // TileOffsets are int32 counts of 16-byte vectors (reference csrc/SpMM_API.cu:226,349)
        std::free(pad);
        std::free(offs);
        return FLASHLLM_E_SHAPE;
    }
    uint32_t* comp  = static_cast<uint32_t*>(std::malloc(sizeof(uint32_t) * static_cast<size_t>(running > 0 ? running : 1)));
    if (!comp) {
        std::free(pad);
        std::free(offs);
        return FLASHLLM_E_NOMEM;
    }
    // pass 2: encode every tile at its offset
    std::atomic<bool> ok{true};
    for_each_tile(tiles, [&](size_t t) {
        const uint16_t* tile = A + (t / tc) * kTileRows * ld + (t % tc) * kTileCols;
        uint32_t*       dst  = comp + static_cast<size_t>(offs[t]) * kVec;
        if (reorder) {
            if (!encode_tile_reorder(tile, ld, pad[t], dst))
                ok = false;
        }
        else {
            encode_tile_scan(tile, ld, pad[t], dst);
        }
    });
    std::free(pad);
    if (!ok) {
        std::free(comp);
        std::free(offs);
        return FLASHLLM_E_NOZERO;
    }
    *comp_out = comp;
    *offs_out = offs;
    return static_cast<int>(tiles + 2);
}

}  // namespace

extern "C" {

// No exception may cross the C boundary: what little can still throw in there (the thread pool's
// bookkeeping) is reported as an allocation failure.
int flashllm_init_sparse_matrix_a(const uint16_t* A_h, int M, int K, uint32_t** Compressed_A, int** TileOffsets)
{
    try {
        return compress(A_h, M, K, Compressed_A, TileOffsets, true);
    }
    catch (...) {
        return FLASHLLM_E_NOMEM;
    }
}

int flashllm_init_sparse_matrix_a_noreorder(
    const uint16_t* A_h, int M, int K, uint32_t** Compressed_A, int** TileOffsets)
{
    try {
        return compress(A_h, M, K, Compressed_A, TileOffsets, false);
    }
    catch (...) {
        return FLASHLLM_E_NOMEM;
    }
}

void flashllm_free(void* p)
{
    std::free(p);
}

void flashllm_set_compress_threads(int n)
{
    g_threads.store(n);
}

}  // extern "C"
