// Host-only driver for the sanitizer build (`make -C flash-llm_amd asan`): the Tiled-CSL compressors and the
// .bin exporter compiled with -fsanitize=address,undefined, run on a dense fp16 matrix read from a file.
//   asan_compress dense.bin M K out_prefix
// writes <prefix>.reorder.bin and <prefix>.noreorder.bin (int32 count of TileOffsets, the offsets, the items) for
// one and for three worker threads (which must agree), and the exporter's three files as <prefix>.NZWeights.bin,
// <prefix>.TileOffsets.bin, <prefix>.OutputSizes.bin.  Any sanitizer report ends the process with a non-zero code.
#include "flashllm_spmm.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace {
using compressor = int (*)(const uint16_t*, int, int, uint32_t**, int**);

bool run(compressor fn, const std::vector<uint16_t>& a, int m, int k, const std::string& out)
{
    std::vector<uint32_t> first_items;
    std::vector<int>      first_offsets;
    for (int threads : {1, 3}) {
        flashllm_set_compress_threads(threads);
        uint32_t* items   = nullptr;
        int*      offsets = nullptr;
        const int n       = fn(a.data(), m, k, &items, &offsets);
        if (n < 0) {
            std::fprintf(stderr, "compressor returned %d\n", n);
            return false;
        }
        const size_t nnz = 4u * static_cast<size_t>(offsets[n - 1]);
        if (threads == 1) {
            first_items.assign(items, items + nnz);
            first_offsets.assign(offsets, offsets + n);
        }
        else if (first_offsets.size() != static_cast<size_t>(n) || std::memcmp(first_offsets.data(), offsets, sizeof(int) * n)
                 || first_items.size() != nnz || (nnz && std::memcmp(first_items.data(), items, sizeof(uint32_t) * nnz))) {
            std::fprintf(stderr, "bytes depend on the number of threads\n");
            return false;
        }
        flashllm_free(items);
        flashllm_free(offsets);
    }
    std::FILE* f = std::fopen(out.c_str(), "wb");
    if (!f)
        return false;
    const int n = static_cast<int>(first_offsets.size());
    std::fwrite(&n, sizeof(int), 1, f);
    std::fwrite(first_offsets.data(), sizeof(int), first_offsets.size(), f);
    if (!first_items.empty())
        std::fwrite(first_items.data(), sizeof(uint32_t), first_items.size(), f);
    return std::fclose(f) == 0;
}
}  // namespace

int main(int argc, char** argv)
{
    if (argc != 5) {
        std::fprintf(stderr, "usage: %s dense.bin M K out_prefix\n", argv[0]);
        return 2;
    }
    const int         m = std::atoi(argv[2]), k = std::atoi(argv[3]);
    const std::string prefix = argv[4];
    // shapes the compressors must refuse without touching the matrix
    uint32_t* items   = nullptr;
    int*      offsets = nullptr;
    const uint16_t one = 0x3c00;
    if (flashllm_init_sparse_matrix_a(&one, 100, 64, &items, &offsets) != FLASHLLM_E_SHAPE || items || offsets)
        return 3;
    if (flashllm_init_sparse_matrix_a(nullptr, 128, 64, &items, &offsets) != FLASHLLM_E_ARG || items || offsets)
        return 3;
    if (m <= 0 || k <= 0)
        return 2;
    std::vector<uint16_t> a(static_cast<size_t>(m) * k);
    std::FILE*            in = std::fopen(argv[1], "rb");
    if (!in || std::fread(a.data(), sizeof(uint16_t), a.size(), in) != a.size())
        return 4;
    std::fclose(in);
    if (!run(flashllm_init_sparse_matrix_a, a, m, k, prefix + ".reorder.bin"))
        return 5;
    if (!run(flashllm_init_sparse_matrix_a_noreorder, a, m, k, prefix + ".noreorder.bin"))
        return 6;
    const int rc = flashllm_gen_sparse_matrix_bin_file(argv[1], m, k, (prefix + ".NZWeights.bin").c_str(),
                                                      (prefix + ".TileOffsets.bin").c_str(), (prefix + ".OutputSizes.bin").c_str());
    if (rc) {
        std::fprintf(stderr, "exporter returned %d\n", rc);
        return 7;
    }
    // a short file is an I/O error, not a read past the buffer
    if (flashllm_gen_sparse_matrix_bin_file(argv[1], m + 128, k, (prefix + ".x1").c_str(), (prefix + ".x2").c_str(),
                                            (prefix + ".x3").c_str()) != FLASHLLM_E_IO)
        return 8;
    std::printf("ok %dx%d\n", m, k);
    return 0;
}
