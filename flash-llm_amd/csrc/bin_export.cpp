// Offline weight files: dense fp16 .bin in, the three Tiled-CSL files out
// (reference csrc/SpMM_API.cu:500-555; consumers
// end2end_inference/ft_tools/huggingface_opt_convert_Phase2.py:36-59 and the
// loaders in third_party/ft.patch:3744-3794).
//   <name>.NZWeights.bin    uint32 x NNZ(padded)
//   <name>.TileOffsets.bin  int32  x NumOffsets
//   <name>.OutputSizes.bin  int32 NNZ(padded), int32 NumOffsets
#include "flashllm_spmm.h"

#include <climits>
#include <cstdio>
#include <cstdlib>
#include <vector>

namespace {
bool write_all(const char* name, const void* data, size_t bytes)
{
    std::FILE* f = std::fopen(name, "wb");
    if (!f)
        return false;
    const bool ok = bytes == 0 || std::fwrite(data, 1, bytes, f) == bytes;
    return std::fclose(f) == 0 && ok;
}
}  // namespace

extern "C" int flashllm_gen_sparse_matrix_bin_file(const char* dense_name,
                                                   int         M,
                                                   int         K,
                                                   const char* nz_name,
                                                   const char* offsets_name,
                                                   const char* sizes_name)
{
    if (!dense_name || !nz_name || !offsets_name || !sizes_name)
        return FLASHLLM_E_ARG;
    if (M <= 0 || K <= 0 || M % 128 || K % 64)
        return FLASHLLM_E_SHAPE;
    const size_t          count = static_cast<size_t>(M) * K;
    std::vector<uint16_t> dense;
    try {
        dense.resize(count);
    }
    catch (...) {
        return FLASHLLM_E_NOMEM;
    }
    std::FILE* in = std::fopen(dense_name, "rb");
    if (!in)
        return FLASHLLM_E_IO;
    const size_t got = std::fread(dense.data(), sizeof(uint16_t), count, in);
    std::fclose(in);
    if (got != count)
        return FLASHLLM_E_IO;
    uint32_t* nz      = nullptr;
    int*      offsets = nullptr;
    const int n_off   = flashllm_init_sparse_matrix_a(dense.data(), M, K, &nz, &offsets);
    if (n_off < 0)
        return n_off;
    // .OutputSizes.bin holds NNZ as an int32 (reference csrc/SpMM_API.cu:533,551): a weight whose padded
    // item count does not fit cannot be described by the format
    const long long nnz = 4LL * offsets[n_off - 1];
    if (nnz > INT_MAX) {
        flashllm_free(nz);
        flashllm_free(offsets);
        return FLASHLLM_E_SHAPE;
    }
    const int  sizes[2] = {static_cast<int>(nnz), n_off};
    const bool ok = write_all(sizes_name, sizes, sizeof(sizes)) && write_all(nz_name, nz, sizeof(uint32_t) * static_cast<size_t>(nnz))
                    && write_all(offsets_name, offsets, sizeof(int) * static_cast<size_t>(n_off));
    flashllm_free(nz);
    flashllm_free(offsets);
    return ok ? 0 : FLASHLLM_E_IO;
}

extern "C" void GenSparseMatrixBinFile(char* dense_name, int M, int K, char* nz_name, char* offsets_name, char* sizes_name)
{
    const int rc = flashllm_gen_sparse_matrix_bin_file(dense_name, M, K, nz_name, offsets_name, sizes_name);
    if (rc != 0) {
        std::printf("GenSparseMatrixBinFile() ERROR %d: %s -> %s, %s, %s\n", rc, dense_name, nz_name, offsets_name, sizes_name);
        std::exit(-1);
    }
}
