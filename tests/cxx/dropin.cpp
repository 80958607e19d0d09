// A caller written against the C++ header, the way kernel_benchmark/spmm_test.cu uses the
// reference's SpMM_API.cuh (spmm_test.cu:251-306): compress on the host, upload, multiply, download.
//
//   dropin compress M K sparsity% out.bin          host only: writes NumOffsets, TileOffsets, Compressed_A
//   dropin spmm     M K N sparsity% Split_K        needs a GPU: prints the max relative error against
//                                                  an fp32 product computed on the host
#include "SpMM_API.h"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

static void fill(std::vector<half>& a, std::vector<half>& b, int M, int K, int N, int pct)
{
    unsigned long long s = 0x9E3779B97F4A7C15ull;
    auto rnd = [&]() { s ^= s << 13; s ^= s >> 7; s ^= s << 17; return s; };
    for (size_t i = 0; i < a.size(); i++) {
        const unsigned long long r = rnd();
        a[i] = (r % 100 >= (unsigned)pct) ? __float2half(((r >> 20) % 2001) / 1000.0f - 1.0f) : __float2half(0.0f);
    }
    for (size_t i = 0; i < b.size(); i++)
        b[i] = __float2half((rnd() % 2001) / 1000.0f - 1.0f);
    (void)M; (void)K; (void)N;
}

int main(int argc, char** argv)
{
    if (argc < 5)
        return 2;
    const bool spmm = !strcmp(argv[1], "spmm");
    const int  M = atoi(argv[2]), K = atoi(argv[3]);
    const int  N = spmm ? atoi(argv[4]) : 8, pct = atoi(argv[spmm ? 5 : 4]);
    std::vector<half> A_h((size_t)M * K), B_h((size_t)K * N);
    fill(A_h, B_h, M, K, N, pct);

    uint32_t* NZWeights_CPU   = nullptr;
    int*      TileOffsets_CPU = nullptr;
    const int NumOffsets = InitSparseMatrixA_API(A_h.data(), M, N, K, &NZWeights_CPU, &TileOffsets_CPU);
    if (NumOffsets < 0)
        return 3;
    int NNZ = TileOffsets_CPU[NumOffsets - 1] * 4;

    if (!spmm) {
        FILE* f = fopen(argv[5], "wb");
        fwrite(&NumOffsets, 4, 1, f);
        fwrite(TileOffsets_CPU, 4, NumOffsets, f);
        fwrite(NZWeights_CPU, 4, NNZ, f);
        fwrite(A_h.data(), 2, A_h.size(), f);
        fclose(f);
        free(TileOffsets_CPU);
        free(NZWeights_CPU);
        return 0;
    }

    const int Split_K = atoi(argv[6]);
    uint32_t* NZWeights_GPU; int* TileOffsets_GPU; half *B, *C, *Reduction_Workspace;
    hipMalloc(&TileOffsets_GPU, sizeof(int) * NumOffsets);
    hipMalloc(&NZWeights_GPU, sizeof(uint32_t) * (NNZ ? NNZ : 1));
    hipMalloc(&B, sizeof(half) * K * N);
    hipMalloc(&C, sizeof(half) * M * N);
    hipMalloc(&Reduction_Workspace, sizeof(half) * M * N * Split_K);
    hipMemcpy(NZWeights_GPU, NZWeights_CPU, sizeof(uint32_t) * NNZ, hipMemcpyHostToDevice);
    hipMemcpy(TileOffsets_GPU, TileOffsets_CPU, sizeof(int) * NumOffsets, hipMemcpyHostToDevice);
    hipMemcpy(B, B_h.data(), sizeof(half) * K * N, hipMemcpyHostToDevice);
    free(TileOffsets_CPU);
    free(NZWeights_CPU);
    hipStream_t stream;
    hipStreamCreate(&stream);
    const hipError_t e = SpMM_SplitK_API(stream, nullptr, reinterpret_cast<const uint4*>(NZWeights_GPU), TileOffsets_GPU,
                                         B, C, M, N, K, Reduction_Workspace, Split_K);
    if (e != hipSuccess) {
        printf("SpMM_SplitK_API: %s\n", hipGetErrorString(e));
        return 4;
    }
    hipStreamSynchronize(stream);
    std::vector<half> C_h((size_t)M * N);
    hipMemcpy(C_h.data(), C, sizeof(half) * M * N, hipMemcpyDeviceToHost);
    double worst = 0, scale = 0;
    for (int n = 0; n < N; n++)
        for (int m = 0; m < M; m += 7) {
            float acc = 0;
            for (int k = 0; k < K; k++)
                acc += __half2float(A_h[(size_t)m * K + k]) * __half2float(B_h[(size_t)n * K + k]);
            const double d = fabs((double)__half2float(C_h[(size_t)n * M + m]) - acc);
            if (d > worst) worst = d;
            if (fabs(acc) > scale) scale = fabs(acc);
        }
    printf("max_rel_err %.6e\n", worst / scale);
    return worst / scale <= 1e-2 ? 0 : 5;
}
