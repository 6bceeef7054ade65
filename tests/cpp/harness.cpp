// C++ caller of libSpMM_API.so in the order the reference's benchmark harness uses it
// (kernel_benchmark/spmm_test.cu:309-404): InitSparseMatrixA_bitmap through the overload with the reference's
// signature (half*, int& max_nnz), device copies of the five arrays, a workspace of M*N*Split_K halves, warm-up and
// timed calls of the 14-argument SpMM_SplitK_API_bitmap_v3 on the null stream.  The result is checked on the host
// against a float64 product of sampled rows; the north-star entry point is called on the same arrays as well.
//   usage: spmm_harness M K N sparsity_percent Split_K      -> prints one line, exit code 0 when both checks pass
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "spmm_api.h"

typedef __half half;

#define HIP_OK(call)                                                                                              \
    do {                                                                                                          \
        hipError_t e_ = (call);                                                                                   \
        if (e_ != hipSuccess) {                                                                                   \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);                            \
            return 2;                                                                                             \
        }                                                                                                         \
    } while (0)

static double check_rows(const std::vector<half>& Wh, const std::vector<half>& Xh, const std::vector<half>& Ch, int M,
                         int K, int N, double& max_ref)
{
    double max_err = 0;
    max_ref        = 0;
    for (int s = 0; s < 32; ++s) {
        const int m = (int)(((long long)s * 2654435761LL) % M);
        for (int n = 0; n < N; ++n) {
            double acc = 0;
            for (int k = 0; k < K; ++k)
                acc += (double)__half2float(Wh[(size_t)m * K + k]) * (double)__half2float(Xh[(size_t)n * K + k]);
            const double got = (double)__half2float(Ch[(size_t)n * M + m]);
            max_err = std::fmax(max_err, std::fabs(got - acc));
            max_ref = std::fmax(max_ref, std::fabs(acc));
        }
    }
    return max_err;
}

int main(int argc, char** argv)
{
    if (argc != 6) {
        std::printf("usage: %s M K N sparsity_percent Split_K\n", argv[0]);
        return 2;
    }
    const int M = std::atoi(argv[1]), K = std::atoi(argv[2]), N = std::atoi(argv[3]), sparsity = std::atoi(argv[4]);
    const int Split_K = std::atoi(argv[5]);

    std::srand(7);
    std::vector<half> A_h((size_t)M * K), B_h((size_t)N * K);
    for (auto& v : A_h)
        v = (std::rand() % 100 < sparsity) ? __float2half(0.f) : __float2half((float)(std::rand() % 5 - 2) * 0.5f + 0.25f);
    for (auto& v : B_h)
        v = __float2half((float)(std::rand() % 9 - 4) * 0.25f);

    half*     Compressed_Val   = nullptr;
    int *     TileOffsets = nullptr, *TileOffsets_median = nullptr, *TileOffsets_global = nullptr;
    uint64_t* bitmap      = nullptr;
    int       max_nnz     = 0;
    const int G = InitSparseMatrixA_bitmap(A_h.data(), M, K, 8, 16, 64, 8, 64, 64, &Compressed_Val, &TileOffsets,
                                           &TileOffsets_median, &TileOffsets_global, &bitmap, max_nnz);
    if (G != (M / 64) * (K / 64)) {
        std::printf("encoder returned %d group tiles\n", G);
        return 1;
    }
    if (max_nnz % 64 != 0)
        max_nnz = ((max_nnz / 64) + 1) * 64;
    const int    num_ltiles = G * 64, num_mtiles = G * 4;
    const size_t val_count  = (size_t)TileOffsets_global[G];

    half *    values_d, *B_d, *C_d, *ws_d;
    int *     global_d, *median_d, *max_nnz_d;
    uint64_t* bitmap_d;
    HIP_OK(hipMalloc(&values_d, sizeof(half) * (val_count ? val_count : 1)));
    HIP_OK(hipMalloc(&global_d, sizeof(int) * (G + 1)));
    HIP_OK(hipMalloc(&median_d, sizeof(int) * num_mtiles));
    HIP_OK(hipMalloc(&bitmap_d, sizeof(uint64_t) * num_ltiles));
    HIP_OK(hipMalloc(&max_nnz_d, sizeof(int)));
    HIP_OK(hipMalloc(&B_d, sizeof(half) * B_h.size()));
    HIP_OK(hipMalloc(&C_d, sizeof(half) * (size_t)M * N));
    HIP_OK(hipMalloc(&ws_d, sizeof(half) * (size_t)M * N * Split_K));
    HIP_OK(hipMemcpy(values_d, Compressed_Val, sizeof(half) * val_count, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(global_d, TileOffsets_global, sizeof(int) * (G + 1), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(median_d, TileOffsets_median, sizeof(int) * num_mtiles, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(bitmap_d, bitmap, sizeof(uint64_t) * num_ltiles, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(max_nnz_d, &max_nnz, sizeof(int), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(B_d, B_h.data(), sizeof(half) * B_h.size(), hipMemcpyHostToDevice));
    std::free(Compressed_Val), std::free(TileOffsets), std::free(TileOffsets_median), std::free(TileOffsets_global);
    std::free(bitmap);

    hipEvent_t start, stop;
    HIP_OK(hipEventCreate(&start));
    HIP_OK(hipEventCreate(&stop));
    const int warm_up = 5, iterations = 50;
    for (int i = 0; i < warm_up; ++i)
        if (SpMM_SplitK_API_bitmap_v3(0, nullptr, values_d, global_d, median_d, bitmap_d, max_nnz_d, B_d, C_d, M, N, K,
                                      ws_d, Split_K) != (int)hipSuccess)
            return 1;
    HIP_OK(hipEventRecord(start, 0));
    for (int i = 0; i < iterations; ++i)
        SpMM_SplitK_API_bitmap_v3(0, nullptr, values_d, global_d, median_d, bitmap_d, max_nnz_d, B_d, C_d, M, N, K, ws_d,
                                  Split_K);
    HIP_OK(hipEventRecord(stop, 0));
    HIP_OK(hipEventSynchronize(stop));
    float ms = 0;
    HIP_OK(hipEventElapsedTime(&ms, start, stop));
    ms /= iterations;
    const double tflops = 2.0 * M * N * K / (ms / 1000.0) / 1e12;

    std::vector<half> C_h((size_t)M * N);
    HIP_OK(hipMemcpy(C_h.data(), C_d, sizeof(half) * C_h.size(), hipMemcpyDeviceToHost));
    double       ref_v3, ref_ns;
    const double err_v3 = check_rows(A_h, B_h, C_h, M, K, N, ref_v3);

    // the shorter entry point on the same arrays, Split_K chosen by the library
    void* ws2 = nullptr;
    if (const size_t bytes = SpMM_WorkspaceBytes(M, N, K, 0))
        HIP_OK(hipMalloc(&ws2, bytes));
    HIP_OK(hipMemset(C_d, 0xff, sizeof(half) * C_h.size()));
    if (SpMM_SplitK_API(0, values_d, bitmap_d, global_d, B_d, C_d, M, N, K, ws2, 0) != (int)hipSuccess)
        return 1;
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(C_h.data(), C_d, sizeof(half) * C_h.size(), hipMemcpyDeviceToHost));
    const double err_ns = check_rows(A_h, B_h, C_h, M, K, N, ref_ns);

    const bool ok = err_v3 <= 1e-2 * ref_v3 && err_ns <= 1e-2 * ref_ns;
    std::printf("%s M %d K %d N %d sparsity %d%% Split_K %d: %d group tiles, NNZ %zu, max_nnz %d; v3 %.4f ms = %.2f TFLOP/s, "
                "max|d| %.3g of %.3g; SpMM_SplitK_API (Split_K %d) max|d| %.3g -> %s\n",
                SpMM_Version(), M, K, N, sparsity, Split_K, G, val_count, max_nnz, ms, tflops, err_v3, ref_v3,
                SpMM_SplitK_Auto(M, N, K), err_ns, ok ? "PASS" : "FAIL");
    return ok ? 0 : 1;
}
