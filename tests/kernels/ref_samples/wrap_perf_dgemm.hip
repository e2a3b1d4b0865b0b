// Runs the device kernel of the reference's samples/perf_dgemm.cpp (cooperative global -> LDS staging,
// transforms, 2 x 2 blocks per wave), compiled unchanged against this library's headers, with the
// sample's launch geometry (samples/perf_dgemm.cpp:729-765).
#define main sample_main_unused
#include "perf_dgemm.cpp"
#undef main

extern "C" int ref_perf_dgemm(uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b, const void* c, void* d,
                              uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, double alpha, double beta)
{
    auto blockDim = dim3(TBLOCK_X, TBLOCK_Y);
    auto gridDim  = dim3(rocwmma::ceilDiv(m, MACRO_TILE_X), rocwmma::ceilDiv(n, MACRO_TILE_Y));
    const int lds = 2u * sizeof(InputT) * (MACRO_TILE_X + MACRO_TILE_Y) * ROCWMMA_K;
    hipLaunchKernelGGL(gemm_rocwmma_d, gridDim, blockDim, lds, 0, m, n, k, static_cast<const InputT*>(a),
                       static_cast<const InputT*>(b), static_cast<const OutputT*>(c), static_cast<OutputT*>(d), lda, ldb,
                       ldc, ldd, static_cast<ComputeT>(alpha), static_cast<ComputeT>(beta));
    return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
}
