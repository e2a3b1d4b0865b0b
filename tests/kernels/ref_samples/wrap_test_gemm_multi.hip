// Runs the multi-block, non-cooperative GEMM device kernel of the reference's test suite, compiled unchanged against
// this library's headers: gemm_PGR0_LB0_MP0_MB_NC (BlocksX x BlocksY blocks per wave,
// test/gemm/gemm_PGR0_LB0_MP0_MB_NC/device/kernel_device_func.hpp:50-200), launch geometry from detail/kernel_impl.hpp
// of that suite (:123-129).  A translation unit of its own: the suites' device headers share their include guards.
// The suite's build predicates (test/gemm/gemm_predicates_base.hpp:58-83) admit a kernel only when its
// ArchId template argument equals the compiler's current architecture id AND is one of gfx908..gfx942, so
// this translation unit is compiled with ROCWMMA_REPORT_ARCH_ID = 0x942 (see internal/constants.hpp).
#define ROCWMMA_REPORT_ARCH_ID 0x942
#include <iostream>

#include <hip/hip_runtime.h>

#include <rocwmma/rocwmma.hpp>
#include <rocwmma/rocwmma_coop.hpp>
#include <rocwmma/rocwmma_transforms.hpp>

#include "gemm/gemm_PGR0_LB0_MP0_MB_NC/device/kernel_device_func.hpp"

namespace
{
    using namespace rocwmma;
    constexpr uint32_t WAVE = 64, ARCH = Constants::AMDGCN_ARCH_ID_GFX942;
    constexpr uint32_t TBX = 128, TBY = 2;

    template <uint32_t BM, uint32_t BN, uint32_t BK, typename InT, typename OutT, typename CompT, typename LA, typename LB,
              typename LC, uint32_t BX, uint32_t BY>
    int multi(uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b, const void* c, void* d, uint32_t lda,
              uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta)
    {
        dim3 grid(ceilDiv(m, BM * BX * TBX / WAVE), ceilDiv(n, BN * BY * TBY));
        hipLaunchKernelGGL(
            (gemm_PGR0_LB0_MP0_MB_NC<BM, BN, BK, InT, OutT, CompT, LA, LB, LC, LC, BX, BY, TBX, TBY, WAVE, ARCH>), grid,
            dim3(TBX, TBY), 0, 0, m, n, k, static_cast<const InT*>(a), static_cast<const InT*>(b),
            static_cast<const OutT*>(c), static_cast<OutT*>(d), lda, ldb, ldc, ldd, static_cast<CompT>(alpha),
            static_cast<CompT>(beta));
        return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
    }
} // namespace

#define GEMM_ARGS                                                                                                  \
    uint32_t m, uint32_t n, uint32_t k, const void *a, const void *b, const void *c, void *d, uint32_t lda, uint32_t ldb, \
        uint32_t ldc, uint32_t ldd, float alpha, float beta
#define GEMM_PASS m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta

// id 0: 32x32x16 f16 -> f32, 2 x 2 blocks per wave (A row-major, B col-major); id 1: 16x16x16 bf16 -> bf16, 4 x 2
// (A col-major, B row-major); id 2: 32x32x32 int8 -> int32, 2 x 4 (A row-major, B col-major); id 3: 16x16x16
// f16 -> f16, 8 x 8 (A and B row-major).  C / D row-major.
extern "C" int ref_test_gemm_multi(int id, GEMM_ARGS)
{
    switch(id)
    {
    case 0: return multi<32, 32, 16, float16_t, float32_t, float32_t, row_major, col_major, row_major, 2, 2>(GEMM_PASS);
    case 1: return multi<16, 16, 16, bfloat16_t, bfloat16_t, float32_t, col_major, row_major, row_major, 4, 2>(GEMM_PASS);
    case 2: return multi<32, 32, 32, int8_t, int32_t, int32_t, row_major, col_major, row_major, 2, 4>(GEMM_PASS);
    case 3: return multi<16, 16, 16, float16_t, float16_t, float32_t, row_major, row_major, row_major, 8, 8>(GEMM_PASS);
    default: return -2;
    }
}
