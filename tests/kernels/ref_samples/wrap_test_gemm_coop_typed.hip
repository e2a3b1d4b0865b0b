// Other element types and operand orientations through the cooperative GEMM device kernel of the reference's test
// suite (the f16 col-major x row-major cases are in wrap_test_gemm_coop.hip), compiled unchanged against this
// library's headers: gemm_PGR1_LB2_MP0_MB_CP -- cooperative global reads, double-buffered LDS, BlocksX x
// BlocksY blocks per wave, driven by the CooperativeGemm::{Block,Wave,Workgroup}Level configurations
// (test/gemm/gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp:52-283, test/gemm/gemm_config.hpp:64-431,
// gemm_driver_impl.hpp, gemm_global_mapping.hpp, gemm_local_mapping.hpp, gemm_coop_schedule.hpp).
// Launch geometry and LDS size follow the suite (detail/kernel_impl.hpp:134-194).  The suite's build
// predicates (test/gemm/gemm_predicates_base.hpp:58-83) admit a kernel only when its ArchId template
// argument equals the compiler's current architecture id AND is one of gfx908..gfx942, so this translation
// unit is compiled with ROCWMMA_REPORT_ARCH_ID = 0x942 (see internal/constants.hpp).
#define ROCWMMA_REPORT_ARCH_ID 0x942
#include <iostream>

#include <hip/hip_runtime.h>

#include <rocwmma/rocwmma.hpp>
#include <rocwmma/rocwmma_coop.hpp>
#include <rocwmma/rocwmma_transforms.hpp>

#include "gemm/gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp"

namespace
{
    using namespace rocwmma;
    constexpr uint32_t WAVE = 64, ARCH = Constants::AMDGCN_ARCH_ID_GFX942;

    template <typename Config, typename LLds, uint32_t BM, uint32_t BN, uint32_t BK, typename InT, typename OutT,
              typename CompT, typename LA, typename LB, typename LC, uint32_t BX, uint32_t BY, uint32_t TBX = 128,
              uint32_t TBY = 2>
    int coop(uint32_t m, uint32_t n, uint32_t k, const void* a, const void* b, const void* c, void* d, uint32_t lda,
             uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta)
    {
        dim3           grid(ceilDiv(m, BM * BX * TBX / WAVE), ceilDiv(n, BN * BY * TBY));
        const uint32_t lds = 2u * sizeof(InT) * (TBX / WAVE * BX * BM + TBY * BY * BN) * BK;
        hipLaunchKernelGGL(
            (gemm_PGR1_LB2_MP0_MB_CP<BM, BN, BK, InT, OutT, CompT, LA, LB, LC, LC, LLds, Config, BX, BY, TBX, TBY, WAVE, ARCH>),
            grid, dim3(TBX, TBY), lds, 0, m, n, k, static_cast<const InT*>(a), static_cast<const InT*>(b),
            static_cast<const OutT*>(c), static_cast<OutT*>(d), lda, ldb, ldc, ldd, static_cast<CompT>(alpha),
            static_cast<CompT>(beta));
        return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
    }
} // namespace

#define GEMM_ARGS                                                                                                  \
    uint32_t m, uint32_t n, uint32_t k, const void *a, const void *b, const void *c, void *d, uint32_t lda, uint32_t ldb, \
        uint32_t ldc, uint32_t ldd, float alpha, float beta
#define GEMM_PASS m, n, k, a, b, c, d, lda, ldb, ldc, ldd, alpha, beta

// variant: 0 int8 -> int32, A row-major, B col-major, 32x32x32; 1 bf16 -> f32, A and B row-major, 16x16x16;
// 2 f32 -> f32, A and B col-major, 32x32x8; 3 f64 -> f64, A row-major, B col-major, 16x16x16; 4 e4m3 -> f32,
// A col-major, B row-major, 32x32x32.  2 x 2 blocks per wave, C / D row-major.
// cfg: 0 Workgroup LdsNT (LDS row-major), 1 Block LdsTN (LDS col-major), 2 Wave LdsNT (LDS col-major).
extern "C" int ref_test_gemm_coop_typed(int variant, int cfg, GEMM_ARGS)
{
    namespace CG = rocwmma::CooperativeGemm;
#define CFGS(BM, BK, IN, OUT, COMP, LA, LB)                                                                     \
    switch(cfg)                                                                                                 \
    {                                                                                                           \
    case 0: return coop<CG::WorkgroupLevel::LdsNT, row_major, BM, BM, BK, IN, OUT, COMP, LA, LB, row_major, 2, 2>(GEMM_PASS); \
    case 1: return coop<CG::BlockLevel::LdsTN, col_major, BM, BM, BK, IN, OUT, COMP, LA, LB, row_major, 2, 2>(GEMM_PASS);     \
    case 2: return coop<CG::WaveLevel::LdsNT, col_major, BM, BM, BK, IN, OUT, COMP, LA, LB, row_major, 2, 2>(GEMM_PASS);      \
    default: return -2;                                                                                         \
    }
    switch(variant)
    {
    case 0: CFGS(32, 32, int8_t, int32_t, int32_t, row_major, col_major)
    case 1: CFGS(16, 16, bfloat16_t, float32_t, float32_t, row_major, row_major)
    case 2: CFGS(32, 8, float32_t, float32_t, float32_t, col_major, col_major)
    case 3: CFGS(16, 16, float64_t, float64_t, float64_t, row_major, col_major)
    case 4: CFGS(32, 32, float8_t, float32_t, float32_t, col_major, row_major)
    default: return -2;
    }
#undef CFGS
}
