// Runs the cooperative GEMM device kernel of the reference's test suite, compiled unchanged against this
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

// f16 -> f16 (f32 compute), A col-major, B row-major, C / D row-major, 32x32x16 blocks, 2 x 2 blocks per wave.
// id: 0 Workgroup LdsNT, 1 Block LdsNT, 2 Block LdsTN, 3 Wave LdsNT, 4 Wave LdsTN (128 x 2 threads),
// 5 Block LdsRF (64 x 1 threads, BlockK 32);
// lds_col_major selects the LDS data layout.
extern "C" int ref_test_gemm_coop(int id, int lds_col_major, GEMM_ARGS)
{
    namespace CG = rocwmma::CooperativeGemm;
#define COOP(CFG)                                                                                                      \
    (lds_col_major ? coop<CFG, col_major, 32, 32, 16, float16_t, float16_t, float32_t, col_major, row_major, row_major, 2, \
                          2>(GEMM_PASS)                                                                                \
                   : coop<CFG, row_major, 32, 32, 16, float16_t, float16_t, float32_t, col_major, row_major, row_major, 2, \
                          2>(GEMM_PASS))
    switch(id)
    {
    case 0: return COOP(CG::WorkgroupLevel::LdsNT);
    case 1: return COOP(CG::BlockLevel::LdsNT);
    case 2: return COOP(CG::BlockLevel::LdsTN);
    case 3: return COOP(CG::WaveLevel::LdsNT);
    case 4: return COOP(CG::WaveLevel::LdsTN);
    case 5:
        // the suite admits the register-file LDS image for single-wave workgroups only, with more than 8
        // elements per lane and fragment (kernel_predicates.hpp:81-103): 64 x 1 threads, BlockK = 32
        return lds_col_major ? coop<CG::BlockLevel::LdsRF, col_major, 32, 32, 32, float16_t, float16_t, float32_t, col_major,
                                    row_major, row_major, 2, 2, 64, 1>(GEMM_PASS)
                             : coop<CG::BlockLevel::LdsRF, row_major, 32, 32, 32, float16_t, float16_t, float32_t, col_major,
                                    row_major, row_major, 2, 2, 64, 1>(GEMM_PASS);
    default: return -2;
    }
#undef COOP
}
