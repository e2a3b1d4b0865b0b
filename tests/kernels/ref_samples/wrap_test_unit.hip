// Runs device kernels of the reference's unit-test suite, compiled unchanged against this library's headers:
//   LoadStoreMatrixSync{A,B,Acc}      test/unit/load_store_matrix_sync_test/device/load_store_matrix_sync.hpp
//   LoadStoreMatrixCoopSync{A,B,Acc}  test/unit/load_store_matrix_coop_sync_test/device/load_store_matrix_coop_sync.hpp
//   fillFragment{A,B,Acc}             test/unit/fill_fragment_test/device/fill_fragment.hpp
//   loadContamination{A,B,Acc}, storeContamination{A,B,Acc}   test/unit/contamination_test/device/*.hpp
//   MapBlockToMatrix[OverrideM|N], MapMatrixToData[OverrideM|N], MapThreadToMatrix, MapWaveToMatrix
//                                     test/unit/map_util_test/device/*.hpp
// Every kernel has the suite's uniform signature (m, n, in, out, ld, param1, param2) and is launched on
// 128 x 2 threads (2 x 2 waves), one block of the matrix per wave, grid from the problem size
// (test/unit/unit_kernel_base_impl.hpp).  The kernels enable their bodies only for architecture ids
// gfx908..gfx942 (test/unit/unit_test_traits.hpp:68-117), so this translation unit is compiled with
// ROCWMMA_REPORT_ARCH_ID = 0x942 (see internal/constants.hpp).
#define ROCWMMA_REPORT_ARCH_ID 0x942
#include <iostream>

#include <hip/hip_runtime.h>

#include <rocwmma/rocwmma.hpp>
#include <rocwmma/rocwmma_coop.hpp>

#include "unit/contamination_test/device/load_contamination.hpp"
#include "unit/contamination_test/device/store_contamination.hpp"
#include "unit/fill_fragment_test/device/fill_fragment.hpp"
#include "unit/load_store_matrix_coop_sync_test/device/load_store_matrix_coop_sync.hpp"
#include "unit/load_store_matrix_sync_test/device/load_store_matrix_sync.hpp"
#include "unit/map_util_test/device/map_block_to_matrix.hpp"
#include "unit/map_util_test/device/map_block_to_matrix_override.hpp"
#include "unit/map_util_test/device/map_matrix_to_data.hpp"
#include "unit/map_util_test/device/map_matrix_to_data_override.hpp"
#include "unit/map_util_test/device/map_thread_to_matrix.hpp"
#include "unit/map_util_test/device/map_wave_to_matrix.hpp"

// (id, BlockM, BlockN, type, layout): block extents from test/unit/unit_test_params.hpp:89-139
#define UNIT_CASES(X)                        \
    X(0, 16, 16, float16_t, row_major)       \
    X(1, 16, 64, float16_t, col_major)       \
    X(2, 32, 8, float16_t, row_major)        \
    X(3, 32, 32, float16_t, col_major)       \
    X(4, 64, 16, float16_t, row_major)       \
    X(5, 128, 32, float16_t, col_major)      \
    X(6, 256, 16, float16_t, row_major)      \
    X(7, 16, 32, int8_t, row_major)          \
    X(8, 32, 64, int8_t, col_major)          \
    X(9, 64, 64, int8_t, row_major)          \
    X(10, 128, 128, int8_t, col_major)       \
    X(11, 16, 16, float32_t, col_major)      \
    X(12, 32, 16, float32_t, row_major)      \
    X(13, 64, 32, float32_t, col_major)      \
    X(14, 256, 8, float32_t, row_major)      \
    X(15, 16, 16, float64_t, row_major)      \
    X(16, 32, 32, float64_t, col_major)      \
    X(17, 64, 8, float64_t, row_major)       \
    X(18, 32, 32, bfloat16_t, row_major)     \
    X(19, 64, 128, bfloat16_t, col_major)    \
    X(20, 16, 16, int8_t, col_major)         \
    X(21, 32, 8, int8_t, row_major)

extern "C" int ref_unit_case_info(int id, uint32_t* blockM, uint32_t* blockN, uint32_t* elemBytes, uint32_t* rowMajor)
{
    using namespace rocwmma;
    switch(id)
    {
#define X(ID, BM, BN, T, L)                          \
    case ID:                                         \
        *blockM = BM, *blockN = BN;                  \
        *elemBytes = sizeof(T);                      \
        *rowMajor  = std::is_same_v<L, row_major>;   \
        return 0;
        UNIT_CASES(X)
#undef X
    default: return -1;
    }
}

// kind: 0..2 LoadStoreMatrixSync A/B/Acc, 3..5 LoadStoreMatrixCoopSync A/B/Acc, 6..8 fillFragment A/B/Acc,
// 9..11 loadContamination A/B/Acc, 12..14 storeContamination A/B/Acc, 15..17 MapBlockToMatrix / OverrideM / OverrideN,
// 18..20 MapMatrixToData / OverrideM / OverrideN, 21 MapThreadToMatrix, 22 MapWaveToMatrix
extern "C" int ref_unit_run(int kind, int id, uint32_t m, uint32_t n, const void* in, void* out, uint32_t ld, double p1,
                            double p2)
{
    using namespace rocwmma;
    constexpr uint32_t TBX = 128, TBY = 2, WAVE = 64;
    switch(id)
    {
#define LAUNCH(KERNEL, BM, BN, T, L)                                                                               \
    hipLaunchKernelGGL((KERNEL<BM, BN, T, L>), dim3(ceilDiv(m, BM * TBX / WAVE), ceilDiv(n, BN * TBY)), dim3(TBX, TBY), 0, \
                       0, m, n, static_cast<T const*>(in), static_cast<T*>(out), ld, static_cast<T>(p1), static_cast<T>(p2))
#define X(ID, BM, BN, T, L)                                               \
    case ID:                                                              \
        switch(kind)                                                      \
        {                                                                 \
        case 0: LAUNCH(LoadStoreMatrixSyncA, BM, BN, T, L); break;         \
        case 1: LAUNCH(LoadStoreMatrixSyncB, BM, BN, T, L); break;         \
        case 2: LAUNCH(LoadStoreMatrixSyncAcc, BM, BN, T, L); break;       \
        case 3: LAUNCH(LoadStoreMatrixCoopSyncA, BM, BN, T, L); break;     \
        case 4: LAUNCH(LoadStoreMatrixCoopSyncB, BM, BN, T, L); break;     \
        case 5: LAUNCH(LoadStoreMatrixCoopSyncAcc, BM, BN, T, L); break;   \
        case 6: LAUNCH(fillFragmentA, BM, BN, T, L); break;                \
        case 7: LAUNCH(fillFragmentB, BM, BN, T, L); break;                \
        case 8: LAUNCH(fillFragmentAcc, BM, BN, T, L); break;              \
        case 9: LAUNCH(loadContaminationA, BM, BN, T, L); break;           \
        case 10: LAUNCH(loadContaminationB, BM, BN, T, L); break;          \
        case 11: LAUNCH(loadContaminationAcc, BM, BN, T, L); break;        \
        case 12: LAUNCH(storeContaminationA, BM, BN, T, L); break;         \
        case 13: LAUNCH(storeContaminationB, BM, BN, T, L); break;         \
        case 14: LAUNCH(storeContaminationAcc, BM, BN, T, L); break;       \
        case 15: LAUNCH(MapBlockToMatrix, BM, BN, T, L); break;            \
        case 16: LAUNCH(MapBlockToMatrixOverrideM, BM, BN, T, L); break;   \
        case 17: LAUNCH(MapBlockToMatrixOverrideN, BM, BN, T, L); break;   \
        case 18: LAUNCH(MapMatrixToData, BM, BN, T, L); break;             \
        case 19: LAUNCH(MapMatrixToDataOverrideM, BM, BN, T, L); break;    \
        case 20: LAUNCH(MapMatrixToDataOverrideN, BM, BN, T, L); break;    \
        case 21: LAUNCH(MapThreadToMatrix, BM, BN, T, L); break;           \
        case 22: LAUNCH(MapWaveToMatrix, BM, BN, T, L); break;             \
        default: return -1;                                               \
        }                                                                 \
        break;
        UNIT_CASES(X)
#undef X
#undef LAUNCH
    default: return -1;
    }
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}
