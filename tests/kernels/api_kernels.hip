// Device-side checks of the fragment API, one small kernel per invariant, in the spirit of
// the reference's unit suites (test/unit/load_store_matrix_sync_test, fill_fragment_test,
// load_store_matrix_coop_sync_test, contamination_test) but without gtest: the host test
// (tests/test_fragment_api.py) drives them through this C ABI and compares on the host.
#include <rocwmma/rocwmma.hpp>
#include <rocwmma/rocwmma_coop.hpp>
#include <rocwmma/rocwmma_sparse.hpp>
#include <rocwmma/rocwmma_transforms.hpp>

using namespace rocwmma;

namespace
{
    template <typename FragT>
    __global__ void roundTrip(const GetDataType_t<FragT>* in, GetDataType_t<FragT>* out, uint32_t ldIn, uint32_t ldOut)
    {
        FragT frag;
        load_matrix_sync(frag, in, ldIn);
        store_matrix_sync(out, frag, ldOut);
    }

    template <typename FragT>
    __global__ void roundTripRuntime(const GetDataType_t<FragT>* in, GetDataType_t<FragT>* out, uint32_t ld, layout_t layout)
    {
        FragT frag; // DataLayoutT = void
        load_matrix_sync(frag, in, ld, layout);
        store_matrix_sync(out, frag, ld, layout);
    }

    template <typename FragT>
    __global__ void fillStore(GetDataType_t<FragT>* out, uint32_t ld, GetDataType_t<FragT> value)
    {
        FragT frag;
        fill_fragment(frag, value);
        store_matrix_sync(out, frag, ld);
    }

    // all waves of the workgroup share one fragment: global -> (coop) registers -> (coop) LDS -> global
    template <typename FragT>
    __global__ void coopRoundTrip(const GetDataType_t<FragT>* in, GetDataType_t<FragT>* out, uint32_t ld, uint32_t useLds)
    {
        using DataT = GetDataType_t<FragT>;
        using Shape = GetIOShape_t<FragT>;
        using Map   = GetDataLayout_t<FragT>;
        HIP_DYNAMIC_SHARED(void*, ldsRaw);
        DataT* lds = reinterpret_cast<DataT*>(ldsRaw);
        FragT  frag;
        load_matrix_coop_sync(frag, in, ld);
        if(useLds)
        {
            const uint32_t ldsLd = Map::leadingDim(make_coord2d((uint32_t)Shape::BlockHeight, (uint32_t)Shape::BlockWidth));
            store_matrix_coop_sync(lds, frag, ldsLd);
            synchronize_workgroup();
            // every wave re-reads its share from LDS with the same split and writes it out
            FragT again;
            load_matrix_coop_sync(again, lds, ldsLd);
            store_matrix_coop_sync(out, again, ld);
        }
        else
            store_matrix_coop_sync(out, frag, ld);
    }

    template <uint32_t WaveCount, typename FragT>
    __global__ void coopRoundTripStatic(const GetDataType_t<FragT>* in, GetDataType_t<FragT>* out, uint32_t ld)
    {
        FragT          frag;
        const uint32_t waveIndex = threadIdx.x / 64u + threadIdx.y * (blockDim.x / 64u);
        load_matrix_coop_sync<WaveCount>(frag, in, ld, waveIndex);
        store_matrix_coop_sync<WaveCount>(out, frag, ld, waveIndex);
    }

    // transpose relabel: a matrix_b fragment loaded row-major, viewed as the transposed matrix_a
    // fragment (col-major), stores the same memory image
    template <typename FragB>
    __global__ void transposeStore(const GetDataType_t<FragB>* in, GetDataType_t<FragB>* out, uint32_t ld)
    {
        FragB frag;
        load_matrix_sync(frag, in, ld);
        store_matrix_sync(out, applyTranspose(frag), ld);
    }

    // data-layout relabel: load with one orientation, store with the other = memory transpose
    template <typename FragT, typename OtherLayout>
    __global__ void relayoutStore(const GetDataType_t<FragT>* in, GetDataType_t<FragT>* out, uint32_t ldIn, uint32_t ldOut)
    {
        FragT frag;
        load_matrix_sync(frag, in, ldIn);
        store_matrix_sync(out, applyDataLayout<OtherLayout>(frag), ldOut);
    }

    template <uint32_t Blk, uint32_t BK, typename InT, typename AccT, typename LA, typename LB>
    __global__ void mmaTile(const InT* a, const InT* b, const AccT* c, AccT* d, uint32_t lda, uint32_t ldb, uint32_t ldc,
                            layout_t layoutC)
    {
        fragment<matrix_a, Blk, Blk, BK, InT, LA> fa;
        fragment<matrix_b, Blk, Blk, BK, InT, LB> fb;
        fragment<accumulator, Blk, Blk, BK, AccT> fc;
        load_matrix_sync(fa, a, lda);
        load_matrix_sync(fb, b, ldb);
        load_matrix_sync(fc, c, ldc, layoutC);
        mma_sync(fc, fa, fb, fc);
        store_matrix_sync(d, fc, ldc, layoutC);
    }

    // one tile D = A B + C with A 2:4 sparse in the K-blocked storage of a Blk-row matrix (rocwmma_sparse.hpp)
    template <uint32_t Blk, uint32_t BK, typename InT, typename AccT, typename LB>
    __global__ void sparseMmaTile(const InT* aVals, const uint8_t* aMeta, const InT* b, const AccT* c, AccT* d, uint32_t ldb,
                                  uint32_t ldc, layout_t layoutC)
    {
        using S = Sparse24<InT>;
        fragment<sparse_matrix_a, Blk, Blk, BK, InT, row_major> fa;
        fragment<sparse_metadata, Blk, Blk, BK, InT>            fm;
        fragment<matrix_b, Blk, Blk, BK, InT, LB>               fb;
        fragment<accumulator, Blk, Blk, BK, AccT>               fc;
        load_matrix_sync(fa, aVals + S::valueOffset(0u, 0u, Blk), S::valueStageStride(Blk));
        load_matrix_sync(fm, aMeta + S::metaOffset(0u, 0u, Blk), S::metaStageStride(Blk));
        load_matrix_sync(fb, b, ldb);
        load_matrix_sync(fc, c, ldc, layoutC);
        mma_sync(fc, fa, fm, fb, fc);
        store_matrix_sync(d, fc, ldc, layoutC);
    }

    // MappingUtil: every wave writes its (block row, block col, matrix row, matrix col) and data offset
    __global__ void mappingProbe(uint32_t* out, uint32_t ld)
    {
        using Mapping = MappingUtil<32, 16, float, row_major>;
        if(Mapping::laneId() != 0)
            return;
        auto           wave = Mapping::waveCoord();
        auto           blk  = Mapping::blockCoord();
        auto           mat  = Mapping::matrixCoord();
        auto           dim  = Mapping::workgroupDim();
        const uint32_t w    = (blockIdx.y * gridDim.x + blockIdx.x) * get<0>(dim) * get<1>(dim)
                           + get<0>(wave) * get<1>(dim) + get<1>(wave);
        uint32_t* o = out + w * 8u;
        o[0] = get<0>(wave), o[1] = get<1>(wave), o[2] = get<0>(blk), o[3] = get<1>(blk);
        o[4] = get<0>(mat), o[5] = get<1>(mat), o[6] = Mapping::dataOffset(mat, ld);
        o[7] = static_cast<uint32_t>(Mapping::dataCoord(static_cast<float*>(nullptr), ld) - static_cast<float*>(nullptr));
    }
} // namespace

// ---- dispatch tables.  A case id selects (role, BlockM, BlockN, BlockK, type, layout).
// Cases 26..89 sample the reference's unit-test matrix (test/unit/unit_test_params.hpp:86-146:
// block extents 16..256 x 8..256, 8/16/32-bit types, both layouts) within 64 registers per lane.
#define FRAG_CASES(X)                                                                  \
    X(0, matrix_a, 16, 16, 16, float16_t, row_major)                                   \
    X(1, matrix_a, 16, 16, 16, float16_t, col_major)                                   \
    X(2, matrix_b, 16, 16, 16, float16_t, row_major)                                   \
    X(3, matrix_b, 16, 16, 16, float16_t, col_major)                                   \
    X(4, matrix_a, 32, 32, 16, float16_t, row_major)                                   \
    X(5, matrix_a, 32, 32, 16, float16_t, col_major)                                   \
    X(6, matrix_b, 32, 32, 16, bfloat16_t, row_major)                                  \
    X(7, matrix_b, 32, 32, 16, bfloat16_t, col_major)                                  \
    X(8, accumulator, 16, 16, 16, float32_t, row_major)                                \
    X(9, accumulator, 16, 16, 16, float32_t, col_major)                                \
    X(10, accumulator, 32, 32, 16, float32_t, row_major)                               \
    X(11, accumulator, 32, 32, 16, float32_t, col_major)                               \
    X(12, accumulator, 32, 32, 8, float16_t, row_major)                                \
    X(13, matrix_a, 16, 16, 64, int8_t, row_major)                                     \
    X(14, matrix_b, 32, 32, 32, int8_t, col_major)                                     \
    X(15, matrix_a, 32, 32, 16, float8_t, row_major)                                   \
    X(16, matrix_b, 16, 16, 32, float8_t, row_major)                                   \
    X(17, matrix_a, 128, 32, 16, float16_t, col_major)                                 \
    X(18, matrix_b, 32, 128, 16, float16_t, row_major)                                 \
    X(19, matrix_a, 64, 16, 32, float16_t, row_major)                                  \
    X(20, matrix_b, 16, 256, 8, float32_t, row_major)                                  \
    X(21, matrix_a, 256, 16, 64, int8_t, row_major)                                    \
    X(22, accumulator, 32, 32, 16, int32_t, row_major)                                 \
    X(23, matrix_a, 32, 32, 32, float16_t, row_major)                                  \
    X(24, matrix_b, 16, 16, 4, float32_t, col_major)                                   \
    X(25, accumulator, 64, 64, 16, float32_t, col_major)                               \
    X(26, matrix_a, 16, 16, 128, bfloat16_t, row_major)                                \
    X(27, matrix_b, 16, 32, 16, bfloat16_t, row_major)                                 \
    X(28, matrix_a, 32, 16, 32, bfloat16_t, col_major)                                 \
    X(29, matrix_b, 16, 32, 64, bfloat16_t, col_major)                                 \
    X(30, matrix_a, 32, 16, 256, bfloat16_t, row_major)                                \
    X(31, matrix_b, 16, 64, 8, bfloat16_t, row_major)                                  \
    X(32, matrix_a, 64, 16, 64, bfloat16_t, col_major)                                 \
    X(33, matrix_b, 16, 128, 8, bfloat16_t, col_major)                                 \
    X(34, matrix_a, 128, 16, 16, bfloat16_t, row_major)                                \
    X(35, matrix_b, 16, 256, 16, bfloat16_t, row_major)                                \
    X(36, matrix_a, 16, 16, 16, float16_t, col_major)                                  \
    X(37, matrix_b, 16, 16, 256, float16_t, col_major)                                 \
    X(38, matrix_a, 32, 16, 8, float16_t, row_major)                                   \
    X(39, matrix_b, 16, 32, 16, float16_t, row_major)                                  \
    X(40, matrix_a, 32, 16, 128, float16_t, col_major)                                 \
    X(41, matrix_b, 16, 32, 256, float16_t, col_major)                                 \
    X(42, matrix_a, 64, 16, 16, float16_t, row_major)                                  \
    X(43, matrix_b, 16, 64, 128, float16_t, row_major)                                 \
    X(44, matrix_a, 128, 16, 16, float16_t, col_major)                                 \
    X(45, matrix_b, 16, 128, 32, float16_t, col_major)                                 \
    X(46, matrix_a, 128, 16, 64, float16_t, row_major)                                 \
    X(47, matrix_b, 16, 256, 8, float16_t, row_major)                                  \
    X(48, matrix_a, 256, 16, 32, float16_t, col_major)                                 \
    X(49, matrix_b, 16, 16, 32, float32_t, col_major)                                  \
    X(50, matrix_a, 32, 16, 32, float32_t, row_major)                                  \
    X(51, matrix_b, 16, 64, 8, float32_t, row_major)                                   \
    X(52, matrix_a, 64, 16, 64, float32_t, col_major)                                  \
    X(53, matrix_b, 16, 16, 32, float8_t, col_major)                                   \
    X(54, matrix_a, 16, 16, 128, float8_t, row_major)                                  \
    X(55, matrix_b, 16, 32, 32, float8_t, row_major)                                   \
    X(56, matrix_a, 32, 16, 64, float8_t, col_major)                                   \
    X(57, matrix_b, 16, 32, 256, float8_t, col_major)                                  \
    X(58, matrix_a, 64, 16, 64, float8_t, row_major)                                   \
    X(59, matrix_b, 16, 64, 128, float8_t, row_major)                                  \
    X(60, matrix_a, 128, 16, 16, float8_t, col_major)                                  \
    X(61, matrix_b, 16, 128, 64, float8_t, col_major)                                  \
    X(62, matrix_a, 256, 16, 8, float8_t, row_major)                                   \
    X(63, matrix_b, 16, 256, 32, float8_t, row_major)                                  \
    X(64, matrix_a, 256, 16, 64, float8_t, col_major)                                  \
    X(65, matrix_b, 16, 16, 128, int8_t, col_major)                                    \
    X(66, matrix_a, 32, 16, 32, int8_t, row_major)                                     \
    X(67, matrix_b, 16, 32, 128, int8_t, row_major)                                    \
    X(68, matrix_a, 32, 16, 256, int8_t, col_major)                                    \
    X(69, matrix_b, 16, 64, 32, int8_t, col_major)                                     \
    X(70, matrix_a, 64, 16, 64, int8_t, row_major)                                     \
    X(71, matrix_b, 16, 128, 8, int8_t, row_major)                                     \
    X(72, matrix_a, 128, 16, 64, int8_t, col_major)                                    \
    X(73, matrix_b, 16, 256, 32, int8_t, col_major)                                    \
    X(74, accumulator, 16, 64, 16, float32_t, row_major)                               \
    X(75, accumulator, 16, 64, 16, float32_t, col_major)                               \
    X(76, accumulator, 64, 16, 16, float32_t, row_major)                               \
    X(77, accumulator, 64, 16, 16, float32_t, col_major)                               \
    X(78, accumulator, 128, 32, 16, float32_t, row_major)                              \
    X(79, accumulator, 128, 32, 16, float32_t, col_major)                              \
    X(80, accumulator, 32, 128, 16, int32_t, row_major)                                \
    X(81, accumulator, 32, 128, 16, int32_t, col_major)                                \
    X(82, accumulator, 64, 64, 16, float16_t, row_major)                               \
    X(83, accumulator, 64, 64, 16, float16_t, col_major)                               \
    X(84, accumulator, 256, 16, 16, float32_t, row_major)                              \
    X(85, accumulator, 256, 16, 16, float32_t, col_major)                              \
    X(86, accumulator, 16, 16, 16, int32_t, row_major)                                 \
    X(87, accumulator, 16, 16, 16, int32_t, col_major)                                 \
    X(88, accumulator, 16, 256, 16, float16_t, row_major)                              \
    X(89, accumulator, 16, 256, 16, float16_t, col_major)                              \
    X(90, matrix_a, 16, 16, 16, float64_t, row_major)                                  \
    X(91, matrix_b, 16, 16, 16, float64_t, row_major)                                  \
    X(92, accumulator, 16, 16, 16, float64_t, col_major)                               \
    X(93, matrix_a, 64, 16, 8, float64_t, col_major)

// Coord2d arithmetic is element-wise and usable in constant expressions (the reference's two-element vector)
namespace
{
    constexpr rocwmma::Coord2d coordOps()
    {
        auto c = rocwmma::make_coord2d(6u, 20u);
        c *= rocwmma::make_coord2d(2u, 3u); // 12, 60
        c -= rocwmma::make_coord2d(2u, 4u); // 10, 56
        c /= rocwmma::make_coord2d(2u, 8u); // 5, 7
        c %= rocwmma::make_coord2d(3u, 4u); // 2, 3
        c += rocwmma::make_coord2d(1u, 1u); // 3, 4
        return c;
    }
    static_assert(coordOps() == rocwmma::make_coord2d(3u, 4u) && coordOps() != rocwmma::make_coord2d(3u, 5u));
    static_assert(coordOps()[0] == 3u && coordOps()[1] == 4u && rocwmma::get<1>(coordOps()) == 4u);
    static_assert(rocwmma::make_coord2d(9u, 8u) / rocwmma::make_coord2d(2u, 4u) == rocwmma::make_coord2d(4u, 2u));
    static_assert(rocwmma::make_coord2d(9u, 8u) % rocwmma::make_coord2d(2u, 5u) == rocwmma::make_coord2d(1u, 3u));
} // namespace

extern "C" {

// Describes a case: rows, cols of the block in memory, element bytes; returns 0 if the id exists.
int api_case_info(int id, uint32_t* rows, uint32_t* cols, uint32_t* elemBytes, uint32_t* rowMajor, uint32_t* numElements)
{
    switch(id)
    {
#define X(ID, ROLE, M, N, K, T, L)                                     \
    case ID: {                                                         \
        using F    = fragment<ROLE, M, N, K, T, L>;                    \
        *rows      = GetIOShape_t<F>::BlockHeight;                     \
        *cols      = GetIOShape_t<F>::BlockWidth;                      \
        *elemBytes = sizeof(T);                                        \
        *rowMajor  = std::is_same_v<L, row_major>;                     \
        *numElements = F::num_elements;                                \
        return 0;                                                      \
    }
        FRAG_CASES(X)
#undef X
    default: return -1;
    }
}

int api_round_trip(int id, const void* in, void* out, uint32_t ldIn, uint32_t ldOut)
{
    switch(id)
    {
#define X(ID, ROLE, M, N, K, T, L)                                                                             \
    case ID:                                                                                                   \
        hipLaunchKernelGGL((roundTrip<fragment<ROLE, M, N, K, T, L>>), dim3(1), dim3(64), 0, 0,                \
                           static_cast<const T*>(in), static_cast<T*>(out), ldIn, ldOut);                      \
        break;
        FRAG_CASES(X)
#undef X
    default: return -1;
    }
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}

// runtime-layout overloads on the DataLayoutT = void fragment of the same shape
int api_round_trip_runtime(int id, const void* in, void* out, uint32_t ld)
{
    switch(id)
    {
#define X(ID, ROLE, M, N, K, T, L)                                                                              \
    case ID:                                                                                                    \
        hipLaunchKernelGGL((roundTripRuntime<fragment<ROLE, M, N, K, T>>), dim3(1), dim3(64), 0, 0,             \
                           static_cast<const T*>(in), static_cast<T*>(out), ld,                                 \
                           std::is_same_v<L, row_major> ? mem_row_major : mem_col_major);                       \
        break;
        FRAG_CASES(X)
#undef X
    default: return -1;
    }
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}

int api_fill(int id, void* out, uint32_t ld, float value)
{
    switch(id)
    {
#define X(ID, ROLE, M, N, K, T, L)                                                                         \
    case ID:                                                                                               \
        hipLaunchKernelGGL((fillStore<fragment<ROLE, M, N, K, T, L>>), dim3(1), dim3(64), 0, 0,            \
                           static_cast<T*>(out), ld, convert<T>(value));                                   \
        break;
        FRAG_CASES(X)
#undef X
    default: return -1;
    }
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}

// wavesX * wavesY waves share the fragment; useLds routes the data through LDS
int api_coop_round_trip(int id, const void* in, void* out, uint32_t ld, uint32_t wavesX, uint32_t wavesY, uint32_t useLds)
{
    switch(id)
    {
#define X(ID, ROLE, M, N, K, T, L)                                                                               \
    case ID:                                                                                                     \
        hipLaunchKernelGGL((coopRoundTrip<fragment<ROLE, M, N, K, T, L>>), dim3(1), dim3(64 * wavesX, wavesY),   \
                           (GetIOShape_t<fragment<ROLE, M, N, K, T, L>>::BlockHeight)                            \
                               * (GetIOShape_t<fragment<ROLE, M, N, K, T, L>>::BlockWidth) * sizeof(T),          \
                           0, static_cast<const T*>(in), static_cast<T*>(out), ld, useLds);                      \
        break;
        FRAG_CASES(X)
#undef X
    default: return -1;
    }
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}

// template-WaveCount overloads with 4 waves on the two big staging fragments (cases 17, 18)
int api_coop_round_trip_static4(int id, const void* in, void* out, uint32_t ld)
{
    using T = float16_t;
    if(id == 17)
        hipLaunchKernelGGL((coopRoundTripStatic<4, fragment<matrix_a, 128, 32, 16, T, col_major>>), dim3(1),
                           dim3(128, 2), 0, 0, static_cast<const T*>(in), static_cast<T*>(out), ld);
    else if(id == 18)
        hipLaunchKernelGGL((coopRoundTripStatic<4, fragment<matrix_b, 32, 128, 16, T, row_major>>), dim3(1),
                           dim3(128, 2), 0, 0, static_cast<const T*>(in), static_cast<T*>(out), ld);
    else
        return -1;
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}

int api_transpose_store(const void* in, void* out, uint32_t ld)
{
    using T = float16_t;
    hipLaunchKernelGGL((transposeStore<fragment<matrix_b, 32, 64, 16, T, row_major>>), dim3(1), dim3(64), 0, 0,
                       static_cast<const T*>(in), static_cast<T*>(out), ld);
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}

int api_relayout_store(const void* in, void* out, uint32_t ldIn, uint32_t ldOut)
{
    using T = float16_t;
    hipLaunchKernelGGL((relayoutStore<fragment<matrix_a, 32, 32, 16, T, row_major>, col_major>), dim3(1), dim3(64), 0,
                       0, static_cast<const T*>(in), static_cast<T*>(out), ldIn, ldOut);
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}

// one tile D = A B + C.  type: 0 f16, 1 bf16, 2 e4m3, 3 i8, 4 f32, 5 f16 accumulate, 6 f64, 7 e5m2, 8 bf16 accumulate, 9 / 10 __half (f32 / __half accumulate); blk 16 | 32; bk per the table in the test
int api_mma_tile(int type, uint32_t blk, uint32_t bk, int aRow, int bRow, int cRow, const void* a, const void* b,
                 const void* c, void* d, uint32_t lda, uint32_t ldb, uint32_t ldc)
{
    const layout_t lc = cRow ? mem_row_major : mem_col_major;
#define LAUNCH(BLK, BKK, T, ACC, LA, LB)                                                                      \
    hipLaunchKernelGGL((mmaTile<BLK, BKK, T, ACC, LA, LB>), dim3(1), dim3(64), 0, 0, static_cast<const T*>(a), \
                       static_cast<const T*>(b), static_cast<const ACC*>(c), static_cast<ACC*>(d), lda, ldb, ldc, lc)
#define LAYOUTS(BLK, BKK, T, ACC)                     \
    do                                                \
    {                                                 \
        if(aRow && bRow)                              \
            LAUNCH(BLK, BKK, T, ACC, row_major, row_major); \
        else if(aRow && !bRow)                        \
            LAUNCH(BLK, BKK, T, ACC, row_major, col_major); \
        else if(!aRow && bRow)                        \
            LAUNCH(BLK, BKK, T, ACC, col_major, row_major); \
        else                                          \
            LAUNCH(BLK, BKK, T, ACC, col_major, col_major); \
    } while(0)
#define SHAPE(T, ACC, B1, K1, B2, K2, B3, K3, B4, K4) \
    if(blk == B1 && bk == K1)                          \
        LAYOUTS(B1, K1, T, ACC);                       \
    else if(blk == B2 && bk == K2)                     \
        LAYOUTS(B2, K2, T, ACC);                       \
    else if(blk == B3 && bk == K3)                     \
        LAYOUTS(B3, K3, T, ACC);                       \
    else if(blk == B4 && bk == K4)                     \
        LAYOUTS(B4, K4, T, ACC);                       \
    else                                               \
        return -1
    switch(type)
    {
    case 0: SHAPE(float16_t, float32_t, 16, 16, 16, 32, 32, 8, 32, 16); break;
    case 1: SHAPE(bfloat16_t, float32_t, 16, 16, 16, 32, 32, 8, 32, 16); break;
    case 2: SHAPE(float8_t, float32_t, 16, 32, 16, 64, 32, 16, 32, 32); break;
    case 3: SHAPE(int8_t, int32_t, 16, 32, 16, 64, 32, 16, 32, 32); break;
    case 4: SHAPE(float32_t, float32_t, 16, 4, 16, 16, 32, 2, 32, 8); break;
    case 5: SHAPE(float16_t, float16_t, 16, 16, 16, 32, 32, 8, 32, 16); break; // 16-bit accumulate type
    case 6: SHAPE(float64_t, float64_t, 16, 4, 16, 8, 16, 16, 16, 32); break;
    case 7: SHAPE(bfloat8_t, float32_t, 16, 32, 16, 64, 32, 16, 32, 32); break;
    case 8: SHAPE(bfloat16_t, bfloat16_t, 16, 16, 16, 32, 32, 8, 32, 16); break;
    case 9: SHAPE(hfloat16_t, float32_t, 16, 16, 16, 32, 32, 8, 32, 16); break; // __half operands
    case 10: SHAPE(hfloat16_t, hfloat16_t, 16, 16, 16, 32, 32, 8, 32, 16); break;
    default: return -1;
    }
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}

// one sparse tile.  type: 0 f16, 1 bf16, 2 e4m3, 3 i8, 7 e5m2; blk 16 | 32; stages: K stages of 128 bytes (1 | 2)
int api_sparse_mma_tile(int type, uint32_t blk, uint32_t stages, int bRow, int cRow, const void* aVals, const void* aMeta,
                        const void* b, const void* c, void* d, uint32_t ldb, uint32_t ldc)
{
    const layout_t lc = cRow ? mem_row_major : mem_col_major;
#define SLAUNCH(BLK, BKK, T, ACC, LB)                                                                              \
    hipLaunchKernelGGL((sparseMmaTile<BLK, BKK, T, ACC, LB>), dim3(1), dim3(64), 0, 0, static_cast<const T*>(aVals), \
                       static_cast<const uint8_t*>(aMeta), static_cast<const T*>(b), static_cast<const ACC*>(c),    \
                       static_cast<ACC*>(d), ldb, ldc, lc)
#define SSHAPE(T, ACC, SK)                               \
    do                                                   \
    {                                                    \
        if(blk == 16 && stages == 1 && bRow)             \
            SLAUNCH(16, SK, T, ACC, row_major);          \
        else if(blk == 16 && stages == 1)                \
            SLAUNCH(16, SK, T, ACC, col_major);          \
        else if(blk == 16 && stages == 2 && bRow)        \
            SLAUNCH(16, 2 * SK, T, ACC, row_major);      \
        else if(blk == 16 && stages == 2)                \
            SLAUNCH(16, 2 * SK, T, ACC, col_major);      \
        else if(blk == 32 && stages == 1 && bRow)        \
            SLAUNCH(32, SK, T, ACC, row_major);          \
        else if(blk == 32 && stages == 1)                \
            SLAUNCH(32, SK, T, ACC, col_major);          \
        else if(blk == 32 && stages == 2 && bRow)        \
            SLAUNCH(32, 2 * SK, T, ACC, row_major);      \
        else if(blk == 32 && stages == 2)                \
            SLAUNCH(32, 2 * SK, T, ACC, col_major);      \
        else                                             \
            return -1;                                   \
    } while(0)
    switch(type)
    {
    case 0: SSHAPE(float16_t, float32_t, 64); break;
    case 1: SSHAPE(bfloat16_t, float32_t, 64); break;
    case 2: SSHAPE(float8_t, float32_t, 128); break;
    case 3: SSHAPE(int8_t, int32_t, 128); break;
    case 7: SSHAPE(bfloat8_t, float32_t, 128); break;
    default: return -1;
    }
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}

int api_mapping_probe(uint32_t* out, uint32_t ld, uint32_t gridX, uint32_t gridY, uint32_t wavesX, uint32_t wavesY)
{
    hipLaunchKernelGGL(mappingProbe, dim3(gridX, gridY), dim3(64 * wavesX, wavesY), 0, 0, out, ld);
    return hipDeviceSynchronize() == hipSuccess ? 0 : -2;
}

} // extern "C"
