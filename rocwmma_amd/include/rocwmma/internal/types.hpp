// Scalar data types, matrix/layout tags and clang vector aliases.
//
// Same public names as the reference (library/include/rocwmma/internal/types.hpp:48-114):
// float16_t = _Float16, hfloat16_t = __half, bfloat16_t = hip_bfloat16,
// float8_t = OCP e4m3 (hip_fp8_e4m3).  Registers are plain clang ext_vector_type
// values; there is no wrapper vector class.
#ifndef ROCWMMA_TYPES_HPP
#define ROCWMMA_TYPES_HPP

#if defined(__HIPCC_RTC__)
#include "rtc_compat.hpp"
#else
#include <cstdint>
#include <type_traits>

#include <hip/hip_runtime.h>
#include <hip/hip_bfloat16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_fp8.h>
#endif

#include "config.hpp"

using hip_fp8_e4m3 = __hip_fp8_e4m3;
using hip_fp8_e5m2 = __hip_fp8_e5m2;
using hip_fp8_e4m3_fnuz = __hip_fp8_e4m3_fnuz;
using hip_fp8_e5m2_fnuz = __hip_fp8_e5m2_fnuz;

namespace rocwmma
{
    using float16_t  = _Float16;
    using hfloat16_t = __half;
    using bfloat16_t = hip_bfloat16;
    using float8_t   = hip_fp8_e4m3;
    using bfloat8_t  = hip_fp8_e5m2;
    // Storage-only names kept for source compatibility (types.hpp:108-114 of the reference): gfx950's
    // matrix cores take the OCP encodings only and have no xf32 form, so mma_sync rejects these.
    using float8_fnuz_t  = hip_fp8_e4m3_fnuz;
    using bfloat8_fnuz_t = hip_fp8_e5m2_fnuz;
    struct xfloat32_t
    {
        float data;
    };
    using float32_t  = float;
    using float64_t  = double;
    using int8_t     = ::int8_t;
    using uint8_t    = ::uint8_t;
    using int16_t    = ::int16_t;
    using uint16_t   = ::uint16_t;
    using int32_t    = ::int32_t;
    using uint32_t   = ::uint32_t;
    using int64_t    = ::int64_t;
    using uint64_t   = ::uint64_t;
    using index_t    = ::int32_t;

    // Matrix roles
    struct matrix_a;
    struct matrix_b;
    struct accumulator;

    // Memory orientations
    struct row_major;
    struct col_major;

    // Runtime orientation for accumulator fragments declared with DataLayoutT = void
    enum layout_t : uint32_t
    {
        mem_row_major,
        mem_col_major
    };

    namespace detail
    {
        template <typename T, uint32_t N>
        using vec_t = T __attribute__((ext_vector_type(N)));

        template <typename T>
        inline constexpr bool is_f16_v = std::is_same_v<T, float16_t> || std::is_same_v<T, hfloat16_t>;
        template <typename T>
        inline constexpr bool is_bf16_v = std::is_same_v<T, bfloat16_t>;
        template <typename T>
        inline constexpr bool is_fp8_v = std::is_same_v<T, float8_t>;
        template <typename T>
        inline constexpr bool is_bf8_v = std::is_same_v<T, bfloat8_t>;
        template <typename T>
        inline constexpr bool is_i8_v = std::is_same_v<T, int8_t> || std::is_same_v<T, uint8_t>;

        // Orthogonal orientation
        template <typename L>
        struct orthogonal_layout
        {
            using type = void;
        };
        template <>
        struct orthogonal_layout<row_major>
        {
            using type = col_major;
        };
        template <>
        struct orthogonal_layout<col_major>
        {
            using type = row_major;
        };
    } // namespace detail

    template <typename L>
    using orthogonal_layout_t = typename detail::orthogonal_layout<L>::type;

    // How many elements of DataT share one 32-bit register, and the register's element type
    // (same names as the reference's pack_util.hpp:42-53 / pack_util_impl.hpp:36-200).
    template <typename DataT>
    struct PackTraits
    {
        enum : uint32_t
        {
            PackRatio = sizeof(DataT) >= 4u ? 1u : 4u / sizeof(DataT)
        };
        using UnpackedT = DataT;
        using PackedT   = std::conditional_t<
            sizeof(DataT) >= 4u,
            DataT,
            std::conditional_t<std::is_integral_v<DataT>,
                               std::conditional_t<std::is_signed_v<DataT>, int32_t, uint32_t>,
                               float32_t>>;
    };

} // namespace rocwmma

#endif // ROCWMMA_TYPES_HPP
