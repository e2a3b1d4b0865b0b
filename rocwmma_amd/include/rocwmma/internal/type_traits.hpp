// std::numeric_limits for the narrow floating types, as host helpers of kernels expect
// (samples/common.hpp:329-338 uses epsilon / infinity / signaling_NaN).
// Values: IEEE binary16; bfloat16 (8-bit exponent, 7-bit mantissa); OCP e4m3
// (max 0x7E = 448, epsilon 0x20 = 2^-3, NaN 0x7F, no infinity) as in
// library/include/rocwmma/internal/float8.hpp:529-580.
#ifndef ROCWMMA_TYPE_TRAITS_HPP
#define ROCWMMA_TYPE_TRAITS_HPP

#if !defined(__HIPCC_RTC__)
#include <limits>
#endif

#include "types.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <typename T, typename BitsT>
        ROCWMMA_HOST_DEVICE inline T from_bits(BitsT bits)
        {
            static_assert(sizeof(T) == sizeof(BitsT), "size mismatch");
            T r;
            __builtin_memcpy(&r, &bits, sizeof(T));
            return r;
        }
    } // namespace detail
} // namespace rocwmma

namespace std
{
#define ROCWMMA_LIMITS_FN(NAME, T, BITS_T, BITS)                       \
    ROCWMMA_HOST_DEVICE static inline T NAME() noexcept                \
    {                                                                  \
        return rocwmma::detail::from_bits<T, BITS_T>((BITS_T)(BITS)); \
    }

#if !defined(__STDCPP_FLOAT16_T__) && !defined(_GLIBCXX_FLOAT16_LIMITS)
    template <>
    class numeric_limits<rocwmma::float16_t>
    {
        using T = rocwmma::float16_t;

    public:
        static constexpr bool is_specialized = true, is_signed = true, is_integer = false,
                              is_exact = false, has_infinity = true, has_quiet_NaN = true,
                              has_signaling_NaN = true;
        static constexpr int digits = 11, radix = 2;
        ROCWMMA_LIMITS_FN(epsilon, T, uint16_t, 0x1400)
        ROCWMMA_LIMITS_FN(infinity, T, uint16_t, 0x7C00)
        ROCWMMA_LIMITS_FN(lowest, T, uint16_t, 0xFBFF)
        ROCWMMA_LIMITS_FN(max, T, uint16_t, 0x7BFF)
        ROCWMMA_LIMITS_FN(min, T, uint16_t, 0x0400)
        ROCWMMA_LIMITS_FN(quiet_NaN, T, uint16_t, 0x7FFF)
        ROCWMMA_LIMITS_FN(signaling_NaN, T, uint16_t, 0x7DFF)
    };
#endif

    template <>
    class numeric_limits<rocwmma::hfloat16_t>
    {
        using T = rocwmma::hfloat16_t;

    public:
        static constexpr bool is_specialized = true, is_signed = true, is_integer = false,
                              is_exact = false, has_infinity = true, has_quiet_NaN = true,
                              has_signaling_NaN = true;
        static constexpr int digits = 11, radix = 2;
        ROCWMMA_LIMITS_FN(epsilon, T, uint16_t, 0x1400)
        ROCWMMA_LIMITS_FN(infinity, T, uint16_t, 0x7C00)
        ROCWMMA_LIMITS_FN(lowest, T, uint16_t, 0xFBFF)
        ROCWMMA_LIMITS_FN(max, T, uint16_t, 0x7BFF)
        ROCWMMA_LIMITS_FN(min, T, uint16_t, 0x0400)
        ROCWMMA_LIMITS_FN(quiet_NaN, T, uint16_t, 0x7FFF)
        ROCWMMA_LIMITS_FN(signaling_NaN, T, uint16_t, 0x7DFF)
    };

    template <>
    class numeric_limits<rocwmma::bfloat16_t>
    {
        using T = rocwmma::bfloat16_t;

    public:
        static constexpr bool is_specialized = true, is_signed = true, is_integer = false,
                              is_exact = false, has_infinity = true, has_quiet_NaN = true,
                              has_signaling_NaN = true;
        static constexpr int digits = 8, radix = 2;
        ROCWMMA_LIMITS_FN(epsilon, T, uint16_t, 0x3C00)
        ROCWMMA_LIMITS_FN(infinity, T, uint16_t, 0x7F80)
        ROCWMMA_LIMITS_FN(lowest, T, uint16_t, 0xFF7F)
        ROCWMMA_LIMITS_FN(max, T, uint16_t, 0x7F7F)
        ROCWMMA_LIMITS_FN(min, T, uint16_t, 0x0080)
        ROCWMMA_LIMITS_FN(quiet_NaN, T, uint16_t, 0x7FC0)
        ROCWMMA_LIMITS_FN(signaling_NaN, T, uint16_t, 0x7FA0)
    };

    template <>
    class numeric_limits<rocwmma::float8_t>
    {
        using T = rocwmma::float8_t;

    public:
        static constexpr bool is_specialized = true, is_signed = true, is_integer = false,
                              is_exact = false, has_infinity = false, has_quiet_NaN = true,
                              has_signaling_NaN = false;
        static constexpr int digits = 4, radix = 2;
        ROCWMMA_LIMITS_FN(epsilon, T, uint8_t, 0x20)
        ROCWMMA_LIMITS_FN(infinity, T, uint8_t, 0x7E) // no infinity in the format: max finite
        ROCWMMA_LIMITS_FN(lowest, T, uint8_t, 0xFE)
        ROCWMMA_LIMITS_FN(max, T, uint8_t, 0x7E)
        ROCWMMA_LIMITS_FN(min, T, uint8_t, 0x08)
        ROCWMMA_LIMITS_FN(quiet_NaN, T, uint8_t, 0x7F)
        ROCWMMA_LIMITS_FN(signaling_NaN, T, uint8_t, 0x7F)
    };
#undef ROCWMMA_LIMITS_FN
} // namespace std

#endif // ROCWMMA_TYPE_TRAITS_HPP
