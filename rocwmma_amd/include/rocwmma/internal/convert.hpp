// Scalar conversions between the supported data types (host and device).
// Public name `convert<T>(v)` as in library/include/rocwmma/internal/convert.hpp:38-108.
#ifndef ROCWMMA_CONVERT_HPP
#define ROCWMMA_CONVERT_HPP

#include "types.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <typename T>
        ROCWMMA_HOST_DEVICE inline float to_f32(T const& v)
        {
            if constexpr(std::is_same_v<T, hfloat16_t>)
                return __half2float(v);
            else
                return static_cast<float>(v);
        }

        template <typename T>
        ROCWMMA_HOST_DEVICE inline T from_f32(float v)
        {
            if constexpr(std::is_same_v<T, hfloat16_t>)
                return __float2half(v);
            else if constexpr(std::is_same_v<T, bfloat16_t> || std::is_same_v<T, float8_t>
                              || std::is_same_v<T, bfloat8_t>)
                return T(v);
            else
                return static_cast<T>(v);
        }
    } // namespace detail

    // Value conversion: integers and wide floats cast directly, narrow floats round-trip
    // through f32 (f32 -> f16 / bf16 / e4m3 rounds to nearest even; e4m3 saturates).
    template <typename OutT, typename InT>
    ROCWMMA_HOST_DEVICE inline OutT convert(InT const& v)
    {
        if constexpr(std::is_same_v<OutT, InT>)
            return v;
        else if constexpr(std::is_arithmetic_v<InT> && std::is_arithmetic_v<OutT>
                          && !std::is_same_v<InT, float16_t> && !std::is_same_v<OutT, float16_t>)
            return static_cast<OutT>(v);
        else
            return detail::from_f32<OutT>(detail::to_f32<InT>(v));
    }
} // namespace rocwmma

#endif // ROCWMMA_CONVERT_HPP
