// What a hipRTC compilation lacks: it has no host headers (no <cstdint>, <type_traits>, <limits>,
// no <hip/hip_fp8.h>), only the declarations hipRTC pre-includes (__half, hip_bfloat16, the
// builtins).  This header supplies the handful of names the library uses, so that a kernel string
// that includes <rocwmma/rocwmma.hpp> compiles under hiprtcCompileProgram as it does for the
// reference (samples/hipRTC_gemm.cpp:73-183, options :206).  Included only when __HIPCC_RTC__ is defined.
#ifndef ROCWMMA_RTC_COMPAT_HPP
#define ROCWMMA_RTC_COMPAT_HPP

#if defined(__HIPCC_RTC__)

// fixed-width integers at global scope, as kernel sources written against <cstdint> expect
using int8_t   = signed char;
using uint8_t  = unsigned char;
using int16_t  = short;
using uint16_t = unsigned short;
using int32_t  = int;
using uint32_t = unsigned int;
using int64_t  = long long;
using uint64_t = unsigned long long;

// fp8 storage types: hipRTC ships no fp8 header.  Fragments of these types load, multiply and
// store (the matrix cores do the arithmetic); scalar conversion to and from float is not
// available in a run-time compiled kernel.
struct __hip_fp8_e4m3
{
    unsigned char __x;
};
struct __hip_fp8_e5m2
{
    unsigned char __x;
};
struct __hip_fp8_e4m3_fnuz
{
    unsigned char __x;
};
struct __hip_fp8_e5m2_fnuz
{
    unsigned char __x;
};

// the subset of <type_traits> and <limits> the library uses
namespace std
{
    template <typename T, T V>
    struct integral_constant
    {
        static constexpr T value = V;
        using value_type         = T;
        constexpr operator T() const noexcept
        {
            return V;
        }
    };
    using true_type  = integral_constant<bool, true>;
    using false_type = integral_constant<bool, false>;

    template <typename T, typename U>
    inline constexpr bool is_same_v = false;
    template <typename T>
    inline constexpr bool is_same_v<T, T> = true;
    template <typename T, typename U>
    struct is_same : integral_constant<bool, is_same_v<T, U>>
    {
    };

    template <bool B, typename T, typename F>
    struct conditional
    {
        using type = T;
    };
    template <typename T, typename F>
    struct conditional<false, T, F>
    {
        using type = F;
    };
    template <bool B, typename T, typename F>
    using conditional_t = typename conditional<B, T, F>::type;

    template <bool B, typename T = void>
    struct enable_if
    {
    };
    template <typename T>
    struct enable_if<true, T>
    {
        using type = T;
    };
    template <bool B, typename T = void>
    using enable_if_t = typename enable_if<B, T>::type;

    template <typename T>
    struct remove_reference
    {
        using type = T;
    };
    template <typename T>
    struct remove_reference<T&>
    {
        using type = T;
    };
    template <typename T>
    struct remove_reference<T&&>
    {
        using type = T;
    };
    template <typename T>
    using remove_reference_t = typename remove_reference<T>::type;

    template <typename T>
    struct remove_cv
    {
        using type = T;
    };
    template <typename T>
    struct remove_cv<const T>
    {
        using type = T;
    };
    template <typename T>
    struct remove_cv<volatile T>
    {
        using type = T;
    };
    template <typename T>
    struct remove_cv<const volatile T>
    {
        using type = T;
    };
    template <typename T>
    using remove_cv_t = typename remove_cv<T>::type;

    // no array or function types reach the library's uses of decay
    template <typename T>
    using decay_t = remove_cv_t<remove_reference_t<T>>;

    template <typename T>
    inline constexpr bool is_const_v = false;
    template <typename T>
    inline constexpr bool is_const_v<const T> = true;
    template <typename T>
    inline constexpr bool is_lvalue_reference_v = false;
    template <typename T>
    inline constexpr bool is_lvalue_reference_v<T&> = true;

    namespace rtc_detail
    {
        template <typename T>
        inline constexpr bool integral_v
            = is_same_v<T, bool> || is_same_v<T, char> || is_same_v<T, signed char> || is_same_v<T, unsigned char>
              || is_same_v<T, short> || is_same_v<T, unsigned short> || is_same_v<T, int> || is_same_v<T, unsigned int>
              || is_same_v<T, long> || is_same_v<T, unsigned long> || is_same_v<T, long long>
              || is_same_v<T, unsigned long long>;
        template <typename T>
        inline constexpr bool floating_v = is_same_v<T, float> || is_same_v<T, double> || is_same_v<T, long double>
                                           || is_same_v<T, _Float16>;
    }
    template <typename T>
    inline constexpr bool is_integral_v = rtc_detail::integral_v<remove_cv_t<T>>;
    template <typename T>
    inline constexpr bool is_floating_point_v = rtc_detail::floating_v<remove_cv_t<T>>;
    template <typename T>
    inline constexpr bool is_arithmetic_v = is_integral_v<T> || is_floating_point_v<T>;
    template <typename T, bool = is_arithmetic_v<T>>
    inline constexpr bool is_signed_v = false;
    template <typename T>
    inline constexpr bool is_signed_v<T, true> = T(-1) < T(0);

    // primary template only: the library specialises it for its narrow floating types
    template <typename T>
    class numeric_limits;
} // namespace std

#endif // __HIPCC_RTC__
#endif // ROCWMMA_RTC_COMPAT_HPP
