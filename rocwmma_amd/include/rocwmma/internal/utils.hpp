// Small constexpr helpers used by kernels: 2-d coordinates, ceilDiv, Log2.
// Public names follow library/include/rocwmma/internal/utils.hpp:56-77,140-168.
#ifndef ROCWMMA_UTILS_HPP
#define ROCWMMA_UTILS_HPP

#include "types.hpp"

namespace rocwmma
{
    using Coord2dDataT = uint32_t;

    // (x, y) pair usable in constant expressions on host and device, with the element-wise arithmetic the
    // reference's two-element vector offers (vector.hpp:157-214 there): user kernels scale and step coordinates
    // in place (test/gemm/gemm_PGR0_LB0_MP0_MB_NC/device/kernel_device_func.hpp:110).
    struct Coord2d
    {
        Coord2dDataT x;
        Coord2dDataT y;

        ROCWMMA_HOST_DEVICE constexpr inline Coord2dDataT& operator[](unsigned int idx) noexcept
        {
            return idx == 0u ? x : y;
        }
        ROCWMMA_HOST_DEVICE constexpr inline Coord2dDataT operator[](unsigned int idx) const noexcept
        {
            return idx == 0u ? x : y;
        }
    };

    template <uint32_t Idx>
    ROCWMMA_HOST_DEVICE constexpr inline Coord2dDataT& get(Coord2d& c)
    {
        static_assert(Idx < 2u, "Coord2d has two components");
        return Idx == 0u ? c.x : c.y;
    }

    template <uint32_t Idx>
    ROCWMMA_HOST_DEVICE constexpr inline Coord2dDataT const& get(Coord2d const& c)
    {
        static_assert(Idx < 2u, "Coord2d has two components");
        return Idx == 0u ? c.x : c.y;
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d make_coord2d(Coord2dDataT x, Coord2dDataT y)
    {
        return Coord2d{x, y};
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d swap(Coord2d const& p)
    {
        return Coord2d{p.y, p.x};
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d operator*(Coord2d const& l, Coord2d const& r)
    {
        return Coord2d{l.x * r.x, l.y * r.y};
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d operator+(Coord2d const& l, Coord2d const& r)
    {
        return Coord2d{l.x + r.x, l.y + r.y};
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d operator-(Coord2d const& l, Coord2d const& r)
    {
        return Coord2d{l.x - r.x, l.y - r.y};
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d& operator+=(Coord2d& l, Coord2d const& r)
    {
        l.x += r.x;
        l.y += r.y;
        return l;
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d operator/(Coord2d const& l, Coord2d const& r)
    {
        return Coord2d{l.x / r.x, l.y / r.y};
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d operator%(Coord2d const& l, Coord2d const& r)
    {
        return Coord2d{l.x % r.x, l.y % r.y};
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d& operator-=(Coord2d& l, Coord2d const& r)
    {
        l.x -= r.x;
        l.y -= r.y;
        return l;
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d& operator*=(Coord2d& l, Coord2d const& r)
    {
        l.x *= r.x;
        l.y *= r.y;
        return l;
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d& operator/=(Coord2d& l, Coord2d const& r)
    {
        l.x /= r.x;
        l.y /= r.y;
        return l;
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d& operator%=(Coord2d& l, Coord2d const& r)
    {
        l.x %= r.x;
        l.y %= r.y;
        return l;
    }

    ROCWMMA_HOST_DEVICE constexpr inline bool operator==(Coord2d const& l, Coord2d const& r)
    {
        return l.x == r.x && l.y == r.y;
    }

    ROCWMMA_HOST_DEVICE constexpr inline bool operator!=(Coord2d const& l, Coord2d const& r)
    {
        return !(l == r);
    }

    template <typename IntT1,
              typename IntT2,
              typename = std::enable_if_t<std::is_integral_v<IntT1> && std::is_integral_v<IntT2>>>
    ROCWMMA_HOST_DEVICE constexpr inline IntT1 ceilDiv(const IntT1 numerator, const IntT2 divisor)
    {
        return (numerator + divisor - 1) / divisor;
    }

    template <uint32_t X>
    struct Log2
    {
        static_assert(X != 0u && (X & (X - 1u)) == 0u, "Integer input must be a power of 2");
        static constexpr uint32_t value = 1u + Log2<(X >> 1)>::value;
    };

    template <>
    struct Log2<1u>
    {
        static constexpr uint32_t value = 0u;
    };

    namespace detail
    {
        constexpr inline bool isPow2(uint32_t x)
        {
            return x != 0u && (x & (x - 1u)) == 0u;
        }

        constexpr inline uint32_t cmin(uint32_t a, uint32_t b)
        {
            return a < b ? a : b;
        }
    } // namespace detail

    // Short printable tag of a type, for logs and benchmark tables (utils.hpp:196-325 of the reference).
    // Primary template has no definition: user code may specialise it for its own tag types.
    template <typename DataT>
    constexpr const char* dataTypeToString();

#define ROCWMMA_TYPE_TAG(TYPE, TAG)                            \
    template <>                                                \
    constexpr const char* dataTypeToString<TYPE>()             \
    {                                                          \
        return TAG;                                            \
    }
    ROCWMMA_TYPE_TAG(float8_t, "f8")
    ROCWMMA_TYPE_TAG(bfloat8_t, "bf8")
    ROCWMMA_TYPE_TAG(float8_fnuz_t, "f8(fnuz)")
    ROCWMMA_TYPE_TAG(bfloat8_fnuz_t, "bf8(fnuz)")
    ROCWMMA_TYPE_TAG(float16_t, "f16")
    ROCWMMA_TYPE_TAG(hfloat16_t, "h16")
    ROCWMMA_TYPE_TAG(bfloat16_t, "bf16")
    ROCWMMA_TYPE_TAG(float32_t, "f32")
    ROCWMMA_TYPE_TAG(xfloat32_t, "xf32")
    ROCWMMA_TYPE_TAG(float64_t, "f64")
    ROCWMMA_TYPE_TAG(int8_t, "i8")
    ROCWMMA_TYPE_TAG(uint8_t, "u8")
    ROCWMMA_TYPE_TAG(int16_t, "i16")
    ROCWMMA_TYPE_TAG(uint16_t, "u16")
    ROCWMMA_TYPE_TAG(int32_t, "i32")
    ROCWMMA_TYPE_TAG(uint32_t, "u32")
    ROCWMMA_TYPE_TAG(uint64_t, "u64")
    ROCWMMA_TYPE_TAG(row_major, "T")
    ROCWMMA_TYPE_TAG(col_major, "N")
#undef ROCWMMA_TYPE_TAG

} // namespace rocwmma

#endif // ROCWMMA_UTILS_HPP
