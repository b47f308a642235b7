// 2-D coordinates and the small integer helpers kernels use for address arithmetic.
// Names follow rocWMMA (reference: library/include/rocwmma/internal/utils.hpp:56-75,145-175).
// Convention everywhere: get<0> is the row (x), get<1> is the column (y).
#ifndef ROCWMMA_COORD_HPP
#define ROCWMMA_COORD_HPP

#include "config.hpp"
#include <cstdint>
#include <type_traits>

namespace rocwmma
{
    using Coord2dDataT = uint32_t;

    struct Coord2d
    {
        Coord2dDataT x;
        Coord2dDataT y;
    };

    template <uint32_t I>
    ROCWMMA_HOST_DEVICE constexpr inline Coord2dDataT& get(Coord2d& c)
    {
        static_assert(I < 2, "Coord2d has two components");
        if constexpr(I == 0)
            return c.x;
        else
            return c.y;
    }

    template <uint32_t I>
    ROCWMMA_HOST_DEVICE constexpr inline Coord2dDataT const& get(Coord2d const& c)
    {
        static_assert(I < 2, "Coord2d has two components");
        if constexpr(I == 0)
            return c.x;
        else
            return c.y;
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d make_coord2d(Coord2dDataT x, Coord2dDataT y)
    {
        return Coord2d{x, y};
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d swap(Coord2d const& p)
    {
        return Coord2d{p.y, p.x};
    }

    ROCWMMA_HOST_DEVICE constexpr inline Coord2d operator*(Coord2d const& a, Coord2d const& b)
    {
        return Coord2d{a.x * b.x, a.y * b.y};
    }
    ROCWMMA_HOST_DEVICE constexpr inline Coord2d operator+(Coord2d const& a, Coord2d const& b)
    {
        return Coord2d{a.x + b.x, a.y + b.y};
    }
    ROCWMMA_HOST_DEVICE constexpr inline Coord2d operator-(Coord2d const& a, Coord2d const& b)
    {
        return Coord2d{a.x - b.x, a.y - b.y};
    }
    ROCWMMA_HOST_DEVICE constexpr inline Coord2d& operator+=(Coord2d& a, Coord2d const& b)
    {
        a.x += b.x;
        a.y += b.y;
        return a;
    }
    ROCWMMA_HOST_DEVICE constexpr inline Coord2d& operator-=(Coord2d& a, Coord2d const& b)
    {
        a.x -= b.x;
        a.y -= b.y;
        return a;
    }
    ROCWMMA_HOST_DEVICE constexpr inline Coord2d& operator*=(Coord2d& a, Coord2d const& b)
    {
        a.x *= b.x;
        a.y *= b.y;
        return a;
    }
    ROCWMMA_HOST_DEVICE constexpr inline bool operator==(Coord2d const& a, Coord2d const& b)
    {
        return a.x == b.x && a.y == b.y;
    }

    // ceil(numerator / divisor) for integers
    template <typename intT1,
              class = typename std::enable_if<std::is_integral<intT1>::value>::type,
              typename intT2,
              class = typename std::enable_if<std::is_integral<intT2>::value>::type>
    ROCWMMA_HOST_DEVICE constexpr intT1 ceilDiv(const intT1 numerator, const intT2 divisor)
    {
        return (numerator + divisor - 1) / divisor;
    }

    // Integer log2 of a power of two
    template <uint32_t x>
    struct Log2
    {
        static_assert(x % 2 == 0, "Integer input must be a power of 2");
        static constexpr uint32_t value = 1 + Log2<(x >> 1)>::value;
    };
    template <>
    struct Log2<1>
    {
        static constexpr uint32_t value = 0;
    };
    template <>
    struct Log2<0>
    {
        static constexpr uint32_t value = 0;
    };

    // Mask of the BitCount least significant bits
    template <uint32_t BitCount>
    struct LsbMask
    {
        enum : uint32_t
        {
            value = BitCount >= 32 ? 0xFFFFFFFFu : ((1u << (BitCount & 31u)) - 1u)
        };
    };

} // namespace rocwmma

#endif // ROCWMMA_COORD_HPP
