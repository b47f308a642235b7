// numeric_limits for the library's small floating-point types and a generic element
// conversion helper.  Host harness code written against rocWMMA includes this header by
// this path (reference: library/include/rocwmma/internal/type_traits.hpp, used by
// samples/common.hpp:62,195,399-408).
#ifndef ROCWMMA_TYPE_TRAITS_HPP
#define ROCWMMA_TYPE_TRAITS_HPP

#include <limits>
#include <type_traits>

#include "types.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <typename T, typename BitsT>
        ROCWMMA_HOST_DEVICE inline T fromBits(BitsT bits)
        {
            static_assert(sizeof(T) == sizeof(BitsT), "bit pattern width must match the type");
            T out;
            __builtin_memcpy(&out, &bits, sizeof(T));
            return out;
        }

        // Bit patterns of the characteristic values of each small float type.
        template <typename T>
        struct SmallFloatBits;
        template <>
        struct SmallFloatBits<float16_t>
        {
            using Bits = uint16_t;
            static constexpr Bits eps = 0x1400, inf = 0x7C00, qnan = 0x7E00, snan = 0x7D00, max = 0x7BFF,
                                  min = 0x0400, denorm = 0x0001, sign = 0x8000;
            static constexpr int digits = 11;
        };
        template <>
        struct SmallFloatBits<bfloat16_t>
        {
            using Bits = uint16_t;
            static constexpr Bits eps = 0x3C00, inf = 0x7F80, qnan = 0x7FC0, snan = 0x7FA0, max = 0x7F7F,
                                  min = 0x0080, denorm = 0x0001, sign = 0x8000;
            static constexpr int digits = 8;
        };
        template <>
        struct SmallFloatBits<float8_t> // OCP E4M3: no infinity, max 448
        {
            using Bits = uint8_t;
            static constexpr Bits eps = 0x20, inf = 0x7E, qnan = 0x7F, snan = 0x7F, max = 0x7E, min = 0x08,
                                  denorm = 0x01, sign = 0x80;
            static constexpr int digits = 4;
        };
        template <>
        struct SmallFloatBits<bfloat8_t> // OCP E5M2
        {
            using Bits = uint8_t;
            static constexpr Bits eps = 0x34, inf = 0x7C, qnan = 0x7E, snan = 0x7D, max = 0x7B, min = 0x04,
                                  denorm = 0x01, sign = 0x80;
            static constexpr int digits = 3;
        };

        template <typename T>
        struct SmallFloatLimits
        {
            using B = SmallFloatBits<T>;

            static constexpr bool is_specialized    = true;
            static constexpr bool is_signed         = true;
            static constexpr bool is_integer        = false;
            static constexpr bool is_exact          = false;
            static constexpr bool has_infinity      = !std::is_same<T, float8_t>::value;
            static constexpr bool has_quiet_NaN     = true;
            static constexpr bool has_signaling_NaN = true;
            static constexpr bool is_iec559         = false;
            static constexpr bool is_bounded        = true;
            static constexpr bool is_modulo         = false;
            static constexpr int  digits            = B::digits;
            static constexpr int  radix             = 2;

            ROCWMMA_HOST_DEVICE static T epsilon() noexcept
            {
                return fromBits<T>(B::eps);
            }
            ROCWMMA_HOST_DEVICE static T infinity() noexcept
            {
                return fromBits<T>(B::inf);
            }
            ROCWMMA_HOST_DEVICE static T quiet_NaN() noexcept
            {
                return fromBits<T>(B::qnan);
            }
            ROCWMMA_HOST_DEVICE static T signaling_NaN() noexcept
            {
                return fromBits<T>(B::snan);
            }
            ROCWMMA_HOST_DEVICE static T max() noexcept
            {
                return fromBits<T>(B::max);
            }
            ROCWMMA_HOST_DEVICE static T min() noexcept
            {
                return fromBits<T>(B::min);
            }
            ROCWMMA_HOST_DEVICE static T lowest() noexcept
            {
                return fromBits<T>(static_cast<typename B::Bits>(B::max | B::sign));
            }
            ROCWMMA_HOST_DEVICE static T denorm_min() noexcept
            {
                return fromBits<T>(B::denorm);
            }
            ROCWMMA_HOST_DEVICE static T round_error() noexcept
            {
                return static_cast<T>(0.5f);
            }
        };
    } // namespace detail

    // Element conversion through float for types without a direct conversion.
    template <typename To, typename From>
    ROCWMMA_HOST_DEVICE inline To convert(From const& value)
    {
        if constexpr(std::is_same<To, From>::value)
            return value;
        else if constexpr(std::is_convertible<From, To>::value
                          && (std::is_arithmetic<From>::value || std::is_same<From, float16_t>::value)
                          && (std::is_arithmetic<To>::value || std::is_same<To, float16_t>::value))
            return static_cast<To>(value);
        else
            return static_cast<To>(static_cast<float>(value));
    }

} // namespace rocwmma

namespace std
{
    template <>
    class numeric_limits<rocwmma::float16_t> : public rocwmma::detail::SmallFloatLimits<rocwmma::float16_t>
    {
    };
    template <>
    class numeric_limits<rocwmma::bfloat16_t> : public rocwmma::detail::SmallFloatLimits<rocwmma::bfloat16_t>
    {
    };
    template <>
    class numeric_limits<rocwmma::float8_t> : public rocwmma::detail::SmallFloatLimits<rocwmma::float8_t>
    {
    };
    template <>
    class numeric_limits<rocwmma::bfloat8_t> : public rocwmma::detail::SmallFloatLimits<rocwmma::bfloat8_t>
    {
    };
} // namespace std

#endif // ROCWMMA_TYPE_TRAITS_HPP
