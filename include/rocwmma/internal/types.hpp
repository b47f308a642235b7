// Element types of the library and their per-type facts.
// Public aliases follow rocWMMA's names (reference: library/include/rocwmma/internal/types.hpp:48-114).
// FP8 types are the OCP formats (E4M3 with max 448 / E5M2), which is what gfx950's matrix
// cores implement; the fnuz formats of earlier parts do not exist here.
#ifndef ROCWMMA_TYPES_HPP
#define ROCWMMA_TYPES_HPP

#include <cstdint>
#include <type_traits>

#include <hip/hip_bfloat16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_fp8.h>

#include "config.hpp"

namespace rocwmma
{
    using float16_t = _Float16;
    using float32_t = float;
    using float64_t = double;

    using int8_t   = ::int8_t;
    using uint8_t  = ::uint8_t;
    using int16_t  = ::int16_t;
    using uint16_t = ::uint16_t;
    using int32_t  = ::int32_t;
    using uint32_t = ::uint32_t;
    using int64_t  = ::int64_t;
    using uint64_t = ::uint64_t;
    using index_t  = ::int32_t;

    using bfloat16_t = hip_bfloat16;
#if !ROCWMMA_NO_HALF
    using hfloat16_t = __half;
#endif
    using float8_t  = __hip_fp8_e4m3;
    using bfloat8_t = __hip_fp8_e5m2;

    // Names of element types of other devices, kept so that code which only *mentions* them
    // (type lists, std::is_same tests; e.g. the reference's test/gemm/gemm_test_traits.hpp:115-185)
    // still compiles.  gfx950's matrix cores have neither the fnuz fp8 formats nor xf32: these
    // types cannot be the element type of a fragment here.
    using float8_fnuz_t  = __hip_fp8_e4m3_fnuz;
    using bfloat8_fnuz_t = __hip_fp8_e5m2_fnuz;
    struct xfloat32_t
    {
        float data;
    };

    namespace detail
    {
        // Matrix-core operand class of an element type.
        enum class MmaClass : uint32_t
        {
            None,
            F16,
            BF16,
            F8, // E4M3
            BF8, // E5M2
            I8,
            F32,
            F64
        };

        template <typename T>
        struct TypeInfo
        {
            static constexpr MmaClass cls = MmaClass::None;
        };
        template <>
        struct TypeInfo<float16_t>
        {
            static constexpr MmaClass cls = MmaClass::F16;
        };
#if !ROCWMMA_NO_HALF
        template <>
        struct TypeInfo<hfloat16_t>
        {
            static constexpr MmaClass cls = MmaClass::F16;
        };
#endif
        template <>
        struct TypeInfo<bfloat16_t>
        {
            static constexpr MmaClass cls = MmaClass::BF16;
        };
        template <>
        struct TypeInfo<float8_t>
        {
            static constexpr MmaClass cls = MmaClass::F8;
        };
        template <>
        struct TypeInfo<bfloat8_t>
        {
            static constexpr MmaClass cls = MmaClass::BF8;
        };
        template <>
        struct TypeInfo<int8_t>
        {
            static constexpr MmaClass cls = MmaClass::I8;
        };
        template <>
        struct TypeInfo<float32_t>
        {
            static constexpr MmaClass cls = MmaClass::F32;
        };
        template <>
        struct TypeInfo<float64_t>
        {
            static constexpr MmaClass cls = MmaClass::F64;
        };

        // Plain register words used to move fragments without caring about element type.
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2), may_alias));
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4), may_alias));
        typedef uint32_t u32x1 __attribute__((may_alias));
        typedef uint16_t u16x1 __attribute__((may_alias));
        typedef uint8_t  u8x1 __attribute__((may_alias));
    } // namespace detail

    // Minimal fixed-size vector used for the packed / unpacked fragment views.
    template <typename T, uint32_t N>
    struct VecT
    {
        using value_type = T;
        T data[N];

        ROCWMMA_HOST_DEVICE constexpr static uint32_t size()
        {
            return N;
        }
        ROCWMMA_HOST_DEVICE T& operator[](uint32_t i)
        {
            return data[i];
        }
        ROCWMMA_HOST_DEVICE T const& operator[](uint32_t i) const
        {
            return data[i];
        }
    };

    // How many elements of T share one 32-bit register, and the register word type.
    // (reference: library/include/rocwmma/internal/pack_util_impl.hpp:37-239)
    template <typename T>
    struct PackTraits
    {
        static constexpr uint32_t PackRatio = sizeof(T) >= 4 ? 1u : 4u / sizeof(T);
        using UnpackedT                     = T;
        using PackedT = std::conditional_t<
            (sizeof(T) > 4),
            T,
            std::conditional_t<std::is_same<T, float32_t>::value,
                               float32_t,
                               std::conditional_t<std::is_integral<T>::value && std::is_signed<T>::value,
                                                  int32_t,
                                                  std::conditional_t<std::is_integral<T>::value,
                                                                     uint32_t,
                                                                     float32_t>>>>;
    };

} // namespace rocwmma

#endif // ROCWMMA_TYPES_HPP
