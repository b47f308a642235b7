// gfx950 (CDNA4) matrix-core instruction table.
//
// One specialisation per (A class, B class, accumulator type, tile edge, K run per lane).
// Each exec() issues exactly one v_mfma instruction:  acc += X * Y  where X supplies the
// rows of the MFMA result and Y its columns.  (rocWMMA keeps an equivalent table for
// gfx908..gfx942, reference: library/include/rocwmma/internal/mfma_impl.hpp:159-699; this
// one is new and adds the double-rate wide-K CDNA4 shapes.)
//
//   class  tile  kpack  instruction                          K per instruction
//   f16    16    8      v_mfma_f32_16x16x32_f16              32
//   f16    16    4      v_mfma_f32_16x16x16_f16              16
//   f16    32    8      v_mfma_f32_32x32x16_f16              16
//   f16    32    4      v_mfma_f32_32x32x8_f16               8
//   bf16   (same four shapes, *_bf16 / *_bf16_1k)
//   fp8    16    32     v_mfma_f32_16x16x128_f8f6f4          128   (e4m3 / e5m2 in any mix; two 16-byte runs
//                                                                  per lane, see fragment_map.hpp)
//   fp8    16    8      v_mfma_f32_16x16x32_{fp8,bf8}_{fp8,bf8}   32
//   fp8    32    32     v_mfma_f32_32x32x64_f8f6f4           64
//   fp8    32    8      v_mfma_f32_32x32x16_{fp8,bf8}_{fp8,bf8}   16
//   i8     16    16     v_mfma_i32_16x16x64_i8               64
//   i8     16    8      v_mfma_i32_16x16x32_i8               32
//   i8     32    16     v_mfma_i32_32x32x32_i8               32
//   i8     32    8      v_mfma_i32_32x32x16_i8               16
//   f32    16    1      v_mfma_f32_16x16x4_f32               4
//   f32    32    1      v_mfma_f32_32x32x2_f32               2
//   f64    16    1      v_mfma_f64_16x16x4_f64               4   (results strided over rows: AccMapStrided)
#ifndef ROCWMMA_MFMA_GFX950_HPP
#define ROCWMMA_MFMA_GFX950_HPP

#include "types.hpp"

namespace rocwmma
{
    namespace detail
    {
        typedef _Float16 f16x4_t __attribute__((ext_vector_type(4), may_alias));
        typedef _Float16 f16x8_t __attribute__((ext_vector_type(8), may_alias));
        typedef __bf16   bf16x8_t __attribute__((ext_vector_type(8), may_alias));
        typedef short    s16x4_t __attribute__((ext_vector_type(4), may_alias));
        typedef int      i32x4_t __attribute__((ext_vector_type(4), may_alias));
        typedef int      i32x8_t __attribute__((ext_vector_type(8), may_alias));
        typedef int      i32x16_t __attribute__((ext_vector_type(16), may_alias));
        typedef float    f32x4_t __attribute__((ext_vector_type(4), may_alias));
        typedef float    f32x16_t __attribute__((ext_vector_type(16), may_alias));
        typedef long     i64x1_t __attribute__((may_alias));
        typedef float    f32x1_t __attribute__((may_alias));
        typedef double   f64x1_t __attribute__((may_alias));
        typedef double   f64x4_t __attribute__((ext_vector_type(4), may_alias));

        // Accumulator register block of one MFMA: 4 (16x16) or 16 (32x32) values.
        template <typename AccT, uint32_t Tile>
        struct AccRegs;
        template <>
        struct AccRegs<float, 16>
        {
            using type = f32x4_t;
        };
        template <>
        struct AccRegs<float, 32>
        {
            using type = f32x16_t;
        };
        template <>
        struct AccRegs<int32_t, 16>
        {
            using type = i32x4_t;
        };
        template <>
        struct AccRegs<double, 16>
        {
            using type = f64x4_t;
        };
        template <>
        struct AccRegs<int32_t, 32>
        {
            using type = i32x16_t;
        };

        // f8f6f4 format selectors (cbsz for the first multiplicand, blgp for the second)
        template <MmaClass C>
        struct F8Format;
        template <>
        struct F8Format<MmaClass::F8>
        {
            static constexpr int value = 0; // E4M3
        };
        template <>
        struct F8Format<MmaClass::BF8>
        {
            static constexpr int value = 1; // E5M2
        };

        template <MmaClass CX, MmaClass CY, typename AccT, uint32_t Tile, uint32_t KPack>
        struct Mfma
        {
            static constexpr bool supported = false;
        };

#define ROCWMMA_MFMA_ENTRY(CX, CY, ACCT, TILE, KPACK, OPT, EXPR)                              \
    template <>                                                                               \
    struct Mfma<MmaClass::CX, MmaClass::CY, ACCT, TILE, KPACK>                                \
    {                                                                                         \
        static constexpr bool supported = true;                                               \
        using Acc                       = typename AccRegs<ACCT, TILE>::type;                 \
        /* x, y point at KPACK consecutive elements of the fragments' register arrays */      \
        ROCWMMA_DEVICE static ROCWMMA_INLINE Acc exec(const void* x, const void* y, Acc acc)  \
        {                                                                                     \
            const OPT& X = *reinterpret_cast<const OPT*>(x);                                  \
            const OPT& Y = *reinterpret_cast<const OPT*>(y);                                  \
            return EXPR;                                                                      \
        }                                                                                     \
    };

#if ROCWMMA_ARCH_GFX950
        // clang-format off
        ROCWMMA_MFMA_ENTRY(F16, F16, float, 16, 8, f16x8_t, __builtin_amdgcn_mfma_f32_16x16x32_f16(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(F16, F16, float, 16, 4, f16x4_t, __builtin_amdgcn_mfma_f32_16x16x16f16(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(F16, F16, float, 32, 8, f16x8_t, __builtin_amdgcn_mfma_f32_32x32x16_f16(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(F16, F16, float, 32, 4, f16x4_t, __builtin_amdgcn_mfma_f32_32x32x8f16(X, Y, acc, 0, 0, 0))

        ROCWMMA_MFMA_ENTRY(BF16, BF16, float, 16, 8, bf16x8_t, __builtin_amdgcn_mfma_f32_16x16x32_bf16(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(BF16, BF16, float, 16, 4, s16x4_t, __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(BF16, BF16, float, 32, 8, bf16x8_t, __builtin_amdgcn_mfma_f32_32x32x16_bf16(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(BF16, BF16, float, 32, 4, s16x4_t, __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(X, Y, acc, 0, 0, 0))

        ROCWMMA_MFMA_ENTRY(I8, I8, int32_t, 16, 16, i32x4_t, __builtin_amdgcn_mfma_i32_16x16x64_i8(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(I8, I8, int32_t, 16, 8, i64x1_t, __builtin_amdgcn_mfma_i32_16x16x32_i8(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(I8, I8, int32_t, 32, 16, i32x4_t, __builtin_amdgcn_mfma_i32_32x32x32_i8(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(I8, I8, int32_t, 32, 8, i64x1_t, __builtin_amdgcn_mfma_i32_32x32x16_i8(X, Y, acc, 0, 0, 0))

        ROCWMMA_MFMA_ENTRY(F8, F8, float, 16, 8, i64x1_t, __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(F8, BF8, float, 16, 8, i64x1_t, __builtin_amdgcn_mfma_f32_16x16x32_fp8_bf8(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(BF8, F8, float, 16, 8, i64x1_t, __builtin_amdgcn_mfma_f32_16x16x32_bf8_fp8(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(BF8, BF8, float, 16, 8, i64x1_t, __builtin_amdgcn_mfma_f32_16x16x32_bf8_bf8(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(F8, F8, float, 32, 8, i64x1_t, __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(F8, BF8, float, 32, 8, i64x1_t, __builtin_amdgcn_mfma_f32_32x32x16_fp8_bf8(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(BF8, F8, float, 32, 8, i64x1_t, __builtin_amdgcn_mfma_f32_32x32x16_bf8_fp8(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(BF8, BF8, float, 32, 8, i64x1_t, __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(X, Y, acc, 0, 0, 0))

        ROCWMMA_MFMA_ENTRY(F32, F32, float, 16, 1, f32x1_t, __builtin_amdgcn_mfma_f32_16x16x4f32(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(F32, F32, float, 32, 1, f32x1_t, __builtin_amdgcn_mfma_f32_32x32x2f32(X, Y, acc, 0, 0, 0))
        ROCWMMA_MFMA_ENTRY(F64, F64, double, 16, 1, f64x1_t, __builtin_amdgcn_mfma_f64_16x16x4f64(X, Y, acc, 0, 0, 0))

        // Wide-K fp8 family: one opcode, operand formats chosen by cbsz / blgp, scales unused
        // (scale operands of 0 select the unscaled form of the instruction).
#define ROCWMMA_MFMA_F8F6F4(CX, CY)                                                                                   \
        ROCWMMA_MFMA_ENTRY(CX, CY, float, 16, 32, i32x8_t,                                                            \
            __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(X, Y, acc, F8Format<MmaClass::CX>::value,                \
                                                             F8Format<MmaClass::CY>::value, 0, 0, 0, 0))              \
        ROCWMMA_MFMA_ENTRY(CX, CY, float, 32, 32, i32x8_t,                                                            \
            __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(X, Y, acc, F8Format<MmaClass::CX>::value,                 \
                                                            F8Format<MmaClass::CY>::value, 0, 0, 0, 0))
        ROCWMMA_MFMA_F8F6F4(F8, F8)
        ROCWMMA_MFMA_F8F6F4(F8, BF8)
        ROCWMMA_MFMA_F8F6F4(BF8, F8)
        ROCWMMA_MFMA_F8F6F4(BF8, BF8)
#undef ROCWMMA_MFMA_F8F6F4
        // clang-format on
#endif // ROCWMMA_ARCH_GFX950

        // The same wide-K family with block scales (OCP microscaling, MX): every 32 elements along K
        // of a row share an E8M0 scale (a biased power-of-two exponent: value = element *
        // 2^(scale - 127)).  Lane l passes, for each multiplicand, the scale of row (column) l % Tile and
        // K block l / Tile of the instruction's K range, in one byte of a 32-bit register.  SelX / SelY
        // choose that byte (instruction immediates), so one register can carry the scales of four
        // instructions.
        template <MmaClass CX, MmaClass CY, uint32_t Tile>
        struct MfmaScaled
        {
            static constexpr bool supported = false;
        };

#if ROCWMMA_ARCH_GFX950
#define ROCWMMA_MFMA_SCALED(CX, CY, TILE, SHAPE)                                                                     \
    template <>                                                                                                       \
    struct MfmaScaled<MmaClass::CX, MmaClass::CY, TILE>                                                              \
    {                                                                                                                 \
        static constexpr bool supported = true;                                                                       \
        using Acc                       = typename AccRegs<float, TILE>::type;                                        \
        template <int SelX = 0, int SelY = 0>                                                                         \
        ROCWMMA_DEVICE static ROCWMMA_INLINE Acc exec(const void* x, const void* y, Acc acc, uint32_t scaleX,         \
                                                      uint32_t scaleY)                                                \
        {                                                                                                             \
            const i32x8_t& X = *reinterpret_cast<const i32x8_t*>(x);                                                  \
            const i32x8_t& Y = *reinterpret_cast<const i32x8_t*>(y);                                                  \
            return __builtin_amdgcn_mfma_scale_f32_##SHAPE##_f8f6f4(X, Y, acc, F8Format<MmaClass::CX>::value,         \
                                                                    F8Format<MmaClass::CY>::value, SelX,              \
                                                                    static_cast<int>(scaleX), SelY,                   \
                                                                    static_cast<int>(scaleY));                        \
        }                                                                                                             \
    };
#define ROCWMMA_MFMA_SCALED_PAIR(CX, CY)       \
    ROCWMMA_MFMA_SCALED(CX, CY, 16, 16x16x128) \
    ROCWMMA_MFMA_SCALED(CX, CY, 32, 32x32x64)
        ROCWMMA_MFMA_SCALED_PAIR(F8, F8)
        ROCWMMA_MFMA_SCALED_PAIR(F8, BF8)
        ROCWMMA_MFMA_SCALED_PAIR(BF8, F8)
        ROCWMMA_MFMA_SCALED_PAIR(BF8, BF8)
#undef ROCWMMA_MFMA_SCALED_PAIR
#undef ROCWMMA_MFMA_SCALED
#endif // ROCWMMA_ARCH_GFX950

#undef ROCWMMA_MFMA_ENTRY

    } // namespace detail
} // namespace rocwmma

#endif // ROCWMMA_MFMA_GFX950_HPP
