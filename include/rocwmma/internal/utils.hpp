// Small helpers existing kernels take from <rocwmma/internal/utils.hpp>: coordinate arithmetic
// (Coord2d, make_coord2d, get<I>), ceilDiv, Log2 and friends live in coord.hpp here
// (reference: library/include/rocwmma/internal/utils.hpp:56-152).  This header keeps the
// reference's include path working and keeps the toolchain's own rocWMMA copy from being
// picked up instead.
#ifndef ROCWMMA_UTILS_HPP
#define ROCWMMA_UTILS_HPP

#include "config.hpp"
#include "constants.hpp"
#include "coord.hpp"
#include "types.hpp"

namespace rocwmma
{
    struct row_major;
    struct col_major;
    struct matrix_a;
    struct matrix_b;
    struct accumulator;

    // Short printable name of an element type, layout tag or matrix tag, for logs and test
    // names (reference: library/include/rocwmma/internal/utils.hpp:203-330).  The primary
    // template is only declared: callers add specializations for their own tag types.
    template <typename T>
    constexpr const char* dataTypeToString();

#define ROCWMMA_AMD_TYPE_NAME(TYPE, NAME)               \
    template <>                                         \
    constexpr const char* dataTypeToString<TYPE>()      \
    {                                                   \
        return NAME;                                    \
    }
    ROCWMMA_AMD_TYPE_NAME(float8_t, "f8")
    ROCWMMA_AMD_TYPE_NAME(bfloat8_t, "bf8")
    ROCWMMA_AMD_TYPE_NAME(float8_fnuz_t, "f8(fnuz)")
    ROCWMMA_AMD_TYPE_NAME(bfloat8_fnuz_t, "bf8(fnuz)")
    ROCWMMA_AMD_TYPE_NAME(float16_t, "f16")
#if !ROCWMMA_NO_HALF
    ROCWMMA_AMD_TYPE_NAME(hfloat16_t, "h16")
#endif
    ROCWMMA_AMD_TYPE_NAME(bfloat16_t, "bf16")
    ROCWMMA_AMD_TYPE_NAME(float32_t, "f32")
    ROCWMMA_AMD_TYPE_NAME(float64_t, "f64")
    ROCWMMA_AMD_TYPE_NAME(int8_t, "i8")
    ROCWMMA_AMD_TYPE_NAME(uint8_t, "u8")
    ROCWMMA_AMD_TYPE_NAME(int16_t, "i16")
    ROCWMMA_AMD_TYPE_NAME(uint16_t, "u16")
    ROCWMMA_AMD_TYPE_NAME(int32_t, "i32")
    ROCWMMA_AMD_TYPE_NAME(uint32_t, "u32")
    ROCWMMA_AMD_TYPE_NAME(int64_t, "i64")
    ROCWMMA_AMD_TYPE_NAME(uint64_t, "u64")
    ROCWMMA_AMD_TYPE_NAME(xfloat32_t, "xf32")
    ROCWMMA_AMD_TYPE_NAME(row_major, "T")
    ROCWMMA_AMD_TYPE_NAME(col_major, "N")
    ROCWMMA_AMD_TYPE_NAME(matrix_a, "matrix_a")
    ROCWMMA_AMD_TYPE_NAME(matrix_b, "matrix_b")
    ROCWMMA_AMD_TYPE_NAME(accumulator, "accumulator")
#undef ROCWMMA_AMD_TYPE_NAME
} // namespace rocwmma

#endif // ROCWMMA_UTILS_HPP
