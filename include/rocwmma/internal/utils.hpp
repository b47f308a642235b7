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

#endif // ROCWMMA_UTILS_HPP
