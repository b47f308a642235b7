// Build configuration of the gfx950-native wave-level MMA library.
//
// Public macro names follow rocWMMA's (reference: library/include/rocwmma/internal/config.hpp:48-177)
// so that kernels written against it compile unchanged.  This library targets exactly one
// device ISA: gfx950 (CDNA4, wave64).  Any other device target is a compile error.
#ifndef ROCWMMA_CONFIG_HPP
#define ROCWMMA_CONFIG_HPP

#include <hip/hip_runtime.h>

// Identifies this implementation; translation units can static_assert on it to make sure
// the toolchain's own rocWMMA copy was not picked up by include order.
#define ROCWMMA_AMD_GFX950_NATIVE 1
#define ROCWMMA_VERSION_MAJOR 1
#define ROCWMMA_VERSION_MINOR 7
#define ROCWMMA_VERSION_PATCH 0

#if defined(__HIP_DEVICE_COMPILE__) && __HIP_DEVICE_COMPILE__
#define ROCWMMA_DEVICE_COMPILE 1
#else
#define ROCWMMA_DEVICE_COMPILE 0
#endif

#if ROCWMMA_DEVICE_COMPILE
#if defined(__gfx950__)
#define ROCWMMA_ARCH_GFX950 1
#define ROCWMMA_ARCH_HOST 0
#else
#error "this rocWMMA implementation is gfx950 (MI350X/MI355X) only: build with --offload-arch=gfx950"
#endif
#else
#define ROCWMMA_ARCH_GFX950 0
#define ROCWMMA_ARCH_HOST 1
#endif

// Family macros existing kernels test.  gfx950 is a wave64 gfx9 part with 16- and 32-wide blocks.
#define ROCWMMA_ARCH_GFX9 ROCWMMA_ARCH_GFX950
#define ROCWMMA_ARCH_GFX94X 0
#define ROCWMMA_ARCH_GFX11 0
#define ROCWMMA_ARCH_GFX12 0
#define ROCWMMA_ARCH_GFX908 0
#define ROCWMMA_ARCH_GFX90A 0
#define ROCWMMA_ARCH_GFX940 0
#define ROCWMMA_ARCH_GFX941 0
#define ROCWMMA_ARCH_GFX942 0
#define ROCWMMA_ARCH_GFX1100 0
#define ROCWMMA_ARCH_GFX1101 0
#define ROCWMMA_ARCH_GFX1102 0
#define ROCWMMA_ARCH_GFX1200 0
#define ROCWMMA_ARCH_GFX1201 0
#define ROCWMMA_WAVE64_MODE ROCWMMA_ARCH_GFX950
#define ROCWMMA_WAVE32_MODE 0
#define ROCWMMA_BLOCK_DIM_16_SUPPORTED 1
#define ROCWMMA_BLOCK_DIM_32_SUPPORTED 1

#if defined(HIP_NO_HALF)
#define ROCWMMA_NO_HALF 1
#else
#define ROCWMMA_NO_HALF 0
#endif

#define ROCWMMA_DEVICE __device__
#define ROCWMMA_HOST __host__
#define ROCWMMA_HOST_DEVICE __host__ __device__
#define ROCWMMA_KERNEL __global__

#define ROCWMMA_INLINE __attribute__((always_inline)) inline

#endif // ROCWMMA_CONFIG_HPP
