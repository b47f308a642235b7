// Hardware constants of the one supported device (gfx950 / CDNA4).
// Member names follow rocWMMA (reference: library/include/rocwmma/internal/constants.hpp:33-103).
#ifndef ROCWMMA_CONSTANTS_HPP
#define ROCWMMA_CONSTANTS_HPP

#include "config.hpp"
#include <cstdint>

namespace rocwmma
{
    struct Constants
    {
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX950 = 0x950;
        static constexpr uint32_t AMDGCN_ARCH_ID_NONE   = 0x0;
        // identifiers of the devices this library does not target: existing code compares
        // AMDGCN_CURRENT_ARCH_ID against them (never equal here)
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX908  = 0x908;
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX90A  = 0x90A;
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX940  = 0x940;
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX941  = 0x941;
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX942  = 0x942;
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX1100 = 0x1100;
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX1101 = 0x1101;
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX1102 = 0x1102;
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX1200 = 0x1200;
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX1201 = 0x1201;

        static constexpr uint32_t AMDGCN_WAVE_SIZE_64   = 64u;
        static constexpr uint32_t AMDGCN_WAVE_SIZE_32   = 32u;
        static constexpr uint32_t AMDGCN_WAVE_SIZE_NONE = 0u;

        // Code written before gfx950 existed gates its kernels on the identifiers it knows
        // (e.g. the reference's test kernels: test/unit/unit_test_traits.hpp:70-90).  Defining
        // ROCWMMA_AMD_REPORT_ARCH_ID (say to 0x942) makes the device pass report that identifier.
#if defined(ROCWMMA_AMD_REPORT_ARCH_ID)
        static constexpr uint32_t AMDGCN_CURRENT_ARCH_ID
            = ROCWMMA_ARCH_GFX950 ? uint32_t{ROCWMMA_AMD_REPORT_ARCH_ID} : AMDGCN_ARCH_ID_NONE;
#else
        static constexpr uint32_t AMDGCN_CURRENT_ARCH_ID
            = ROCWMMA_ARCH_GFX950 ? AMDGCN_ARCH_ID_GFX950 : AMDGCN_ARCH_ID_NONE;
#endif

        // wave64 on the device; the host pass uses the same value so shared constexpr code agrees
        static constexpr uint32_t AMDGCN_WAVE_SIZE = AMDGCN_WAVE_SIZE_64;

        static constexpr uint32_t AMDGCN_REGISTER_ELEMENT_SIZE_BYTES = 4u;
        static constexpr uint32_t AMDGCN_REGISTER_SIZE_BYTES
            = AMDGCN_REGISTER_ELEMENT_SIZE_BYTES * AMDGCN_WAVE_SIZE;

        // gfx950: 160 KiB of LDS per CU, 64 banks of 4 bytes, 128-byte L2 lines
        static constexpr uint32_t AMDGCN_LDS_MAX_SIZE_BYTES    = 163840u;
        static constexpr uint32_t AMDGCN_LDS_BANK_COUNT        = 64u;
        static constexpr uint32_t AMDGCN_CACHE_LINE_SIZE_BYTES = 128u;
        static constexpr uint32_t AMDGCN_DWORD_SIZE_BYTES      = 4u;
    };
} // namespace rocwmma

#endif // ROCWMMA_CONSTANTS_HPP
