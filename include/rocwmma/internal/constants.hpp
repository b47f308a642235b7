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

        static constexpr uint32_t AMDGCN_WAVE_SIZE_64   = 64u;
        static constexpr uint32_t AMDGCN_WAVE_SIZE_32   = 32u;
        static constexpr uint32_t AMDGCN_WAVE_SIZE_NONE = 0u;

        static constexpr uint32_t AMDGCN_CURRENT_ARCH_ID
            = ROCWMMA_ARCH_GFX950 ? AMDGCN_ARCH_ID_GFX950 : AMDGCN_ARCH_ID_NONE;

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
