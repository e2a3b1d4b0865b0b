// Hardware constants of the one supported target (gfx950 / MI355X).
// Public names follow library/include/rocwmma/internal/constants.hpp:33-101.
#ifndef ROCWMMA_CONSTANTS_HPP
#define ROCWMMA_CONSTANTS_HPP

#include "types.hpp"

namespace rocwmma
{
    struct Constants
    {
        static constexpr uint32_t AMDGCN_ARCH_ID_GFX950 = 0x950;
        static constexpr uint32_t AMDGCN_ARCH_ID_NONE   = 0x0;
        // Identifiers of the targets the reference knows (constants.hpp:39-49).  They exist so that
        // code comparing AMDGCN_CURRENT_ARCH_ID against them still compiles; none of them is ever
        // the current architecture here.
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

        // Code written before gfx950 existed often gates its wave64 matrix-core branch on one of the
        // gfx90a / gfx94x ids above.  Compiling it with -DROCWMMA_REPORT_ARCH_ID=0x942 makes the device
        // pass report that id instead, so such gates pick the branch this hardware can run; nothing else
        // in the library depends on the value.
#if ROCWMMA_ARCH_GFX950 && defined(ROCWMMA_REPORT_ARCH_ID)
        static constexpr uint32_t AMDGCN_CURRENT_ARCH_ID = ROCWMMA_REPORT_ARCH_ID;
#elif ROCWMMA_ARCH_GFX950
        static constexpr uint32_t AMDGCN_CURRENT_ARCH_ID = AMDGCN_ARCH_ID_GFX950;
#else
        static constexpr uint32_t AMDGCN_CURRENT_ARCH_ID = AMDGCN_ARCH_ID_NONE;
#endif
        // Host code sees the device's wave size too: there is only one.
        static constexpr uint32_t AMDGCN_WAVE_SIZE = AMDGCN_WAVE_SIZE_64;

        static constexpr uint32_t AMDGCN_REGISTER_ELEMENT_SIZE_BYTES = 4u;
        static constexpr uint32_t AMDGCN_REGISTER_SIZE_BYTES
            = AMDGCN_REGISTER_ELEMENT_SIZE_BYTES * AMDGCN_WAVE_SIZE;

        static constexpr uint32_t AMDGCN_LDS_MAX_SIZE_BYTES    = 163840u; // 160 KiB per CU
        static constexpr uint32_t AMDGCN_CACHE_LINE_SIZE_BYTES = 128u;
        static constexpr uint32_t AMDGCN_DWORD_SIZE_BYTES      = 4u;
    };
} // namespace rocwmma

#endif // ROCWMMA_CONSTANTS_HPP
