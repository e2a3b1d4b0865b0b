// Wave-level flow control helpers kernels built on the fragment API reach for when they tune their
// own schedules: workgroup barrier, scheduling fence, wave priority and explicit counter waits.
// Same names and template parameters as library/include/rocwmma/internal/flow_control.hpp:30-120.
#ifndef ROCWMMA_FLOW_CONTROL_HPP
#define ROCWMMA_FLOW_CONTROL_HPP

#include "config.hpp"
#include "types.hpp"

namespace rocwmma
{
    // s_barrier: every wave of the workgroup arrives before any leaves.
    struct Barrier
    {
        ROCWMMA_DEVICE static inline void exec()
        {
#if ROCWMMA_DEVICE_COMPILE
            __builtin_amdgcn_s_barrier();
#endif
        }
    };

    // Compiler scheduling fence: `mask` selects the instruction classes that may still cross it
    // (0 = nothing moves across).
    template <int32_t mask>
    struct SchedBarrier
    {
        ROCWMMA_DEVICE static inline void exec()
        {
#if ROCWMMA_DEVICE_COMPILE
            __builtin_amdgcn_sched_barrier(mask);
#endif
        }
    };

    // s_setprio: issue priority of this wave among the waves of its SIMD, 0 (default) to 3.
    template <int32_t priority>
    struct SetPrio
    {
        static_assert(priority >= 0 && priority <= 3, "wave priority is 0..3");
        ROCWMMA_DEVICE static inline void exec()
        {
#if ROCWMMA_DEVICE_COMPILE
            __builtin_amdgcn_s_setprio(static_cast<short>(priority));
#endif
        }
    };

    // s_waitcnt on gfx9: vmcnt is 6 bits split over simm16[3:0] and [15:14], lgkmcnt 4 bits at [11:8],
    // expcnt 3 bits at [6:4] (waited down to 0 here, as the reference's encoding does).
    template <int32_t vmcnt, int32_t lgkmcnt>
    struct Waitcnt
    {
        static_assert(vmcnt >= 0 && vmcnt < 64, "vmcnt has 6 bits");
        static_assert(lgkmcnt >= 0 && lgkmcnt < 16, "lgkmcnt has 4 bits");
        ROCWMMA_DEVICE static inline void exec()
        {
#if ROCWMMA_DEVICE_COMPILE
            __builtin_amdgcn_s_waitcnt((vmcnt & 0xF) | ((vmcnt >> 4) << 14) | (lgkmcnt << 8));
#endif
        }
    };

    // Vector-memory only / LDS-scalar-memory only forms: the other counter is waited down to 0.
    template <int32_t vmcnt>
    using WaitVmcnt = Waitcnt<vmcnt, 0>;

    template <int32_t lgkmcnt>
    using WaitLgkmcnt = Waitcnt<0, lgkmcnt>;

} // namespace rocwmma

#endif // ROCWMMA_FLOW_CONTROL_HPP
