// Wave-level flow control primitives with the names existing kernels use
// (reference: library/include/rocwmma/internal/flow_control.hpp:100-118): each is a type with a
// static exec().
//
//   Barrier              workgroup barrier instruction alone (no memory ordering implied)
//   SchedBarrier<mask>   compiler scheduling fence (mask as for __builtin_amdgcn_sched_barrier)
//   SetPrio<p>           wave priority 0..3 for the instruction arbiter
//   Waitcnt<vm, lgkm>    wait until at most `vm` vector-memory and `lgkm` LDS / scalar operations
//                        of this wave are outstanding;  WaitVmcnt<vm> = Waitcnt<vm, 0> and
//                        WaitLgkmcnt<lgkm> = Waitcnt<0, lgkm>, as in the reference
#ifndef ROCWMMA_FLOW_CONTROL_HPP
#define ROCWMMA_FLOW_CONTROL_HPP

#include "config.hpp"
#include <cstdint>

namespace rocwmma
{
    struct Barrier
    {
        ROCWMMA_DEVICE static inline void exec()
        {
            __builtin_amdgcn_s_barrier();
        }
    };

    template <int32_t mask>
    struct SchedBarrier
    {
        ROCWMMA_DEVICE static inline void exec()
        {
            __builtin_amdgcn_sched_barrier(mask);
        }
    };

    template <int32_t priority>
    struct SetPrio
    {
        static_assert(priority >= 0 && priority <= 3, "wave priority is a 2-bit field");
        ROCWMMA_DEVICE static inline void exec()
        {
            __builtin_amdgcn_s_setprio(static_cast<short>(priority));
        }
    };

    template <int32_t vmcnt, int32_t lgkmcnt>
    struct Waitcnt
    {
        static_assert(vmcnt >= 0 && vmcnt < 64, "vmcnt is a 6-bit field");
        static_assert(lgkmcnt >= 0 && lgkmcnt < 16, "lgkmcnt is a 4-bit field");
        // gfx9 encoding of s_waitcnt: vmcnt[3:0] in bits 3:0, vmcnt[5:4] in bits 15:14,
        // lgkmcnt in bits 11:8; expcnt (bits 6:4) left at its maximum = not waited for
        static constexpr int32_t encoded
            = (vmcnt & 0xF) | ((vmcnt & 0x30) << 10) | (0x7 << 4) | ((lgkmcnt & 0xF) << 8);
        ROCWMMA_DEVICE static inline void exec()
        {
            __builtin_amdgcn_s_waitcnt(encoded);
        }
    };

    template <int32_t vmcnt>
    using WaitVmcnt = Waitcnt<vmcnt, 0>;

    template <int32_t lgkmcnt>
    using WaitLgkmcnt = Waitcnt<0, lgkmcnt>;

} // namespace rocwmma

#endif // ROCWMMA_FLOW_CONTROL_HPP
