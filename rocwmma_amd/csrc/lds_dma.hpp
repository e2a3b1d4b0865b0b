// Direct global -> LDS loads under explicit wait control, shared by the macro-tile kernels.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace r355
{
    using dma_i32x4 = int __attribute__((ext_vector_type(4)));

    // One 16-byte-per-lane direct load: the memory pipeline writes lane l's data at LDS byte
    // ldsAddr + 16 l.  rsrc is a raw buffer descriptor (wave-uniform), laneOffset the lane's byte
    // offset, uniformOffset a scalar byte offset.  Inline assembly on purpose: for the builtin the
    // compiler cannot tell which LDS buffer a later ds_read depends on and waits for vmcnt(0) every
    // time, which serialises exactly the loads that are meant to stay in flight.  Issued this way the
    // only vmcnt waits are the ones the kernels write themselves (waitVmcnt).  The "memory" clobber
    // keeps LDS reads from moving across the load.
    __device__ inline void loadToLds(dma_i32x4 rsrc, uint32_t laneOffset, uint32_t uniformOffset, uint32_t ldsAddr)
    {
        asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
                     :
                     : "v"(laneOffset), "s"(rsrc), "s"(uniformOffset), "s"(ldsAddr)
                     : "memory");
    }

    // raw buffer descriptor over [addr, addr + 2 GiB): 32-bit data format, no swizzle, no stride
    // (addr must be wave-uniform; the readfirstlane calls only tell the compiler so and fold away when it
    // already knows)
    __device__ inline dma_i32x4 rawBuffer(uint64_t addr)
    {
        const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr));
        const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr >> 32));
        return dma_i32x4{static_cast<int>(lo), static_cast<int>(hi & 0xFFFFu), 0x7FFFFFFF, 0x00020000};
    }

    // a wave-uniform address as an integer the compiler can see is uniform
    __device__ inline uint64_t uniformAddress(const void* ptr)
    {
        const uint64_t v  = reinterpret_cast<uint64_t>(ptr);
        const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
        const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
        return (static_cast<uint64_t>(hi) << 32) | lo;
    }

    // wait until at most N vector-memory operations of this wave are outstanding
    template <uint32_t N>
    __device__ inline void waitVmcnt()
    {
        // vmcnt is split over bits [3:0] and [15:14]; expcnt and lgkmcnt stay at their maxima
        __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15u) | ((N >> 4) << 14));
    }

    // barrier that orders LDS traffic only: __syncthreads() also fences global memory, which drains
    // the direct loads
    __device__ inline void ldsBarrier()
    {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    }
} // namespace r355
