// Build configuration: one target (gfx950, wave64), one compiler (ROCm clang).
//
// Replaces the per-architecture macro forest of the reference
// (library/include/rocwmma/internal/config.hpp:48-221) with the single case this
// library is written for.  ROCWMMA_ARCH_GFX9 is true in the device pass so that
// kernels written against the reference pick their wave64 parameter sets
// (samples/perf_hgemm.cpp:254-258).
#ifndef ROCWMMA_CONFIG_HPP
#define ROCWMMA_CONFIG_HPP

#if defined(__HIP_DEVICE_COMPILE__) && __HIP_DEVICE_COMPILE__
#define ROCWMMA_DEVICE_COMPILE 1
#else
#define ROCWMMA_DEVICE_COMPILE 0
#endif

#if ROCWMMA_DEVICE_COMPILE
#if !defined(__gfx950__)
#error "this library targets gfx950 (MI355X) only: compile with --offload-arch=gfx950"
#endif
#define ROCWMMA_ARCH_GFX950 1
#define ROCWMMA_ARCH_GFX9 1
#define ROCWMMA_ARCH_HOST 0
#else
#define ROCWMMA_ARCH_GFX950 0
#define ROCWMMA_ARCH_GFX9 0
#define ROCWMMA_ARCH_HOST 1
#endif

#define ROCWMMA_ARCH_GFX11 0
#define ROCWMMA_ARCH_GFX12 0
#define ROCWMMA_WAVE64_MODE ROCWMMA_ARCH_GFX9
#define ROCWMMA_WAVE32_MODE 0
#define ROCWMMA_BLOCK_DIM_16_SUPPORTED 1
#define ROCWMMA_BLOCK_DIM_32_SUPPORTED 1

#define ROCWMMA_DEVICE __device__
#define ROCWMMA_HOST __host__
#define ROCWMMA_HOST_DEVICE ROCWMMA_HOST ROCWMMA_DEVICE
#define ROCWMMA_KERNEL __global__

#endif // ROCWMMA_CONFIG_HPP
