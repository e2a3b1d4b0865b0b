// Runs the device kernels of the reference's DLRM test suite (test/dlrm/device/dlrm_dot_fwd.hpp,
// dlrm_dot_bwd.hpp and their LDS-staged twins dlrm_dot_fwd_lds.hpp / dlrm_dot_bwd_lds.hpp with the
// register-file LDS mapping, dynamic LDS size from test/dlrm/detail/dlrm_dot_lds.hpp:48-54), compiled unchanged against this library's headers, with the suite's launch
// geometry (test/dlrm/dlrm_kernel_base_impl.hpp:78-104, 300-392): 128-thread workgroups, forward grid
// (m / (T * 2), m / T, b), backward = trilReconstruct then dlrmDotBwd on grid (m / (T * 2), k / T, b).
#include <hip/hip_runtime.h>

#include <rocwmma/rocwmma.hpp>

#include "device/dlrm_dot_bwd.hpp"
#include "device/dlrm_dot_bwd_lds.hpp"
#include "device/dlrm_dot_fwd.hpp"
#include "device/dlrm_dot_fwd_lds.hpp"

namespace
{
    constexpr uint32_t TBLOCK = 128, WAVE = 64;

    template <typename T, uint32_t TILE>
    int fwd(const void* in, void* out, float* acc, uint32_t m, uint32_t k, uint32_t b)
    {
        dim3 grid(rocwmma::ceilDiv(m, TILE * TBLOCK / WAVE), rocwmma::ceilDiv(m, TILE), b);
        hipLaunchKernelGGL((rocwmma::dlrmDotFwd<T, TILE>), grid, dim3(TBLOCK), 0, 0, static_cast<const T*>(in),
                           static_cast<T*>(out), acc, m, k, b, m * k, ((m * (m - 1)) / 2) + k, m * m);
        return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
    }

    template <typename T, uint32_t TILE>
    int bwd(const void* in, const void* up, void* grad, void* mlpGrad, void* acc, uint32_t m, uint32_t k, uint32_t b)
    {
        const uint32_t upOff = ((m * (m - 1)) / 2) + k;
        dim3 trilGrid(rocwmma::ceilDiv(m * m, TBLOCK), 1, b);
        hipLaunchKernelGGL((rocwmma::trilReconstruct<T>), trilGrid, dim3(TBLOCK), 0, 0, static_cast<const T*>(up),
                           static_cast<T*>(acc), m, k, b, upOff, m * m);
        if(hipDeviceSynchronize() != hipSuccess)
            return -1;
        dim3 grid(rocwmma::ceilDiv(m, TILE * TBLOCK / WAVE), rocwmma::ceilDiv(k, TILE), b);
        hipLaunchKernelGGL((rocwmma::dlrmDotBwd<T, TILE>), grid, dim3(TBLOCK), 0, 0, static_cast<const T*>(in),
                           static_cast<const T*>(up), static_cast<T*>(grad), static_cast<T*>(mlpGrad), static_cast<T*>(acc),
                           m, k, b, m * k, upOff, m * m);
        return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
    }
    template <typename T, uint32_t TILE>
    uint32_t ldsBytes()
    {
        return 2u * sizeof(T) * ((TBLOCK / WAVE) + 1u) * (TILE * TILE);
    }

    template <typename T, uint32_t TILE>
    int fwdLds(const void* in, void* out, float* acc, uint32_t m, uint32_t k, uint32_t b)
    {
        dim3 grid(rocwmma::ceilDiv(m, TILE * TBLOCK / WAVE), rocwmma::ceilDiv(m, TILE), b);
        const uint32_t lds = ldsBytes<T, TILE>();
        hipLaunchKernelGGL((rocwmma::dlrmDotFwdLds<T, TILE, rocwmma::LdsRF>), grid, dim3(TBLOCK), lds, 0,
                           static_cast<const T*>(in), static_cast<T*>(out), acc, m, k, b, m * k, ((m * (m - 1)) / 2) + k,
                           m * m);
        return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
    }

    template <typename T, uint32_t TILE>
    int bwdLds(const void* in, const void* up, void* grad, void* mlpGrad, void* acc, uint32_t m, uint32_t k, uint32_t b)
    {
        const uint32_t upOff = ((m * (m - 1)) / 2) + k;
        dim3 trilGrid(rocwmma::ceilDiv(m * m, TBLOCK), 1, b);
        hipLaunchKernelGGL((rocwmma::trilReconstructLds<T>), trilGrid, dim3(TBLOCK), 0, 0, static_cast<const T*>(up),
                           static_cast<T*>(acc), m, k, b, upOff, m * m);
        if(hipDeviceSynchronize() != hipSuccess)
            return -1;
        dim3 grid(rocwmma::ceilDiv(m, TILE * TBLOCK / WAVE), rocwmma::ceilDiv(k, TILE), b);
        const uint32_t lds = ldsBytes<T, TILE>();
        hipLaunchKernelGGL((rocwmma::dlrmDotBwdLds<T, TILE, rocwmma::LdsRF>), grid, dim3(TBLOCK), lds, 0,
                           static_cast<const T*>(in), static_cast<const T*>(up), static_cast<T*>(grad),
                           static_cast<T*>(mlpGrad), static_cast<T*>(acc), m, k, b, m * k, upOff, m * m);
        return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
    }
} // namespace

// LDS-staged twins, f16 only here (tile 16 or 32)
extern "C" int ref_test_dlrm_fwd_lds(uint32_t tile, const void* in, void* out, float* acc, uint32_t m, uint32_t k,
                                     uint32_t b)
{
    using namespace rocwmma;
    return tile == 32 ? fwdLds<float16_t, 32>(in, out, acc, m, k, b) : fwdLds<float16_t, 16>(in, out, acc, m, k, b);
}

extern "C" int ref_test_dlrm_bwd_lds(uint32_t tile, const void* in, const void* up, void* grad, void* mlpGrad, void* acc,
                                     uint32_t m, uint32_t k, uint32_t b)
{
    using namespace rocwmma;
    return tile == 32 ? bwdLds<float16_t, 32>(in, up, grad, mlpGrad, acc, m, k, b)
                      : bwdLds<float16_t, 16>(in, up, grad, mlpGrad, acc, m, k, b);
}

// dtype: 0 = float16_t, 4 = float32_t; tile: 16 or 32
extern "C" int ref_test_dlrm_fwd(int dtype, uint32_t tile, const void* in, void* out, float* acc, uint32_t m, uint32_t k,
                                 uint32_t b)
{
    using namespace rocwmma;
    if(dtype == 0)
        return tile == 32 ? fwd<float16_t, 32>(in, out, acc, m, k, b) : fwd<float16_t, 16>(in, out, acc, m, k, b);
    return tile == 32 ? fwd<float32_t, 32>(in, out, acc, m, k, b) : fwd<float32_t, 16>(in, out, acc, m, k, b);
}

extern "C" int ref_test_dlrm_bwd(int dtype, uint32_t tile, const void* in, const void* up, void* grad, void* mlpGrad,
                                 void* acc, uint32_t m, uint32_t k, uint32_t b)
{
    using namespace rocwmma;
    if(dtype == 0)
        return tile == 32 ? bwd<float16_t, 32>(in, up, grad, mlpGrad, acc, m, k, b)
                          : bwd<float16_t, 16>(in, up, grad, mlpGrad, acc, m, k, b);
    return tile == 32 ? bwd<float32_t, 32>(in, up, grad, mlpGrad, acc, m, k, b)
                      : bwd<float32_t, 16>(in, up, grad, mlpGrad, acc, m, k, b);
}
