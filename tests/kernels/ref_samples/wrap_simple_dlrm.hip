// Runs the forward device kernel of the reference's samples/simple_dlrm.cpp, compiled unchanged
// against this library's headers, with the sample's launch geometry (samples/simple_dlrm.cpp:503-533).
#define main sample_main_unused
#include "simple_dlrm.cpp"
#undef main

extern "C" int ref_simple_dlrm_fwd(const void* in, void* out, float* acc, uint32_t m, uint32_t k, uint32_t b)
{
    auto gridDim  = dim3(rocwmma::ceilDiv(m, TILE_DIM * T_BLOCK_X / 64u), rocwmma::ceilDiv(m, TILE_DIM), b);
    auto blockDim = dim3(T_BLOCK_X);
    hipLaunchKernelGGL(dlrmDotFwd, gridDim, blockDim, 0, 0, static_cast<const float16_t*>(in), static_cast<float16_t*>(out),
                       acc, m, k, b, m * k, ((m * (m - 1)) / 2) + k, m * m);
    return hipDeviceSynchronize() == hipSuccess ? 0 : -1;
}
