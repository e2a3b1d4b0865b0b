// Runs the reference's io_traits unit-test kernel (test/unit/io_traits_test/device/io_traits.hpp:34-101),
// compiled unchanged against this library's headers: it checks PackTraits<DataT> and
// IOTraits<BlockDim, BlockK, DataT, VectorWidth> against closed forms on the device and writes
// SUCCESS_VALUE (0) or ERROR_VALUE (7) to out[0].  Cases sample the suite's parameter lists
// (test/unit/io_traits_test/test/io_traits_{16,32,64,128,256}.cpp).
#include <iostream>

#include <hip/hip_runtime.h>

#include <rocwmma/rocwmma.hpp>

#include "test/common.hpp" // SUCCESS_VALUE / ERROR_VALUE (test/common.hpp:75-76)
#include "unit/io_traits_test/device/io_traits.hpp"

#define IO_CASES(X)                  \
    X(0, int8_t, 16, 16, 4)          \
    X(1, int8_t, 32, 64, 4)          \
    X(2, int8_t, 128, 32, 16)        \
    X(3, int8_t, 256, 256, 16)       \
    X(4, float16_t, 16, 16, 1)       \
    X(5, float16_t, 16, 64, 4)       \
    X(6, float16_t, 32, 8, 2)        \
    X(7, float16_t, 64, 64, 4)       \
    X(8, float16_t, 128, 16, 8)      \
    X(9, float16_t, 256, 32, 16)     \
    X(10, bfloat16_t, 32, 32, 4)     \
    X(11, bfloat16_t, 128, 128, 8)   \
    X(12, float32_t, 16, 16, 2)      \
    X(13, float32_t, 32, 128, 4)     \
    X(14, float32_t, 64, 8, 1)       \
    X(15, float32_t, 256, 64, 4)     \
    X(16, float64_t, 16, 16, 1)      \
    X(17, float64_t, 64, 32, 2)      \
    X(18, float64_t, 128, 8, 4)      \
    X(19, int32_t, 32, 32, 4)        \
    X(20, float8_t, 16, 32, 4)       \
    X(21, float8_t, 64, 64, 16)

// Returns the value the kernel wrote (0 = all identities hold), -1 for an unknown case, -2 for a HIP error.
extern "C" int ref_test_io_traits(int id)
{
    using namespace rocwmma;
    double* out = nullptr; // wide enough for every element type
    if(hipMalloc(&out, sizeof(double)) != hipSuccess)
        return -2;
    int result = -1;
    switch(id)
    {
#define X(ID, T, DIM, K, VW)                                                                                       \
    case ID: {                                                                                                     \
        hipLaunchKernelGGL((ioTraitsTest<T, DIM, K, VW>), dim3(1), dim3(64), 0, 0, 0u, 0u,                          \
                           static_cast<T const*>(nullptr), reinterpret_cast<T*>(out), 0u, static_cast<T>(64),       \
                           static_cast<T>(0));                                                                     \
        T host;                                                                                                    \
        if(hipMemcpy(&host, out, sizeof(T), hipMemcpyDeviceToHost) != hipSuccess)                                   \
            result = -2;                                                                                           \
        else                                                                                                       \
            result = static_cast<int>(static_cast<float>(host));                                                   \
        break;                                                                                                     \
    }
        IO_CASES(X)
#undef X
    default: break;
    }
    (void)hipFree(out);
    return result;
}

extern "C" int ref_test_io_traits_cases()
{
    return 22;
}
