// Shared host-side plumbing of the C ABI: status codes, error text, dtype helpers.
#ifndef R355_COMMON_HPP
#define R355_COMMON_HPP

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include <hip/hip_runtime.h>

#include "../../include/r355_wmma.h"

namespace r355
{
    // Records a formatted message for r355_last_error() and returns `code`.
    int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

    inline uint32_t dtypeBytes(int32_t t)
    {
        switch(t)
        {
        case R355_F16:
        case R355_BF16: return 2;
        case R355_E4M3:
        case R355_E5M2:
        case R355_I8: return 1;
        case R355_F32:
        case R355_I32: return 4;
        case R355_F64: return 8;
        default: return 0;
        }
    }

    inline bool aligned(const void* p, size_t bytes)
    {
        return (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
    }

    // The thread's pending HIP error belongs to whoever caused it: an error the caller has not fetched yet (its own
    // failed call, a probing call of another library) must still be there after a call into this library, as it is
    // after the reference's plain kernel launch.  So an entry point only looks at it (beginCall), and checkLaunch
    // reports - and then fetches, since the status code carries it - an error that was not pending at entry.  (A launch
    // failure with the very code that was already pending cannot be told apart and goes unreported.)
    inline hipError_t& pendingAtEntry()
    {
        thread_local hipError_t pending = hipSuccess;
        return pending;
    }

    inline void beginCall()
    {
        pendingAtEntry() = hipPeekAtLastError();
    }

    inline int checkLaunch(const char* what)
    {
        const hipError_t e = hipPeekAtLastError();
        if(e != hipSuccess && e != pendingAtEntry())
        {
            (void)hipGetLastError();
            return fail(R355_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
        }
        return R355_OK;
    }

    // CUs of the current device; where the query fails (no device: plan queries on a build host) MI355X's 256
    inline uint32_t computeUnits()
    {
        static const uint32_t cus = [] {
            int dev = 0, n = 0;
            if(hipGetDevice(&dev) != hipSuccess
               || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            {
                (void)hipGetLastError();
                return 256u;
            }
            return static_cast<uint32_t>(n);
        }();
        return cus;
    }

    // Kernel families (defined in their own translation units)
    int gemmSimpleCheck(const r355_gemm_args& g, r355_gemm_plan* plan);
    int gemmSimpleLaunch(const r355_gemm_args& g, hipStream_t stream);
    int gemmTiledCheck(const r355_gemm_args& g, r355_gemm_plan* plan);
    int gemmTiledLaunch(const r355_gemm_args& g, hipStream_t stream);
    int gemmSparseCheck(const r355_gemm_args& g, r355_gemm_plan* plan);
    int gemmSparseLaunch(const r355_gemm_args& g, hipStream_t stream);
    // DLRM shapes beyond the specialised kernels (dlrm_general.hip): m, k multiples of 16
    int dlrmGeneralFwd(int32_t dtype, const void* in, void* out, uint32_t m, uint32_t k, uint32_t batch, hipStream_t stream);
    int dlrmGeneralBwd(int32_t dtype, const void* in, const void* upstream, void* mlpGrad, void* inGrad, uint32_t m, uint32_t k,
                       uint32_t batch, hipStream_t stream);
} // namespace r355

#endif // R355_COMMON_HPP
