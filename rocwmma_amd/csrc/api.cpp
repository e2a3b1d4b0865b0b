// extern "C" entry points of the library (declared in include/r355_wmma.h): argument
// validation, kernel-family selection, timing helpers, error text.
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "common.hpp"

namespace
{
    thread_local char g_lastError[512] = "";

    // Device memory of r355_gemm_noalloc: the split-K partial results of one call.  Every device the library runs on
    // holds its own copy, at its own address, until the process ends.  The name below is only a host-side handle for
    // hipGetSymbolAddress; kernels and copies take the address that call returns.
    constexpr size_t SCRATCH_BYTES = size_t{16} << 20;
    static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

    constexpr int MAX_DEVICES = 64;
    std::mutex    g_scratchLock;
    void*         g_scratchAt[MAX_DEVICES] = {};

    // address of `scratch` on the current device (looked up once per device).  The lookup may make the runtime load the
    // library's device image and back the array, which is not something to do while a stream is recording a graph: a
    // first call on a device that arrives under capture is refused (`capturing` names the stream to test, or nullptr
    // for "do the lookup": r355_get_device_info is the eager call that prepares a device).
    int scratchOfCurrentDevice(void** ptr, const hipStream_t* capturing)
    {
        int dev = 0;
        if(hipGetDevice(&dev) != hipSuccess)
            return r355::fail(R355_ERR_LAUNCH, "gemm_noalloc: no HIP device");
        if(dev < 0 || dev >= MAX_DEVICES)
            return r355::fail(R355_ERR_UNSUPPORTED, "gemm_noalloc: device ordinal %d beyond the %d the library keeps scratch for", dev,
                              MAX_DEVICES);
        std::lock_guard<std::mutex> hold(g_scratchLock);
        if(!g_scratchAt[dev])
        {
            if(capturing)
            {
                hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
                if(hipStreamIsCapturing(*capturing, &status) != hipSuccess || status != hipStreamCaptureStatusNone)
                    return r355::fail(R355_ERR_UNSUPPORTED,
                                      "gemm_noalloc: the first call on device %d looks up the library's scratch buffer, which cannot happen "
                                      "while a stream is capturing; call r355_get_device_info (or r355_gemm_noalloc once) on this device "
                                      "before the capture begins",
                                      dev);
            }
            void*            at = nullptr;
            const hipError_t e  = hipGetSymbolAddress(&at, HIP_SYMBOL(scratch));
            if(e != hipSuccess || !at)
                return r355::fail(R355_ERR_LAUNCH, "gemm_noalloc: hipGetSymbolAddress(scratch) failed on device %d: %s", dev,
                                  hipGetErrorString(e));
            g_scratchAt[dev] = at;
        }
        *ptr = g_scratchAt[dev];
        return R355_OK;
    }

    int validateCommon(const r355_gemm_args* g)
    {
        if(!g)
            return r355::fail(R355_ERR_BAD_ARG, "gemm: args is null");
        if(!g->a || !g->b || !g->d)
            return r355::fail(R355_ERR_BAD_ARG, "gemm: a, b and d must be non-null");
        if(g->beta != 0.0 && !g->c)
            return r355::fail(R355_ERR_BAD_ARG, "gemm: c is null but beta != 0");
        if(g->m == 0 || g->n == 0 || g->k == 0)
            return r355::fail(R355_ERR_BAD_ARG, "gemm: m, n, k must be non-zero");
        for(int32_t l : {g->layout_a, g->layout_b, g->layout_c, g->layout_d})
            if(l != R355_ROW_MAJOR && l != R355_COL_MAJOR)
                return r355::fail(R355_ERR_BAD_ARG, "gemm: layout must be R355_ROW_MAJOR or R355_COL_MAJOR");
        if(r355::dtypeBytes(g->in_type) == 0 || r355::dtypeBytes(g->out_type) == 0)
            return r355::fail(R355_ERR_BAD_ARG, "gemm: unknown dtype");
        const uint32_t ak = g->sparse24 ? g->k / 2 : g->k;
        const uint32_t minLda = g->layout_a == R355_ROW_MAJOR ? ak : g->m;
        const uint32_t minLdb = g->layout_b == R355_ROW_MAJOR ? g->n : g->k;
        const uint32_t minLdc = g->layout_c == R355_ROW_MAJOR ? g->n : g->m;
        const uint32_t minLdd = g->layout_d == R355_ROW_MAJOR ? g->n : g->m;
        if(g->lda < minLda || g->ldb < minLdb || g->ldd < minLdd || (g->beta != 0.0 && g->ldc < minLdc))
            return r355::fail(R355_ERR_BAD_ARG, "gemm: leading dimension smaller than the contiguous extent");
        if(g->kernel != R355_KERNEL_AUTO && g->kernel != R355_KERNEL_SIMPLE && g->kernel != R355_KERNEL_TILED
           && g->kernel != R355_KERNEL_TILED_128 && g->kernel != R355_KERNEL_TILED_128_SPLITK && g->kernel != R355_KERNEL_TILED_DEEP)
            return r355::fail(R355_ERR_BAD_ARG, "gemm: unknown kernel selector %d", g->kernel);
        return R355_OK;
    }

    // Resolve the kernel family; on success *family is the one to launch.
    int plan(const r355_gemm_args* g, r355_gemm_plan* out, int32_t* family)
    {
        int rc = validateCommon(g);
        if(rc != R355_OK)
            return rc;
        if(out)
            out->split_k = 1u, out->workspace_bytes = 0u;
        if(g->sparse24)
        {
            rc = r355::gemmSparseCheck(*g, out);
            *family = -1;
            return rc;
        }
        // AUTO takes a macro-tile kernel wherever its checks pass (down to m = n = 16 the 128 x 128 tile with
        // clamped edge loads is faster than one block per wave without LDS); the block-per-wave kernel
        // covers the rest: f32 / f64, strides or pointers off 16-byte alignment, k off a 16-byte chunk.
        const bool forced = g->kernel == R355_KERNEL_TILED || g->kernel == R355_KERNEL_TILED_128
                            || g->kernel == R355_KERNEL_TILED_128_SPLITK || g->kernel == R355_KERNEL_TILED_DEEP;
        if(forced || g->kernel == R355_KERNEL_AUTO)
        {
            rc = r355::gemmTiledCheck(*g, out);
            if(rc == R355_OK)
            {
                *family = R355_KERNEL_TILED;
                return rc;
            }
            if(forced)
                return rc;
        }
        rc = r355::gemmSimpleCheck(*g, out);
        *family = R355_KERNEL_SIMPLE;
        return rc;
    }

    int launch(const r355_gemm_args* g, int32_t family, hipStream_t stream)
    {
        if(family == -1)
            return r355::gemmSparseLaunch(*g, stream);
        if(family == R355_KERNEL_TILED)
            return r355::gemmTiledLaunch(*g, stream);
        return r355::gemmSimpleLaunch(*g, stream);
    }

    template <typename Fn>
    int timed(hipStream_t stream, int warmup, int iters, float* avgMs, Fn&& fn)
    {
        if(!avgMs || iters <= 0 || warmup < 0)
            return r355::fail(R355_ERR_BAD_ARG, "timed: need avg_ms, iters > 0, warmup >= 0");
        for(int i = 0; i < warmup; ++i)
        {
            int rc = fn();
            if(rc != R355_OK)
                return rc;
        }
        hipEvent_t start, stop;
        if(hipEventCreate(&start) != hipSuccess || hipEventCreate(&stop) != hipSuccess)
            return r355::fail(R355_ERR_LAUNCH, "timed: hipEventCreate failed");
        int rc = R355_OK;
        (void)hipEventRecord(start, stream);
        for(int i = 0; i < iters && rc == R355_OK; ++i)
            rc = fn();
        (void)hipEventRecord(stop, stream);
        hipError_t e = hipEventSynchronize(stop);
        float      ms = 0.0f;
        if(e == hipSuccess)
            e = hipEventElapsedTime(&ms, start, stop);
        (void)hipEventDestroy(start);
        (void)hipEventDestroy(stop);
        if(rc != R355_OK)
            return rc;
        if(e != hipSuccess)
            return r355::fail(R355_ERR_LAUNCH, "timed: %s", hipGetErrorString(e));
        *avgMs = ms / static_cast<float>(iters);
        return R355_OK;
    }
} // namespace

namespace r355
{
    int fail(int code, const char* fmt, ...)
    {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(g_lastError, sizeof(g_lastError), fmt, ap);
        va_end(ap);
        return code;
    }
} // namespace r355

extern "C" {

int r355_gemm(const r355_gemm_args* args, void* stream)
{
    r355::beginCall();
    int32_t family = 0;
    int     rc     = plan(args, nullptr, &family);
    if(rc != R355_OK)
        return rc;
    return launch(args, family, static_cast<hipStream_t>(stream));
}

int r355_gemm_noalloc(const r355_gemm_args* args, void* stream)
{
    if(!args)
        return r355::fail(R355_ERR_BAD_ARG, "gemm_noalloc: args is null");
    r355::beginCall();
    void*             at = nullptr;
    const hipStream_t s  = static_cast<hipStream_t>(stream);
    int               rc = scratchOfCurrentDevice(&at, &s);
    if(rc != R355_OK)
        return rc;
    // plan as if the workspace were unbounded to learn what split-K of this problem needs, then hold it against the array
    r355_gemm_args g  = *args;
    g.workspace       = at;
    g.workspace_bytes = UINT64_MAX;
    r355_gemm_plan need;
    int32_t        family = 0;
    rc                    = plan(&g, &need, &family);
    if(rc != R355_OK)
        return rc;
    if(need.workspace_bytes > SCRATCH_BYTES)
        return r355::fail(R355_ERR_BAD_SIZE,
                          "gemm_noalloc: split-K of this problem (%u shares of %u x %u) needs %llu bytes of scratch, the library's "
                          "static buffer holds %llu; call r355_gemm with a workspace of that size, or without one",
                          need.split_k, g.m, g.n, static_cast<unsigned long long>(need.workspace_bytes),
                          static_cast<unsigned long long>(SCRATCH_BYTES));
    g.workspace_bytes = SCRATCH_BYTES;
    return launch(&g, family, static_cast<hipStream_t>(stream));
}

int r355_gemm_query(const r355_gemm_args* args, r355_gemm_plan* out)
{
    if(!out)
        return r355::fail(R355_ERR_BAD_ARG, "gemm_query: plan is null");
    int32_t family = 0;
    return plan(args, out, &family);
}

int r355_gemm_timed(const r355_gemm_args* args, void* stream, int warmup, int iters, float* avg_ms)
{
    int32_t family = 0;
    int     rc     = plan(args, nullptr, &family);
    if(rc != R355_OK)
        return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    r355::beginCall();
    return timed(s, warmup, iters, avg_ms, [&] { return launch(args, family, s); });
}

int r355_dlrm_fwd_timed(int32_t dtype, const void* in, void* out, uint32_t m, uint32_t k, uint32_t batch,
                        void* stream, int warmup, int iters, float* avg_ms)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    return timed(s, warmup, iters, avg_ms, [&] { return r355_dlrm_fwd(dtype, in, out, m, k, batch, stream); });
}

int r355_gemv_timed(int32_t layout_a, uint32_t m, uint32_t k, const float* a, uint32_t lda, const float* x,
                    const float* y_in, float* y_out, float alpha, float beta, void* stream, int warmup,
                    int iters, float* avg_ms)
{
    hipStream_t s = static_cast<hipStream_t>(stream);
    return timed(s, warmup, iters, avg_ms,
                 [&] { return r355_gemv(layout_a, m, k, a, lda, x, y_in, y_out, alpha, beta, stream); });
}

int r355_get_device_info(r355_device_info* info)
{
    if(!info)
        return r355::fail(R355_ERR_BAD_ARG, "get_device_info: info is null");
    int dev = 0;
    if(hipGetDevice(&dev) != hipSuccess)
        return r355::fail(R355_ERR_LAUNCH, "get_device_info: no HIP device");
    hipDeviceProp_t props;
    if(hipGetDeviceProperties(&props, dev) != hipSuccess)
        return r355::fail(R355_ERR_LAUNCH, "get_device_info: hipGetDeviceProperties failed");
    memset(info, 0, sizeof(*info));
    strncpy(info->arch, props.gcnArchName, sizeof(info->arch) - 1);
    info->compute_units       = props.multiProcessorCount;
    info->wave_size           = props.warpSize;
    info->clock_mhz           = props.clockRate / 1000;
    info->memory_clock_mhz    = props.memoryClockRate / 1000;
    info->lds_bytes_per_block = static_cast<int32_t>(props.sharedMemPerBlock);
    info->hbm_bytes           = props.totalGlobalMem;
    // the library's per-device set-up: from here on r355_gemm_noalloc on this device calls nothing but kernel launches
    void* at = nullptr;
    return scratchOfCurrentDevice(&at, nullptr);
}

const char* r355_last_error(void)
{
    return g_lastError;
}

const char* r355_version(void)
{
    return "rocwmma_amd 0.1 (gfx950)";
}

} // extern "C"
