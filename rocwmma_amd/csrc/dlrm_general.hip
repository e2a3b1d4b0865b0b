// DLRM dot interaction for the shapes the specialised kernels of dlrm.hip do not take: more than 32 features, or an
// embedding width other than 32 / 64 / 128 / 256 (the reference's own tests run m = 128, k = 128 and m = k = 1024 with a
// batch of 64: test/dlrm/test/dlrm_test_params.hpp:55-58).  Written on the fragment API, one 16 x 16 block per wave as in
// the reference's kernels (test/dlrm/device/dlrm_dot_fwd.hpp:37-135, dlrm_dot_bwd.hpp:35-176), m and k multiples of 16
// as there (dlrm_kernel_base_impl.hpp:146-151) - but without their global scratch: the forward kernel takes the lower
// triangle out of the accumulator block through 1 KiB of the wave's LDS instead of a [batch][m][m] f32 buffer, and the
// backward kernel forms each 16 x 16 block of S = T + T^T in LDS from the packed upstream triangle instead of
// reconstructing [batch][m][m] in memory first.  Correctness first: these run at the latency of block-per-wave code.
#include <rocwmma/rocwmma.hpp>

#include "common.hpp"

using namespace rocwmma;

namespace
{
    constexpr uint32_t BLK = 16, WAVES = 4, THREADS = WAVES * 64;
    constexpr uint32_t GRID_BATCH = 65535; // samples per launch (the batch is grid dimension y or z)

    template <typename T>
    constexpr uint32_t blockK()
    {
        return sizeof(T) == 4 ? 4u : 16u; // the K depth of the 16 x 16 matrix instruction behind mma_sync
    }

    // Forward.  Wave p of sample blockIdx.y owns block (ti, tj), tj <= ti, of X X^T; p = ti (ti + 1) / 2 + tj.
    template <typename T>
    __global__ void __launch_bounds__(THREADS) dlrmFwdGeneral(const T* __restrict__ in, T* __restrict__ out, uint32_t m, uint32_t k,
                                                             uint32_t pairs)
    {
        constexpr uint32_t BK = blockK<T>();
        using FragA   = fragment<matrix_a, BLK, BLK, BK, T, row_major>;
        using FragB   = fragment<matrix_b, BLK, BLK, BK, T, col_major>;
        using FragAcc = fragment<accumulator, BLK, BLK, BK, float32_t>;
        __shared__ float block[WAVES][BLK * BLK];

        const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
        const uint32_t p    = blockIdx.x * WAVES + wave;
        if(p >= pairs)
            return;
        uint32_t ti = 0;
        while((ti + 1u) * (ti + 2u) / 2u <= p)
            ++ti;
        const uint32_t tj     = p - ti * (ti + 1u) / 2u;
        const uint64_t stride = (uint64_t)k + (uint64_t)m * (m - 1u) / 2u;
        const T*       x      = in + (uint64_t)blockIdx.y * m * k;
        T*             o      = out + (uint64_t)blockIdx.y * stride;

        if(p == 0u) // the bottom-MLP row
            for(uint32_t e = lane; e < k; e += 64u)
                o[e] = x[e];

        FragAcc acc;
        fill_fragment(acc, 0.0f);
        const T* pa = x + (uint64_t)ti * BLK * k; // rows of X
        const T* pb = x + (uint64_t)tj * BLK * k; // X^T as a col-major k x m matrix: column n is row n of X
        for(uint32_t kk = 0; kk < k; kk += BK)
        {
            FragA a;
            FragB b;
            load_matrix_sync(a, pa + kk, k);
            load_matrix_sync(b, pb + kk, k);
            mma_sync(acc, a, b, acc);
        }
        float* mine = block[wave];
        store_matrix_sync(mine, acc, BLK, mem_row_major);
        __builtin_amdgcn_wave_barrier(); // (LDS is in order within a wave: the reads below see the block)
#pragma unroll
        for(uint32_t i = 0; i < BLK * BLK / 64u; ++i)
        {
            const uint32_t e = i * 64u + lane, r = e / BLK, c = e % BLK;
            const uint64_t gi = (uint64_t)ti * BLK + r, gj = (uint64_t)tj * BLK + c;
            if(gj < gi)
                o[k + gi * (gi - 1u) / 2u + gj] = static_cast<T>(mine[e]);
        }
    }

    // Backward.  Wave (ti, kc) of sample blockIdx.z owns block (ti, kc) of the gradient S X; S(i, j) is the upstream
    // triangle's element (max, min) of i, j and zero on the diagonal.
    template <typename T>
    __global__ void __launch_bounds__(THREADS) dlrmBwdGeneral(const T* __restrict__ in, const T* __restrict__ upstream,
                                                             T* __restrict__ mlpGrad, T* __restrict__ inGrad, uint32_t m, uint32_t k)
    {
        constexpr uint32_t BK = blockK<T>();
        using FragA   = fragment<matrix_a, BLK, BLK, BK, T, row_major>;
        using FragB   = fragment<matrix_b, BLK, BLK, BK, T, row_major>;
        using FragAcc = fragment<accumulator, BLK, BLK, BK, float32_t>;
        __shared__ T     sBlock[WAVES][BLK * BLK];
        __shared__ float block[WAVES][BLK * BLK];

        const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
        const uint32_t kc   = blockIdx.x * WAVES + wave, ti = blockIdx.y;
        if(kc * BLK >= k)
            return;
        const uint64_t stride = (uint64_t)k + (uint64_t)m * (m - 1u) / 2u;
        const T*       x      = in + (uint64_t)blockIdx.z * m * k;
        const T*       up     = upstream + (uint64_t)blockIdx.z * stride;
        const T*       tril   = up + k;

        if(ti == 0u && lane < BLK) // bottom-MLP gradient: the first k values of the upstream row
            mlpGrad[(uint64_t)blockIdx.z * k + kc * BLK + lane] = up[kc * BLK + lane];

        FragAcc acc;
        fill_fragment(acc, 0.0f);
        T* s = sBlock[wave];
        for(uint32_t tj = 0; tj < m / BLK; ++tj)
        {
#pragma unroll
            for(uint32_t i = 0; i < BLK * BLK / 64u; ++i)
            {
                const uint32_t e = i * 64u + lane, r = e / BLK, c = e % BLK;
                const uint64_t gi = (uint64_t)ti * BLK + r, gj = (uint64_t)tj * BLK + c;
                const uint64_t hi = gi > gj ? gi : gj, lo = gi > gj ? gj : gi;
                s[e] = gi == gj ? static_cast<T>(0.0f) : tril[hi * (hi - 1u) / 2u + lo];
            }
            __builtin_amdgcn_wave_barrier();
            const T* pb = x + (uint64_t)tj * BLK * k + kc * BLK;
#pragma unroll
            for(uint32_t kk = 0; kk < BLK; kk += BK)
            {
                FragA a;
                FragB b;
                load_matrix_sync(a, s + kk, BLK);
                load_matrix_sync(b, pb + (uint64_t)kk * k, k);
                mma_sync(acc, a, b, acc);
            }
            __builtin_amdgcn_wave_barrier(); // the block of S is rewritten in the next trip
        }
        float* mine = block[wave];
        store_matrix_sync(mine, acc, BLK, mem_row_major);
        __builtin_amdgcn_wave_barrier();
        T* g = inGrad + (uint64_t)blockIdx.z * m * k + (uint64_t)ti * BLK * k + kc * BLK;
#pragma unroll
        for(uint32_t i = 0; i < BLK * BLK / 64u; ++i)
        {
            const uint32_t e = i * 64u + lane, r = e / BLK, c = e % BLK;
            g[(uint64_t)r * k + c] = static_cast<T>(mine[e]);
        }
    }

    template <typename T>
    int fwd(const void* in, void* out, uint32_t m, uint32_t k, uint32_t batch, hipStream_t s)
    {
        const uint32_t tiles = m / BLK, pairs = tiles * (tiles + 1u) / 2u;
        const uint64_t stride = (uint64_t)k + (uint64_t)m * (m - 1u) / 2u;
        // the batch is a grid dimension of at most 65535: a larger one goes out in several launches on the same stream
        for(uint32_t first = 0; first < batch; first += GRID_BATCH)
        {
            const uint32_t count = batch - first < GRID_BATCH ? batch - first : GRID_BATCH;
            hipLaunchKernelGGL((dlrmFwdGeneral<T>), dim3((pairs + WAVES - 1u) / WAVES, count), dim3(THREADS), 0, s,
                               static_cast<const T*>(in) + (uint64_t)first * m * k, static_cast<T*>(out) + (uint64_t)first * stride, m, k, pairs);
        }
        return r355::checkLaunch("dlrm_fwd (general)");
    }
    template <typename T>
    int bwd(const void* in, const void* up, void* mlp, void* grad, uint32_t m, uint32_t k, uint32_t batch, hipStream_t s)
    {
        const uint64_t stride = (uint64_t)k + (uint64_t)m * (m - 1u) / 2u;
        for(uint32_t first = 0; first < batch; first += GRID_BATCH)
        {
            const uint32_t count = batch - first < GRID_BATCH ? batch - first : GRID_BATCH;
            hipLaunchKernelGGL((dlrmBwdGeneral<T>), dim3((k / BLK + WAVES - 1u) / WAVES, m / BLK, count), dim3(THREADS), 0, s,
                               static_cast<const T*>(in) + (uint64_t)first * m * k, static_cast<const T*>(up) + (uint64_t)first * stride,
                               static_cast<T*>(mlp) + (uint64_t)first * k, static_cast<T*>(grad) + (uint64_t)first * m * k, m, k);
        }
        return r355::checkLaunch("dlrm_bwd (general)");
    }

    int checkGeneral(const char* what, uint32_t m, uint32_t k, uint32_t batch)
    {
        if(m % BLK || k % BLK || m == 0u || k == 0u)
            return r355::fail(R355_ERR_BAD_SIZE,
                              "%s: m=%u, k=%u - beyond m <= 32 with k of 32, 64, 128 or 256 (f32: up to 128) both must be multiples of %u", what,
                              m, k, BLK);
        (void)batch; // any batch: beyond 65535 samples the launch is repeated (fwd / bwd above)
        return R355_OK;
    }
} // namespace

namespace r355
{
    int dlrmGeneralFwd(int32_t dtype, const void* in, void* out, uint32_t m, uint32_t k, uint32_t batch, hipStream_t s)
    {
        const int rc = checkGeneral("dlrm_fwd", m, k, batch);
        if(rc != R355_OK)
            return rc;
        switch(dtype)
        {
        case R355_F16: return fwd<float16_t>(in, out, m, k, batch, s);
        case R355_BF16: return fwd<bfloat16_t>(in, out, m, k, batch, s);
        default: return fwd<float32_t>(in, out, m, k, batch, s);
        }
    }
    int dlrmGeneralBwd(int32_t dtype, const void* in, const void* upstream, void* mlpGrad, void* inGrad, uint32_t m, uint32_t k,
                       uint32_t batch, hipStream_t s)
    {
        const int rc = checkGeneral("dlrm_bwd", m, k, batch);
        if(rc != R355_OK)
            return rc;
        switch(dtype)
        {
        case R355_F16: return bwd<float16_t>(in, upstream, mlpGrad, inGrad, m, k, batch, s);
        case R355_BF16: return bwd<bfloat16_t>(in, upstream, mlpGrad, inGrad, m, k, batch, s);
        default: return bwd<float32_t>(in, upstream, mlpGrad, inGrad, m, k, batch, s);
        }
    }
} // namespace r355
