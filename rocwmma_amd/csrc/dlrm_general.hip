// DLRM dot interaction for the shapes the specialised kernels of dlrm.hip do not take: more than 32 features, or an
// embedding width other than 32 / 64 / 128 / 256 (the reference's own tests run m = 128, k = 128 and m = k = 1024 with a
// batch of 64: test/dlrm/test/dlrm_test_params.hpp:55-58).  Written on the fragment API as the reference's kernels are
// (test/dlrm/device/dlrm_dot_fwd.hpp:37-135, dlrm_dot_bwd.hpp:35-176), m and k multiples of 16 as there
// (dlrm_kernel_base_impl.hpp:146-151) - but without their global scratch: the forward kernels take the lower triangle
// out of an accumulator block through 1 KiB of the wave's LDS instead of a [batch][m][m] f32 buffer, and the backward
// kernels form each 16 x 16 block of S = T + T^T in LDS from the packed upstream triangle instead of reconstructing
// [batch][m][m] in memory first.  Each direction has two forms: one 16 x 16 block per wave, as in the reference, for
// small shapes, and a register-blocked one (several blocks per wave, so that a fragment feeds several matrix
// instructions) for large ones.
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

    // Forward from 64 features on: a wave owns NB x NB blocks at once - super-block (si, sj), sj <= si, of X X^T; p = si (si +
    // 1) / 2 + sj - so that every fragment it loads feeds NB matrix instructions instead of one (a quarter of the bytes
    // from the caches per flop at NB = 4: with a block per wave m = k = 1024 reads every row block of X 64 times over).
    // BK: the K depth per step, 32 for 16-bit elements where k allows it (64-byte runs of a row per lane group instead of 32).
    template <typename T, uint32_t NB, uint32_t BK>
    __global__ void __launch_bounds__(THREADS) dlrmFwdGeneralBlocked(const T* __restrict__ in, T* __restrict__ out, uint32_t m, uint32_t k,
                                                                    uint32_t pairs)
    {
        using FragA   = fragment<matrix_a, BLK, BLK, BK, T, row_major>;
        using FragB   = fragment<matrix_b, BLK, BLK, BK, T, col_major>;
        using FragAcc = fragment<accumulator, BLK, BLK, BK, float32_t>;
        __shared__ float block[WAVES][BLK * BLK];

        const uint32_t lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        const uint32_t p    = blockIdx.x * WAVES + wave;
        if(p >= pairs)
            return;
        uint32_t si = 0;
        while((si + 1u) * (si + 2u) / 2u <= p)
            ++si;
        const uint32_t sj     = p - si * (si + 1u) / 2u;
        const uint32_t tiles  = m / BLK;
        const uint64_t stride = (uint64_t)k + (uint64_t)m * (m - 1u) / 2u;
        const T*       x      = in + (uint64_t)blockIdx.y * m * k;
        T*             o      = out + (uint64_t)blockIdx.y * stride;

        if(p == 0u) // the bottom-MLP row
            for(uint32_t e = lane; e < k; e += 64u)
                o[e] = x[e];

        // block (i, j) of the super-block is block (ti, tj) = (si NB + i, sj NB + j) of X X^T; wanted when it exists and
        // touches the strict lower triangle (tj <= ti)
        auto wanted = [&](uint32_t i, uint32_t j) { return si * NB + i < tiles && sj * NB + j < tiles && sj * NB + j <= si * NB + i; };
        FragAcc acc[NB][NB];
#pragma unroll
        for(uint32_t i = 0; i < NB; ++i)
#pragma unroll
            for(uint32_t j = 0; j < NB; ++j)
                fill_fragment(acc[i][j], 0.0f);
        for(uint32_t kk = 0; kk < k; kk += BK)
        {
            FragA a[NB];
            FragB b[NB];
#pragma unroll
            for(uint32_t i = 0; i < NB; ++i)
            {
                // (a row block past the end reads the last one again: its products are not used)
                const uint32_t ti = si * NB + i < tiles ? si * NB + i : tiles - 1u, tj = sj * NB + i < tiles ? sj * NB + i : tiles - 1u;
                load_matrix_sync(a[i], x + (uint64_t)ti * BLK * k + kk, k);
                load_matrix_sync(b[i], x + (uint64_t)tj * BLK * k + kk, k); // X^T as a col-major k x m matrix: column n is row n of X
            }
#pragma unroll
            for(uint32_t i = 0; i < NB; ++i)
#pragma unroll
                for(uint32_t j = 0; j < NB; ++j)
                    if(wanted(i, j))
                        mma_sync(acc[i][j], a[i], b[j], acc[i][j]);
        }
        float* mine = block[wave];
#pragma unroll
        for(uint32_t i = 0; i < NB; ++i)
#pragma unroll
            for(uint32_t j = 0; j < NB; ++j)
            {
                if(!wanted(i, j))
                    continue;
                store_matrix_sync(mine, acc[i][j], BLK, mem_row_major);
                __builtin_amdgcn_wave_barrier(); // (LDS is in order within a wave: the reads below see the block)
#pragma unroll
                for(uint32_t q = 0; q < BLK * BLK / 64u; ++q)
                {
                    const uint32_t e = q * 64u + lane, r = e / BLK, c = e % BLK;
                    const uint64_t gi = (uint64_t)(si * NB + i) * BLK + r, gj = (uint64_t)(sj * NB + j) * BLK + c;
                    if(gj < gi)
                        o[k + gi * (gi - 1u) / 2u + gj] = static_cast<T>(mine[e]);
                }
                __builtin_amdgcn_wave_barrier(); // the block is rewritten by the next one
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

    // Backward for large launches: a wave owns NBI x NBK blocks of the gradient - row blocks ti0 .. ti0 + NBI - 1, column
    // blocks kc0 .. kc0 + NBK - 1 - and the four waves of a workgroup share ti0: the NBI blocks of S that a step needs
    // (gathers from the packed triangle with their index arithmetic, the expensive part) are formed once per workgroup,
    // one element per thread and block, in an LDS image that every wave reads, and each feeds NBK matrix instructions per
    // wave and K step.  The 16 rows of X that a step multiplies them with go the same way: the workgroup's 256 columns of
    // them are fetched with 128-bit loads into an LDS image, from which every wave takes its matrix_b fragments (16-bit
    // types: transposing reads) - a row-major matrix_b fragment straight from global memory is four 2-byte loads per lane.
    // Both images have two buffers, so a step costs one barrier; the gathers and the rows of X for step tj + 1 are in
    // flight while the matrix instructions of step tj run.  Below the diagonal a block's rows are contiguous in the
    // triangle, above it its columns are, and the threads are laid along whichever it is.
    template <typename T, uint32_t NBI, uint32_t NBK>
    __global__ void __launch_bounds__(THREADS) dlrmBwdGeneralBlocked(const T* __restrict__ in, const T* __restrict__ upstream,
                                                                    T* __restrict__ mlpGrad, T* __restrict__ inGrad, uint32_t m, uint32_t k)
    {
        constexpr uint32_t BK = blockK<T>(), KSTEPS = BLK / BK;
        static_assert(THREADS == BLK * BLK, "one thread per element of a block of S");
        using FragA   = fragment<matrix_a, BLK, BLK, BK, T, row_major>;
        using FragB   = fragment<matrix_b, BLK, BLK, BK, T, row_major>;
        using FragAcc = fragment<accumulator, BLK, BLK, BK, float32_t>;
        // (16-bit types.  f32 fragments are four 4-byte loads per lane either way, and the image - 33 KiB - costs more in
        // resident workgroups than it saves: 512 x 128 x 256 0.28 -> 0.32 ms with it; f32 takes its fragments from global memory)
        constexpr bool     STAGE_X = sizeof(T) == 2;
        constexpr uint32_t COLS = WAVES * NBK * BLK; // columns of X (and of the gradient) per workgroup
        constexpr uint32_t XLD  = COLS + 16u / sizeof(T); // row pitch of the image of X: 16 bytes of padding
        constexpr uint32_t CH   = 16u / sizeof(T), XLOADS = BLK * COLS / CH / THREADS; // elements per 128-bit load, loads per thread
        using i32x4             = int __attribute__((ext_vector_type(4)));
        __shared__ T     sBlock[2][NBI][BLK * BLK];
        __shared__ __attribute__((aligned(16))) T xBlock[STAGE_X ? 2 : 1][STAGE_X ? BLK * XLD : CH];
        __shared__ float block[WAVES][BLK * BLK];

        const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t col0 = blockIdx.x * COLS; // first column of the workgroup
        const uint32_t kc0  = (blockIdx.x * WAVES + wave) * NBK, ti0 = blockIdx.y * NBI;
        const uint32_t tilesK = k / BLK, tilesM = m / BLK;
        const bool     active = kc0 < tilesK; // (a wave without column blocks still gathers its share of S)
        const uint64_t stride = (uint64_t)k + (uint64_t)m * (m - 1u) / 2u;
        const T*       x      = in + (uint64_t)blockIdx.z * m * k;
        const T*       up     = upstream + (uint64_t)blockIdx.z * stride;
        const T*       tril   = up + k;

        if(ti0 == 0u && lane < BLK) // bottom-MLP gradient: the first k values of the upstream row
#pragma unroll
            for(uint32_t c = 0; c < NBK; ++c)
                if(kc0 + c < tilesK)
                    mlpGrad[(uint64_t)blockIdx.z * k + (kc0 + c) * BLK + lane] = up[(kc0 + c) * BLK + lane];

        FragAcc acc[NBI][NBK];
#pragma unroll
        for(uint32_t i = 0; i < NBI; ++i)
#pragma unroll
            for(uint32_t c = 0; c < NBK; ++c)
                fill_fragment(acc[i][c], 0.0f);

        T     sNext[NBI];
        i32x4 xNext[STAGE_X ? XLOADS : 1u];
        FragB bNext[STAGE_X ? 1u : KSTEPS][NBK];
        auto  place = [&](uint32_t i, uint32_t tj, uint32_t& r, uint32_t& c) {
            const bool upper = tj > ti0 + i;
            r = upper ? tid % BLK : tid / BLK;
            c = upper ? tid / BLK : tid % BLK;
        };
        auto fetch = [&](uint32_t tj) {
#pragma unroll
            for(uint32_t i = 0; i < NBI; ++i)
            {
                uint32_t r, c;
                place(i, tj, r, c);
                const uint64_t gi = (uint64_t)(ti0 + i < tilesM ? ti0 + i : ti0) * BLK + r, gj = (uint64_t)tj * BLK + c;
                const uint64_t hi = gi > gj ? gi : gj, lo = gi > gj ? gj : gi;
                sNext[i] = gi == gj ? static_cast<T>(0.0f) : tril[hi * (hi - 1u) / 2u + lo];
            }
            if constexpr(STAGE_X)
            {
#pragma unroll
                for(uint32_t j = 0; j < XLOADS; ++j) // rows tj * 16 ... of X, the workgroup's columns (k is a multiple of 16: whole pieces)
                {
                    const uint32_t piece = j * THREADS + tid, r = piece / (COLS / CH), c = col0 + (piece % (COLS / CH)) * CH;
                    if(c < k)
                        xNext[j] = *reinterpret_cast<const i32x4*>(x + ((uint64_t)tj * BLK + r) * k + c);
                }
            }
            else if(active)
            {
#pragma unroll
                for(uint32_t ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
                    for(uint32_t c = 0; c < NBK; ++c) // (a column block past the end reads the last one again: its products are not used)
                        load_matrix_sync(bNext[ks][c],
                                         x + (uint64_t)tj * BLK * k + (uint64_t)(kc0 + c < tilesK ? kc0 + c : tilesK - 1u) * BLK + (uint64_t)ks * BK * k, k);
            }
        };
        fetch(0u);
        for(uint32_t tj = 0; tj < tilesM; ++tj)
        {
            T(*s)[BLK * BLK] = sBlock[tj & 1u];
            T* xs            = xBlock[STAGE_X ? tj & 1u : 0u];
            FragB bNow[STAGE_X ? 1u : KSTEPS][NBK];
#pragma unroll
            for(uint32_t i = 0; i < NBI; ++i)
            {
                uint32_t r, c;
                place(i, tj, r, c);
                s[i][r * BLK + c] = sNext[i];
            }
            if constexpr(STAGE_X)
            {
#pragma unroll
                for(uint32_t j = 0; j < XLOADS; ++j)
                {
                    const uint32_t piece = j * THREADS + tid, r = piece / (COLS / CH), c = (piece % (COLS / CH)) * CH;
                    if(col0 + c < k)
                        *reinterpret_cast<i32x4*>(xs + r * XLD + c) = xNext[j];
                }
            }
            else
            {
#pragma unroll
                for(uint32_t ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
                    for(uint32_t c = 0; c < NBK; ++c)
                        bNow[ks][c] = bNext[ks][c];
            }
            // the one barrier of the step: these buffers are complete; the others, which the next step writes, were last read
            // in the step before this one, and every wave has finished that step to get here
            __syncthreads();
            if(tj + 1u < tilesM)
                fetch(tj + 1u);
            if(active)
#pragma unroll
                for(uint32_t ks = 0; ks < KSTEPS; ++ks)
                {
                    FragA a[NBI];
                    FragB b[NBK];
#pragma unroll
                    for(uint32_t i = 0; i < NBI; ++i)
                        load_matrix_sync(a[i], s[i] + ks * BK, BLK);
#pragma unroll
                    for(uint32_t c = 0; c < NBK; ++c)
                        if constexpr(STAGE_X)
                            load_matrix_sync(b[c], xs + ks * BK * XLD + ((kc0 + c < tilesK ? kc0 + c : tilesK - 1u) * BLK - col0), XLD);
                        else
                            b[c] = bNow[ks][c];
#pragma unroll
                    for(uint32_t i = 0; i < NBI; ++i)
#pragma unroll
                        for(uint32_t c = 0; c < NBK; ++c)
                            if(ti0 + i < tilesM && kc0 + c < tilesK)
                                mma_sync(acc[i][c], a[i], b[c], acc[i][c]);
                }
        }
        if(!active)
            return;
        float* mine = block[wave];
#pragma unroll
        for(uint32_t i = 0; i < NBI; ++i)
#pragma unroll
            for(uint32_t c = 0; c < NBK; ++c)
            {
                if(ti0 + i >= tilesM || kc0 + c >= tilesK)
                    continue;
                store_matrix_sync(mine, acc[i][c], BLK, mem_row_major);
                __builtin_amdgcn_wave_barrier();
                T* g = inGrad + (uint64_t)blockIdx.z * m * k + (uint64_t)(ti0 + i) * BLK * k + (uint64_t)(kc0 + c) * BLK;
#pragma unroll
                for(uint32_t q = 0; q < BLK * BLK / 64u; ++q)
                {
                    const uint32_t e = q * 64u + lane, r = e / BLK, cc = e % BLK;
                    g[(uint64_t)r * k + cc] = static_cast<T>(mine[e]);
                }
                __builtin_amdgcn_wave_barrier(); // the block is rewritten by the next one
            }
    }

    template <typename T>
    int fwd(const void* in, void* out, uint32_t m, uint32_t k, uint32_t batch, hipStream_t s)
    {
        constexpr uint32_t NB = 4;
#ifdef R355_DLRM_BLOCK_PER_WAVE // measurement build: the block-per-wave kernels for every shape
        const bool blocked = false;
#else
        // NB x NB blocks per wave from 64 features on, where that still leaves every SIMD two waves or so (fewer, and the
        // many short waves of the block-per-wave kernel hide latency better: 128 x 128 x 64 runs 8 us against 10)
        const uint32_t supers  = (m / BLK + NB - 1u) / NB;
        const bool     blocked = m >= NB * BLK && (uint64_t)supers * (supers + 1u) / 2u * batch >= 2ull * r355::computeUnits();
#endif
        const uint32_t tiles = blocked ? (m / BLK + NB - 1u) / NB : m / BLK, pairs = tiles * (tiles + 1u) / 2u;
        const uint64_t stride = (uint64_t)k + (uint64_t)m * (m - 1u) / 2u;
        // the batch is a grid dimension of at most 65535: a larger one goes out in several launches on the same stream
        for(uint32_t first = 0; first < batch; first += GRID_BATCH)
        {
            const uint32_t count = batch - first < GRID_BATCH ? batch - first : GRID_BATCH;
            const dim3     grid((pairs + WAVES - 1u) / WAVES, count);
            const T*       src = static_cast<const T*>(in) + (uint64_t)first * m * k;
            T*             dst = static_cast<T*>(out) + (uint64_t)first * stride;
            if(!blocked)
                hipLaunchKernelGGL((dlrmFwdGeneral<T>), grid, dim3(THREADS), 0, s, src, dst, m, k, pairs);
            else if(sizeof(T) == 2 && k % 32u == 0u)
                hipLaunchKernelGGL((dlrmFwdGeneralBlocked<T, NB, sizeof(T) == 2 ? 32u : blockK<T>()>), grid, dim3(THREADS), 0, s, src, dst, m, k, pairs);
            else
                hipLaunchKernelGGL((dlrmFwdGeneralBlocked<T, NB, blockK<T>()>), grid, dim3(THREADS), 0, s, src, dst, m, k, pairs);
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
            constexpr uint32_t NBI = 2, NBK = 4;
            const T*           src = static_cast<const T*>(in) + (uint64_t)first * m * k;
            const T*           ups = static_cast<const T*>(up) + (uint64_t)first * stride;
            T*                 dm  = static_cast<T*>(mlp) + (uint64_t)first * k;
            T*                 dg  = static_cast<T*>(grad) + (uint64_t)first * m * k;
            const uint64_t waves = (uint64_t)((k / BLK + NBK - 1u) / NBK) * ((m / BLK + NBI - 1u) / NBI) * count;
#ifdef R355_DLRM_BLOCK_PER_WAVE
            const bool blocked = false;
#else
            const bool blocked = waves >= 8ull * r355::computeUnits(); // where that still leaves every SIMD two waves
#endif
            if(blocked) // NBI x NBK blocks per wave
                hipLaunchKernelGGL((dlrmBwdGeneralBlocked<T, NBI, NBK>),
                                   dim3(((k / BLK + NBK - 1u) / NBK + WAVES - 1u) / WAVES, (m / BLK + NBI - 1u) / NBI, count), dim3(THREADS), 0,
                                   s, src, ups, dm, dg, m, k);
            else
                hipLaunchKernelGGL((dlrmBwdGeneral<T>), dim3((k / BLK + WAVES - 1u) / WAVES, m / BLK, count), dim3(THREADS), 0, s, src, ups, dm, dg,
                                   m, k);
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
