// GEMV y = alpha * A x + beta * y for f32 and f64, HBM-bound: A is read exactly once with
// coalesced 128-bit loads, several per lane requested before the first is used; the order of the
// sums is fixed by the shape alone (never by scheduling).
//
// Takes the place of samples/simple_sgemv.cpp:103-150 (f64: samples/simple_dgemv.cpp:103), which feeds 16x16x16 f32 fragments
// (the B fragment being x broadcast 16 times) to the matrix core.  At 0.5 flop per byte
// the matrix core contributes nothing; the kernel is organised for memory bandwidth.
//   col-major A (the sample's layout): a workgroup of sixteen waves owns 32 or 64 rows (f64: 16 or 32); its lanes split
//     the columns and combine their partial sums through LDS in a fixed order.
//   row-major A: one wave per row, lanes stride k in 16-byte pieces, then a wave reduction.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.hpp"

namespace
{
    constexpr uint32_t THREADS = 256;
    constexpr uint32_t SHARED_ROWS = 4; // rows per workgroup of gemvRowMajorShared

    // col-major A (m contiguous).  A lane loads 16 bytes = V consecutive rows of one column; RL lanes side by side make a
    // run of RL * 16 bytes of that column and the wave's other lanes take the next 64 / RL - 1 columns, so a workgroup of
    // COL_WAVES waves owns RL * V rows and walks the columns COL_WAVES * 64 / RL at a time, DEPTH steps requested before the
    // first is used.  RL = 8 (128-byte runs, 32 rows of f32 per workgroup) gives 8192 rows a workgroup per CU; RL = 16
    // (256-byte runs) is taken when the rows suffice for that.  Every lane sums its columns in increasing order; the
    // COL_WAVES * 64 / RL partial sums of a row meet in LDS and are added in a fixed order, so the result does not depend
    // on scheduling.  STREAM as in the row-major kernel.
    // SPLIT: workgroup (b, s) of a two-dimensional grid sums columns [s kPer, (s + 1) kPer) only and leaves its rows' sums,
    // unscaled, in an array of partial sums (yOut; element (row, s) at row * partRow + s * partSplit) for gemvAddSplits.
    template <typename T, uint32_t RL, uint32_t COL_WAVES, bool STREAM, bool SPLIT = false>
    __global__ void __launch_bounds__(COL_WAVES * 64) gemvColMajor(uint32_t m,
                                                                  uint32_t k,
                                                                  const T* a,
                                                                  uint32_t lda,
                                                                  const T* x,
                                                                  const T* yIn,
                                                                  T*       yOut,
                                                                  T        alpha,
                                                                  T        beta,
                                                                  uint32_t kPer,
                                                                  uint32_t partRow,
                                                                  uint32_t partSplit)
    {
        constexpr uint32_t V = 16u / sizeof(T), ROWS = RL * V, CL = 64u / RL, COLS = COL_WAVES * CL, DEPTH = 8;
        using VecT = T __attribute__((ext_vector_type(V)));
        __shared__ T   partial[COLS][ROWS];
        const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
        const uint32_t r = lane % RL, c = lane / RL;
        const uint32_t row0 = blockIdx.x * ROWS + r * V; // (m is a multiple of V: a lane's rows are inside or outside together)
        T              acc[V];
#pragma unroll
        for(uint32_t e = 0; e < V; ++e)
            acc[e] = T(0);
        if(row0 < m)
        {
            const T* p     = a + row0;
            auto     fetch = [](const T* at) {
                if constexpr(STREAM)
                    return __builtin_nontemporal_load(reinterpret_cast<const VecT*>(at));
                else
                    return *reinterpret_cast<const VecT*>(at);
            };
            const uint32_t kEnd = SPLIT ? (k - blockIdx.y * kPer < kPer ? k : (blockIdx.y + 1u) * kPer) : k;
            uint32_t       kk   = (SPLIT ? blockIdx.y * kPer : 0u) + wave * CL + c;
            for(; kk + (DEPTH - 1u) * COLS < kEnd; kk += DEPTH * COLS)
            {
                VecT v[DEPTH];
                T    xv[DEPTH];
#pragma unroll
                for(uint32_t u = 0; u < DEPTH; ++u)
                    v[u] = fetch(p + (uint64_t)(kk + u * COLS) * lda);
#pragma unroll
                for(uint32_t u = 0; u < DEPTH; ++u)
                    xv[u] = x[kk + u * COLS];
#pragma unroll
                for(uint32_t u = 0; u < DEPTH; ++u)
#pragma unroll
                    for(uint32_t e = 0; e < V; ++e)
                        acc[e] += v[u][e] * xv[u];
            }
            for(; kk < kEnd; kk += COLS)
            {
                const VecT v  = fetch(p + (uint64_t)kk * lda);
                const T    xv = x[kk];
#pragma unroll
                for(uint32_t e = 0; e < V; ++e)
                    acc[e] += v[e] * xv;
            }
        }
#pragma unroll
        for(uint32_t e = 0; e < V; ++e)
            partial[wave * CL + c][r * V + e] = acc[e];
        __syncthreads();
        if(threadIdx.x < ROWS)
        {
            const uint32_t row = blockIdx.x * ROWS + threadIdx.x;
            if(row < m)
            {
                T sum = T(0);
#pragma unroll
                for(uint32_t w = 0; w < COLS; ++w)
                    sum += partial[w][threadIdx.x];
                if constexpr(SPLIT)
                    yOut[(uint64_t)row * partRow + (uint64_t)blockIdx.y * partSplit] = sum;
                else
                    yOut[row] = beta != T(0) ? alpha * sum + beta * yIn[row] : alpha * sum;
            }
        }
    }

    // Second kernel of the split forms: y = alpha * (sum of a row's partial sums) + beta * y, in an order that the number
    // of splits alone decides.
    // Many splits (32 and more: few rows): the partial sums are stored [m][splits] and a wave takes a row - lane l adds
    // those of splits l, l + 64, ... in that order and the 64 lane sums meet in a fixed tree; one memory latency, where a
    // thread per row walking 64 splits took 4.7 us and 256 splits longer than the first kernel.
    template <typename T>
    __global__ void __launch_bounds__(THREADS) gemvAddSplitsByWave(uint32_t m, uint32_t splits, const T* partial, const T* yIn, T* yOut, T alpha, T beta)
    {
        const uint32_t lane = threadIdx.x & 63u, row = blockIdx.x * (THREADS / 64u) + threadIdx.x / 64u;
        if(row >= m)
            return;
        const T* p   = partial + (uint64_t)row * splits;
        T        sum = T(0);
        for(uint32_t s0 = lane; s0 < splits; s0 += 64u)
            sum += p[s0];
#pragma unroll
        for(uint32_t off = 32; off > 0; off >>= 1)
            sum += __shfl_xor(sum, off, 64);
        if(lane == 0)
            yOut[row] = beta != T(0) ? alpha * sum + beta * yIn[row] : alpha * sum;
    }
    // Few splits (many rows): stored [splits][m], a thread per row adds them in split order, eight requests under way.
    template <typename T>
    __global__ void __launch_bounds__(THREADS) gemvAddSplits(uint32_t m, uint32_t splits, const T* partial, const T* yIn, T* yOut, T alpha, T beta)
    {
        const uint32_t row = blockIdx.x * THREADS + threadIdx.x;
        if(row >= m)
            return;
        T sum = T(0);
        for(uint32_t s0 = 0; s0 < splits; s0 += 8u)
        {
            T v[8];
#pragma unroll
            for(uint32_t u = 0; u < 8u; ++u)
                v[u] = s0 + u < splits ? partial[(uint64_t)(s0 + u) * m + row] : T(0);
#pragma unroll
            for(uint32_t u = 0; u < 8u; ++u)
                sum += v[u];
        }
        yOut[row] = beta != T(0) ? alpha * sum + beta * yIn[row] : alpha * sum;
    }

    // STREAM: A does not fit the 256 MiB memory-side cache, so nothing of it can be there from an earlier call or be wanted
    // by a later one: nontemporal loads (measured: 16384^2 f32 0.174 -> 0.164 ms, 65536 x 2048 0.086 -> 0.073).  Otherwise
    // ordinary loads (8192^2 f32, exactly 256 MiB, called again and again: 0.0389 -> 0.0370 ms; 0.0409 with nontemporal
    // loads) and rows that start at different groups of k.
    template <typename T, bool STREAM>
    __global__ void __launch_bounds__(THREADS) gemvRowMajor(uint32_t m,
                                                           uint32_t k,
                                                           const T* a,
                                                           uint32_t lda,
                                                           const T* x,
                                                           const T* yIn,
                                                           T*       yOut,
                                                           T        alpha,
                                                           T        beta)
    {
        constexpr uint32_t V = 16u / sizeof(T); // elements of a 128-bit load
        using VecT           = T __attribute__((ext_vector_type(V)));
        const uint32_t lane  = threadIdx.x & 63u;
        const uint32_t row   = blockIdx.x * (THREADS / 64u) + threadIdx.x / 64u;
        if(row >= m)
            return;
        const T* p   = a + (uint64_t)row * lda;
        T        acc = T(0);
        // DEPTH loads of A per lane are requested before the first is used (bytes in flight are what keeps HBM busy; one load
        // per trip, waited for at once, left that to the number of resident waves alone).  Unless A streams, rows start at
        // different groups of k and wrap around: with a power-of-two leading dimension all rows are aligned alike, and waves
        // that walk their rows in step are all on the same few memory channels at any one time.
        constexpr uint32_t DEPTH = 4, STEP = 64u * V, GROUP = DEPTH * STEP;
        const uint32_t     groups = k / GROUP, g0 = (!STREAM && groups) ? (row * 5u) % groups : 0u;
        auto               fetch  = [](const T* at) {
            if constexpr(STREAM)
                return __builtin_nontemporal_load(reinterpret_cast<const VecT*>(at));
            else
                return *reinterpret_cast<const VecT*>(at);
        };
        for(uint32_t t = 0; t < groups; ++t)
        {
            const uint32_t g  = g0 + t < groups ? g0 + t : g0 + t - groups;
            const uint32_t kk = g * GROUP + lane * V;
            VecT           v[DEPTH], xv[DEPTH];
#pragma unroll
            for(uint32_t u = 0; u < DEPTH; ++u)
                v[u] = fetch(p + kk + u * STEP);
#pragma unroll
            for(uint32_t u = 0; u < DEPTH; ++u)
                xv[u] = *reinterpret_cast<const VecT*>(x + kk + u * STEP);
#pragma unroll
            for(uint32_t u = 0; u < DEPTH; ++u)
#pragma unroll
                for(uint32_t e = 0; e < V; ++e)
                    acc += v[u][e] * xv[u][e];
        }
        for(uint32_t kk = groups * GROUP + lane * V; kk < k; kk += STEP)
        {
            const VecT v  = fetch(p + kk);
            const VecT xv = *reinterpret_cast<const VecT*>(x + kk);
#pragma unroll
            for(uint32_t e = 0; e < V; ++e)
                acc += v[e] * xv[e];
        }
#pragma unroll
        for(uint32_t off = 32; off > 0; off >>= 1)
            acc += __shfl_xor(acc, off, 64);
        if(lane == 0)
            yOut[row] = beta != T(0) ? alpha * acc + beta * yIn[row] : alpha * acc;
    }

    // Long rows of a matrix too large for the memory-side cache.  One row per wave (above) has every resident wave on a
    // row of its own, thousands of 4 KiB pieces a row length apart at any moment, and its rate falls with the row length
    // (f32, 1 GiB of A: 0.92 of the HBM peak at k = 2048, 0.86 at 8192, 0.82 at 16384, 0.79 at 32768), while the
    // column-major kernel, whose workgroups together sweep memory linearly, holds 0.89.  Here the WAVES waves of a workgroup
    // share each row: one load instruction per wave covers WAVES KiB of it together, the workgroup goes through its RB rows one
    // after the other with that piece of x held in registers, and only then moves on along k.  Each wave waits for its
    // load before it asks for the next row: variants with two or four loads per row under way, or with the next row's
    // requested ahead, were slower the more they had in flight (16384^2 f32: 0.77, 0.67, 0.64 of the peak against 0.86),
    // and so were 8 and 16 rows per workgroup.  Eight waves are ahead for rows below 128 KiB, sixteen from there on
    // (16384^2: 0.887 / 0.844; 8192 x 32768: 0.818 / 0.882; 32768^2: 0.842 / 0.895; one row per wave: 0.82, 0.79, 0.82).
    // STREAM: A lies beyond the memory-side cache and is read with nontemporal loads; a smaller one (few very long rows
    // of a matrix that is multiplied again and again) keeps ordinary loads so that the next call finds it there, as in
    // gemvRowMajor / gemvColMajor.
    // SPLIT: workgroup (s, b) of a grid whose fast index is the split takes elements [s kPer, (s + 1) kPer) of its RB rows
    // only (kPer a multiple of the slice) and leaves the sums, unscaled, in the array of partial sums (yOut, as in
    // gemvColMajor) for gemvAddSplits.  With pieces of 128 KiB the workgroups that run at the same time read neighbouring pieces of the
    // same rows, and the RB rows of a workgroup share every load of x: one row per workgroup reads as many bytes of x
    // (from the caches) as of A, and no variant of it - 4 to 16 waves, 4 to 16 loads in flight, software-pipelined,
    // either grid order - passed 0.80 of the HBM peak on 512 MiB ... 1 GiB of A, where four rows per workgroup of eight
    // waves with two slices of each in flight reach 0.85 - 0.90 (256 x 524288: 0.78 -> 0.88, 1024 x 262144: 0.79 -> 0.90,
    // 64 x 2097152: 0.78 -> 0.86; two rows: 0.89 / 0.89 / 0.86, eight: 0.84 / 0.86 / 0.84).
    // BATCH (without SPLIT): the same loop - every load of a group requested before the first is used, x shared by the
    // workgroup's rows - over whole rows, for a streamed matrix of 384 ... 2047 long rows, where it needs no workspace:
    // two or four rows per workgroup, whichever leaves the CUs evenly loaded (f32, rows of 512 KiB - 1 MiB: 512 rows 0.77
    // -> 0.86, 1024 rows 0.78 -> 0.88, 1536 rows 0.78 -> 0.87, 2000 rows 0.78 -> 0.88 of the HBM peak).
    template <typename T, uint32_t WAVES, uint32_t RB = SHARED_ROWS, bool STREAM = true, bool SPLIT = false, bool BATCH = SPLIT>
    __global__ void __launch_bounds__(WAVES * 64u) gemvRowMajorShared(uint32_t m,
                                                                      uint32_t k,
                                                                      const T* a,
                                                                      uint32_t lda,
                                                                      const T* x,
                                                                      const T* yIn,
                                                                      T*       yOut,
                                                                      T        alpha,
                                                                      T        beta,
                                                                      uint32_t kPer,
                                                                      uint32_t partRow,
                                                                      uint32_t partSplit)
    {
        constexpr uint32_t V = 16u / sizeof(T);
        constexpr uint32_t SLICE = WAVES * 64u * 16u; // bytes one load instruction of the whole workgroup covers
        constexpr int      NT    = STREAM ? 2 : 0; // cache policy of the loads of A: nontemporal when it is read once
        using VecT               = T __attribute__((ext_vector_type(V)));
        __shared__ T   partial[WAVES][RB];
        const uint32_t lane = threadIdx.x & 63u, w = threadIdx.x / 64u;
        const uint32_t row0 = (SPLIT ? blockIdx.y : blockIdx.x) * RB;
        const uint32_t kBeg = SPLIT ? blockIdx.x * kPer : 0u; // (wave-uniform)
        const uint32_t kBytes = (SPLIT ? (k - kBeg < kPer ? k - kBeg : kPer) : k) * (uint32_t)sizeof(T);
        // One buffer per row and one for x, each k elements long: what a load asks for beyond that comes back as zero, so
        // a row that does not fill its last slice needs no separate tail, and a row past m (a buffer of no bytes) adds
        // nothing.  The rows are wave-uniform: their descriptors stay in scalar registers.
        auto buffer = [](const T* base, uint32_t bytes) {
            const uint64_t addr = reinterpret_cast<uint64_t>(base);
            const uint32_t lo   = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr));
            const uint32_t hi   = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr >> 32));
            return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>((static_cast<uint64_t>(hi) << 32) | lo), 0,
                                                     static_cast<int>(__builtin_amdgcn_readfirstlane(bytes)), 0x00020000);
        };
        const __amdgpu_buffer_rsrc_t xr = buffer(x + kBeg, kBytes);
        __amdgpu_buffer_rsrc_t       rows[RB];
        T                            acc[RB];
#pragma unroll
        for(uint32_t r = 0; r < RB; ++r)
        {
            rows[r] = buffer(a + (uint64_t)(row0 + r < m ? row0 + r : 0u) * lda + kBeg, row0 + r < m ? kBytes : 0u);
            acc[r]  = T(0);
        }
        const uint32_t mine = (w * 64u + lane) * 16u;
        uint32_t       kc   = 0;
        if constexpr(BATCH)
        {
            // all of a group's loads - two (four rows) or four (two rows) slices of every row and of x - are requested
            // before the first is used
            constexpr uint32_t AHEAD = RB >= 4u ? 2u : 4u;
            for(; kc < kBytes; kc += AHEAD * SLICE)
            {
                VecT v[RB][AHEAD], xv[AHEAD];
#pragma unroll
                for(uint32_t r = 0; r < RB; ++r)
#pragma unroll
                    for(uint32_t u = 0; u < AHEAD; ++u)
                        v[r][u] = __builtin_bit_cast(VecT, __builtin_amdgcn_raw_buffer_load_b128(rows[r], mine, kc + u * SLICE, NT));
#pragma unroll
                for(uint32_t u = 0; u < AHEAD; ++u)
                    xv[u] = __builtin_bit_cast(VecT, __builtin_amdgcn_raw_buffer_load_b128(xr, mine, kc + u * SLICE, 0));
#pragma unroll
                for(uint32_t r = 0; r < RB; ++r)
#pragma unroll
                    for(uint32_t u = 0; u < AHEAD; ++u)
#pragma unroll
                        for(uint32_t e = 0; e < V; ++e)
                            acc[r] += v[r][u][e] * xv[u][e];
            }
        }
        else if constexpr(RB == 1u)
        {
            // a single row per workgroup: nothing but this row's slices to overlap, so several of them are requested
            // before the first is used
            constexpr uint32_t AHEAD = 4;
            for(; kc + (AHEAD - 1u) * SLICE < kBytes; kc += AHEAD * SLICE)
            {
                VecT v[AHEAD], xv[AHEAD];
#pragma unroll
                for(uint32_t u = 0; u < AHEAD; ++u)
                    v[u] = __builtin_bit_cast(VecT, __builtin_amdgcn_raw_buffer_load_b128(rows[0], mine, kc + u * SLICE, NT));
#pragma unroll
                for(uint32_t u = 0; u < AHEAD; ++u)
                    xv[u] = __builtin_bit_cast(VecT, __builtin_amdgcn_raw_buffer_load_b128(xr, mine, kc + u * SLICE, 0));
#pragma unroll
                for(uint32_t u = 0; u < AHEAD; ++u)
#pragma unroll
                    for(uint32_t e = 0; e < V; ++e)
                        acc[0] += v[u][e] * xv[u][e];
            }
        }
        for(; kc < kBytes; kc += SLICE)
        {
            const VecT xv = __builtin_bit_cast(VecT, __builtin_amdgcn_raw_buffer_load_b128(xr, mine, kc, 0));
            VecT       v  = __builtin_bit_cast(VecT, __builtin_amdgcn_raw_buffer_load_b128(rows[0], mine, kc, NT));
#pragma unroll
            for(uint32_t r = 0; r < RB; ++r)
            {
                __builtin_amdgcn_sched_barrier(0); // (keeps the next row's load behind this row's arithmetic)
#pragma unroll
                for(uint32_t e = 0; e < V; ++e)
                    acc[r] += v[e] * xv[e];
                __builtin_amdgcn_sched_barrier(0);
                if(r + 1u < RB)
                    v = __builtin_bit_cast(VecT, __builtin_amdgcn_raw_buffer_load_b128(rows[r + 1u], mine, kc, NT));
            }
        }
#pragma unroll
        for(uint32_t r = 0; r < RB; ++r)
        {
            T sum = acc[r];
#pragma unroll
            for(uint32_t off = 32; off > 0; off >>= 1)
                sum += __shfl_xor(sum, off, 64);
            if(lane == 0)
                partial[w][r] = sum;
        }
        __syncthreads();
        if(threadIdx.x < RB && row0 + threadIdx.x < m)
        {
            T sum = T(0);
#pragma unroll
            for(uint32_t i = 0; i < WAVES; ++i)
                sum += partial[i][threadIdx.x];
            const uint32_t row = row0 + threadIdx.x;
            if constexpr(SPLIT)
                yOut[(uint64_t)row * partRow + (uint64_t)blockIdx.x * partSplit] = sum;
            else
                yOut[row] = beta != T(0) ? alpha * sum + beta * yIn[row] : alpha * sum;
        }
    }

    // Lanes side by side on one column in the split form of the col-major kernel.  With K divided there are workgroups
    // enough whatever the rows per workgroup, so the runs can be longer than the plain kernel's.  Columns of 512 bytes and
    // more, up to 256 16-byte pieces: a wave takes whole kilobytes of a column, eight waves per workgroup (f32 256 x 262144,
    // 256 splits, first kernel alone: 0.89 of the HBM peak against 0.85 with 128-byte runs and sixteen waves; with sixteen
    // waves 0.72; 128 x 524288: 0.87 - 0.89 against 0.76); shorter columns: 256-byte runs (64 x 1048576: 0.81 against 0.74
    // and 0.58 - 0.67 with whole kilobytes); from 256 pieces per column on 512-byte runs and sixteen waves (1024 x 65536
    // 0.79 against 0.75 with 128-byte runs, 2048 x 32768 0.83 against 0.76, 16640 x 16384 0.83 against 0.65; 1 KiB runs:
    // 0.72, 0.78, 0.78).
    template <typename T>
    uint32_t splitRunLanes(uint32_t m, uint32_t k)
    {
        constexpr uint32_t V = 16u / sizeof(T);
        if(m >= 256u * V)
            return 32u;
        if(k < 128u * 1024u)
            return 8u; // too short for a workgroup per CU with one or two blocks of rows: many blocks of 32 rows (256 x 16384: 6 us against 13)
        return m >= 32u * V ? 64u : 16u;
    }

    // Splits of K for a shape, 1 = the plain kernels serve it.
    // Col-major A: a workgroup per block of 32 or 64 rows (f32) leaves CUs idle when the blocks are few, or just over a
    // multiple of the CU count (8256 rows: 258 blocks, two of them in a round of their own).  The plain launch is priced
    // as rounds over the CUs - a workgroup streams about 50 GB/s on its own, all CUs together 7.2 TB/s - and the split
    // form as A at 7.0 TB/s plus 3 us for the second launch; measured (f32): 4096^2 12.8 us plain / 13.3 split,
    // 4096 x 16384 42.4 / 40.2, 8256 x 8192 67.5 / 46.3, 12288 x 8192 77.0 / 60.0, 2048 x 32768 78.3 / 40.5,
    // 16640 x 16384 261 / 164, 20000 x 16384 274 / 185.  K is divided into pieces of at least 1024 columns so that two
    // (few rows) or eight (512-byte runs) workgroups per CU result, 256 pieces at most.
    // Row-major A with rows of 256 KiB or more, beyond the memory-side cache and fewer than 2048 of them, or at most half
    // as many as CUs: the plain kernels have a workgroup per row (up to 512 rows; too few workgroups below 256 rows, and
    // as many bytes of x as of A to read: 128 rows of 4 MiB 0.46 of the HBM peak, 256 rows of 2 MiB 0.75) or a wave per
    // row (1024 x 262144: 0.76); split, four rows share a workgroup and K is cut into pieces of 128 KiB (32 rows: 0.75,
    // 64 - 128: 0.82, 256: 0.86, 512: 0.87, 1024: 0.89).  From 2048 rows on the plain shared-row kernel does the same
    // without a workspace (2000 x 131072: 0.885 plain, 0.877 split).
    template <typename T>
    uint32_t gemvSplits(int32_t layout_a, uint32_t m, uint32_t k, uint32_t lda, uint32_t& kPer)
    {
        constexpr uint32_t V = 16u / sizeof(T);
        const uint32_t     cus = r355::computeUnits();
        kPer = k;
        uint32_t blocks, grain, perCu, align, rowsPerBlock;
        if(layout_a == R355_COL_MAJOR)
        {
            const uint32_t rows   = (m >= 16u * V * 256u ? 16u : 8u) * V; // per workgroup, as the plain launch chooses them
            const uint32_t plain  = (m + rows - 1u) / rows, rounds = (plain + cus - 1u) / cus;
            const double   bytes  = static_cast<double>(m) * k * sizeof(T), perGroup = static_cast<double>(rows) * k * sizeof(T);
            const double   abreast = static_cast<double>(plain < cus ? plain : cus) * perGroup / 7.2e6; // us: all of a round's workgroups at the HBM's rate
            const double   alone   = perGroup / 50.0e3; // us: a workgroup at its own
            // Columns that do not start on a 128-byte boundary (lda not a multiple of 32 f32): the runs of neighbouring blocks
            // of rows share cache lines, which then travel twice - the plain kernel's 128-byte runs take twice the time
            // (5000 x 16384: 93 us where 4096 x 16384 takes 42), runs of 512 bytes a quarter more.
            const bool     askew   = ((uint64_t)lda * sizeof(T)) % 128u != 0u;
            const uint32_t wide    = splitRunLanes<T>(m, k);
            const double   tPlain  = static_cast<double>(rounds) * (abreast > alone ? abreast : alone) * (askew ? 2.0 : 1.0);
            const double   tSplit  = (bytes / 7.0e6) * (askew ? 1.0 + 8.0 / wide : 1.0) + 3.0;
            if(rounds > 3u || tSplit * 1.03 >= tPlain) // (many rounds even out by themselves as workgroups end at different times)
                return 1u;
            const uint32_t lanes = splitRunLanes<T>(m, k);
            blocks = (m + lanes * V - 1u) / (lanes * V), grain = 1024u, perCu = lanes == 32u ? 8u : 2u;
            align  = lanes == 8u ? 1024u : 256u; // (a multiple of the columns one unrolled trip of the kernel covers)
            rowsPerBlock = lanes * V;
        }
        else
        {
            const uint64_t rowBytes = (uint64_t)k * sizeof(T);
            const bool     beyondCache = rowBytes * m > (256ull << 20); // (within the memory-side cache the plain kernels are 1 - 9 % ahead)
            if(rowBytes < (256u << 10) || rowBytes >= (1ull << 31) || !(m <= cus / 2u || (beyondCache && m < 2048u)))
                return 1u;
            const uint32_t piece = (128u << 10) / (uint32_t)sizeof(T); // pieces of 128 KiB, or the multiple of that which makes 256 of them
            kPer = piece * ((k + 256u * piece - 1u) / (256u * piece));
            return (k + kPer - 1u) / kPer;
        }
        // About perCu workgroups per CU - and of the counts around that the cheapest by a small model of the launch: the
        // workgroups are dealt out evenly over the CUs, all CUs together stream 7 TB/s, and the CUs that hold one workgroup
        // more than the others finish it at what is left of that or at the 50 GB/s a CU streams on its own.  8256 rows are 65
        // blocks, which eight splits turn into 520 workgroups - two per CU and a third on eight CUs - and seven into 455: 49.0
        // -> 43.9 us (0.69 -> 0.77 of the HBM peak; the model says 48.8 and 42.7); 12288 rows, 96 blocks, stay with eight
        // splits (768 workgroups: 60.1 us, model 57.5; five splits, 480 workgroups: 62.5, model 62.9); 16640 x 16384 takes
        // eleven (162.9 us, model 160.5) over sixteen (164.9, 163.8).
        uint32_t want = (perCu * cus + blocks - 1u) / blocks, most = k / grain < 256u ? k / grain : 256u;
        if(want > most)
            want = most;
        if(want < 2u)
            return 1u;
        uint32_t best = 0, bestPer = k;
        double   bestCost = 0.0;
        for(uint32_t t = want / 2u > 2u ? want / 2u : 2u; t <= most && t <= 2u * want; ++t)
        {
            const uint32_t per = ((k + t - 1u) / t + align - 1u) / align * align; // every split but the last is whole unrolled trips
            const uint32_t n = (k + per - 1u) / per, groups = blocks * n, each = groups / cus, over = groups % cus;
            const double   bytes = static_cast<double>(per) * rowsPerBlock * sizeof(T); // of a workgroup
            const double   left  = over ? 7.0e6 / over : 0.0; // bytes per us for each of the CUs with one more
            const double   cost  = static_cast<double>(each) * bytes * cus / 7.0e6 + (over ? bytes / (left < 50.0e3 ? left : 50.0e3) : 0.0);
            // (as cheap within 2 %: the larger count - smaller workgroups even out better than the model knows: 2048 x 32768,
            // 16 workgroups of 128 rows, 0.75 with 16 splits and 0.85 with 32, one and two workgroups per CU)
            if(n >= 2u && (best == 0u || cost < bestCost * 0.98 || (cost <= bestCost * 1.02 && n > best)))
            {
                bestCost = best == 0u || cost < bestCost ? cost : bestCost;
                best = n, bestPer = per;
            }
        }
        if(best < 2u)
            return 1u;
        kPer = bestPer;
        return best;
    }

    // Rows per workgroup of the batched shared-row kernel for a streamed row-major A with long rows and fewer than 2048
    // of them, 0 = another kernel serves it.  Four or two rows, the larger count whose workgroups load the CUs evenly:
    // at least five eighths of them in a single round, at least 80 % of the slots of several rounds (f32, rows of 512 KiB
    // and more, four / two / one row per workgroup: 256 rows 0.35 / 0.56 / 0.75, 384 rows 0.49 / 0.77 / 0.63, 512 rows
    // 0.61 / 0.86 / 0.77, 640 rows 0.71 / 0.63 / 0.68, 896 rows 0.86 / 0.81 / 0.71, 1152 rows 0.62 / 0.73 / 0.73, 1280
    // rows of 256 KiB 0.66 / 0.76 / 0.69, 1792 rows 0.83 / 0.80 / 0.71).
    inline uint32_t batchedRows(uint32_t m, bool stream, uint64_t rowBytes)
    {
        if(!stream || m >= 2048u || rowBytes < (256u << 10) || rowBytes >= (1ull << 31))
            return 0u;
        const uint32_t cus = r355::computeUnits();
        for(uint32_t rb = 4u; rb >= 2u; rb /= 2u)
        {
            const uint32_t groups = (m + rb - 1u) / rb, rounds = (groups + cus - 1u) / cus;
            if(rounds == 1u ? groups * 8u >= cus * 5u : (uint64_t)groups * 10u >= (uint64_t)rounds * cus * 8u)
                return rb;
        }
        return 0u;
    }

    template <typename T>
    int gemvLaunch(int32_t layout_a, uint32_t m, uint32_t k, const T* a, uint32_t lda, const T* x, const T* y_in, T* y_out,
                   T alpha, T beta, void* stream, void* workspace = nullptr, size_t workspaceBytes = 0)
    {
        constexpr uint32_t V = 16u / sizeof(T);
        if(!a || !x || !y_out || (beta != T(0) && !y_in))
            return r355::fail(R355_ERR_BAD_ARG, "gemv: null pointer");
        if(m == 0 || k == 0)
            return r355::fail(R355_ERR_BAD_ARG, "gemv: m and k must be non-zero");
        if(m % V || k % V)
            return r355::fail(R355_ERR_BAD_SIZE, "gemv: m=%u and k=%u must be multiples of %u", m, k, V);
        if(!r355::aligned(a, 16) || lda % V || !r355::aligned(x, 16) || !r355::aligned(y_out, 16))
            return r355::fail(R355_ERR_MISALIGNED, "gemv: a, x, y need 16-byte alignment and lda %% %u == 0", V);
        if(workspace && !r355::aligned(workspace, 16))
            return r355::fail(R355_ERR_MISALIGNED, "gemv: the workspace needs 16-byte alignment");
        hipStream_t s = static_cast<hipStream_t>(stream);
        r355::beginCall();
        // K split over several workgroups per block of rows when the shape calls for it and the workspace holds the partial sums
        uint32_t       kPer   = k;
        const uint32_t splits = (layout_a == R355_COL_MAJOR || layout_a == R355_ROW_MAJOR) && workspace ? gemvSplits<T>(layout_a, m, k, lda, kPer) : 1u;
        const bool     split  = splits > 1u && (uint64_t)splits * m * sizeof(T) <= workspaceBytes;
        T*             parts  = static_cast<T*>(workspace);
        const bool     byWave = splits >= 32u; // layout of the partial sums: [m][splits] for the wave-per-row reduction, else [splits][m]
        const uint32_t partRow = byWave ? splits : 1u, partSplit = byWave ? 1u : m;
        if(layout_a == R355_COL_MAJOR)
        {
            if(lda < m)
                return r355::fail(R355_ERR_BAD_ARG, "gemv: lda < m");
            const bool stream = (uint64_t)k * lda * sizeof(T) > (256ull << 20);
            auto       go     = [&](auto rl, auto waves) {
                constexpr uint32_t RL = decltype(rl)::value, ROWS = RL * V, WAVES = decltype(waves)::value;
                const dim3         grid((m + ROWS - 1u) / ROWS, split ? splits : 1u), block(WAVES * 64);
                if(split && stream)
                    hipLaunchKernelGGL((gemvColMajor<T, RL, WAVES, true, true>), grid, block, 0, s, m, k, a, lda, x, y_in, parts, alpha, beta, kPer, partRow, partSplit);
                else if(split)
                    hipLaunchKernelGGL((gemvColMajor<T, RL, WAVES, false, true>), grid, block, 0, s, m, k, a, lda, x, y_in, parts, alpha, beta, kPer, partRow, partSplit);
                else if(stream)
                    hipLaunchKernelGGL((gemvColMajor<T, RL, WAVES, true>), grid, block, 0, s, m, k, a, lda, x, y_in, y_out, alpha, beta, k, 0u, 0u);
                else
                    hipLaunchKernelGGL((gemvColMajor<T, RL, WAVES, false>), grid, block, 0, s, m, k, a, lda, x, y_in, y_out, alpha, beta, k, 0u, 0u);
            };
            // 256-byte runs once the rows give every CU a workgroup with them (8192^2 f32: 0.0415 ms against 0.0374 with
            // 128-byte runs and twice the workgroups; 16384^2: 0.151 against 0.161); sixteen waves per workgroup either way
            // (four: 0.0399 and 0.163)
            if(split && splitRunLanes<T>(m, k) == 32u)
                go(std::integral_constant<uint32_t, 32>{}, std::integral_constant<uint32_t, 16>{});
            else if(split && splitRunLanes<T>(m, k) == 64u)
                go(std::integral_constant<uint32_t, 64>{}, std::integral_constant<uint32_t, 8>{});
            else if(split && splitRunLanes<T>(m, k) == 16u)
                go(std::integral_constant<uint32_t, 16>{}, std::integral_constant<uint32_t, 8>{});
            else if(split)
                go(std::integral_constant<uint32_t, 8>{}, std::integral_constant<uint32_t, 16>{});
            else if(m >= 16u * V * 256u)
                go(std::integral_constant<uint32_t, 16>{}, std::integral_constant<uint32_t, 16>{});
            else
                go(std::integral_constant<uint32_t, 8>{}, std::integral_constant<uint32_t, 16>{});
        }
        else if(layout_a == R355_ROW_MAJOR)
        {
            if(lda < k)
                return r355::fail(R355_ERR_BAD_ARG, "gemv: lda < k");
            const dim3 grid((m + THREADS / 64 - 1) / (THREADS / 64));
            const bool     stream   = (uint64_t)m * lda * sizeof(T) > (256ull << 20);
            const uint64_t rowBytes = (uint64_t)k * sizeof(T);
            // rows of 16 KiB and more (f32, 1 GiB of A, against a wave per row: +1..2 % at 16 KiB, +4 % at 24 KiB, none at
            // 32 KiB, +5 % at 40 KiB, +7..11 % from 64 KiB on; 8 KiB rows lose 6 %), short enough for a 32-bit buffer
            // offset, and enough of them for two workgroups per CU
            // Few and very long rows leave a wave per row with a handful of waves on the whole chip: a workgroup of sixteen
            // waves per row instead (f32, 512 MiB of A: 512 rows 0.42 -> 0.64 of the HBM peak, 256 rows 0.23 -> 0.77, 128 rows
            // 0.12 -> 0.43; rows of 512 KiB: 640 rows 0.52 -> 0.67, 768 rows 0.61 -> 0.76, 896 rows even; a wave per row is
            // ahead again from there on, and from 768 rows of 128 or 256 KiB)
            if(split)
            {
                const dim3 grid(splits, (m + SHARED_ROWS - 1u) / SHARED_ROWS);
                if(stream)
                    hipLaunchKernelGGL((gemvRowMajorShared<T, 8, SHARED_ROWS, true, true>), grid, dim3(8 * 64), 0, s, m, k, a, lda, x, y_in, parts, alpha, beta, kPer, partRow, partSplit);
                else
                    hipLaunchKernelGGL((gemvRowMajorShared<T, 8, SHARED_ROWS, false, true>), grid, dim3(8 * 64), 0, s, m, k, a, lda, x, y_in, parts, alpha, beta, kPer, partRow, partSplit);
            }
            else if(const uint32_t rb = batchedRows(m, stream, rowBytes); rb != 0u)
            {
                const dim3 blocks((m + rb - 1u) / rb);
                if(rb == 4u)
                    hipLaunchKernelGGL((gemvRowMajorShared<T, 8, 4, true, false, true>), blocks, dim3(8 * 64), 0, s, m, k, a, lda, x, y_in, y_out, alpha, beta, k, 0u, 0u);
                else
                    hipLaunchKernelGGL((gemvRowMajorShared<T, 8, 2, true, false, true>), blocks, dim3(8 * 64), 0, s, m, k, a, lda, x, y_in, y_out, alpha, beta, k, 0u, 0u);
            }
            else if((m <= 512u || (m <= 768u && rowBytes >= (512u << 10))) && rowBytes >= (128u << 10) && rowBytes < (1ull << 31))
            {
                if(stream)
                    hipLaunchKernelGGL((gemvRowMajorShared<T, 16, 1, true>), dim3(m), dim3(16 * 64), 0, s, m, k, a, lda, x, y_in, y_out, alpha, beta, k, 0u, 0u);
                else
                    hipLaunchKernelGGL((gemvRowMajorShared<T, 16, 1, false>), dim3(m), dim3(16 * 64), 0, s, m, k, a, lda, x, y_in, y_out, alpha, beta, k, 0u, 0u);
            }
            else if(stream && rowBytes >= (16u << 10) && rowBytes < (1ull << 31) && m >= SHARED_ROWS * 512u)
            {
                const dim3 blocks((m + SHARED_ROWS - 1u) / SHARED_ROWS);
                if(rowBytes < (128u << 10))
                    hipLaunchKernelGGL((gemvRowMajorShared<T, 8>), blocks, dim3(8 * 64), 0, s, m, k, a, lda, x, y_in, y_out, alpha, beta, k, 0u, 0u);
                else
                    hipLaunchKernelGGL((gemvRowMajorShared<T, 16>), blocks, dim3(16 * 64), 0, s, m, k, a, lda, x, y_in, y_out, alpha, beta, k, 0u, 0u);
            }
            else if(stream)
                hipLaunchKernelGGL((gemvRowMajor<T, true>), grid, dim3(THREADS), 0, s, m, k, a, lda, x, y_in, y_out, alpha, beta);
            else
                hipLaunchKernelGGL((gemvRowMajor<T, false>), grid, dim3(THREADS), 0, s, m, k, a, lda, x, y_in, y_out, alpha, beta);
        }
        else
            return r355::fail(R355_ERR_BAD_ARG, "gemv: unknown layout");
        if(split && byWave)
            hipLaunchKernelGGL(gemvAddSplitsByWave<T>, dim3((m + THREADS / 64u - 1u) / (THREADS / 64u)), dim3(THREADS), 0, s, m, splits, parts, y_in, y_out, alpha, beta);
        else if(split)
            hipLaunchKernelGGL(gemvAddSplits<T>, dim3((m + THREADS - 1u) / THREADS), dim3(THREADS), 0, s, m, splits, parts, y_in, y_out, alpha, beta);
        return r355::checkLaunch("gemv");
    }
} // namespace

extern "C" size_t r355_gemv_workspace_bytes(int32_t layout_a, uint32_t m, uint32_t k, uint32_t elem_bytes)
{
    if((layout_a != R355_COL_MAJOR && layout_a != R355_ROW_MAJOR) || m == 0 || k == 0)
        return 0;
    uint32_t       kPer   = k;
    const uint32_t splits = elem_bytes == 8u ? gemvSplits<double>(layout_a, m, k, layout_a == R355_COL_MAJOR ? m : k, kPer) : gemvSplits<float>(layout_a, m, k, layout_a == R355_COL_MAJOR ? m : k, kPer);
    return splits > 1u ? (size_t)splits * m * (elem_bytes == 8u ? 8u : 4u) : 0;
}

extern "C" int r355_gemv_ws(int32_t layout_a, uint32_t m, uint32_t k, const float* a, uint32_t lda, const float* x,
                            const float* y_in, float* y_out, float alpha, float beta, void* workspace, size_t workspace_bytes, void* stream)
{
    return gemvLaunch<float>(layout_a, m, k, a, lda, x, y_in, y_out, alpha, beta, stream, workspace, workspace_bytes);
}

extern "C" int r355_dgemv_ws(int32_t layout_a, uint32_t m, uint32_t k, const double* a, uint32_t lda, const double* x,
                             const double* y_in, double* y_out, double alpha, double beta, void* workspace, size_t workspace_bytes, void* stream)
{
    return gemvLaunch<double>(layout_a, m, k, a, lda, x, y_in, y_out, alpha, beta, stream, workspace, workspace_bytes);
}

extern "C" int r355_gemv(int32_t layout_a, uint32_t m, uint32_t k, const float* a, uint32_t lda, const float* x,
                         const float* y_in, float* y_out, float alpha, float beta, void* stream)
{
    return gemvLaunch<float>(layout_a, m, k, a, lda, x, y_in, y_out, alpha, beta, stream);
}

extern "C" int r355_dgemv(int32_t layout_a, uint32_t m, uint32_t k, const double* a, uint32_t lda, const double* x,
                          const double* y_in, double* y_out, double alpha, double beta, void* stream)
{
    return gemvLaunch<double>(layout_a, m, k, a, lda, x, y_in, y_out, alpha, beta, stream);
}
