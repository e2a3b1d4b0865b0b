// DLRM dot-interaction forward and backward for gfx950.
//
// Forward takes the place of test/dlrm/device/dlrm_dot_fwd.hpp:35-138 (and the LDS variant
// dlrm_dot_fwd_lds.hpp:35-190, samples/simple_dlrm.cpp:184-284).  The reference gives each
// wave one 16x16 tile of X X^T, stores f32 tiles to a global scratch `acc[b][m][m]` and
// re-reads them to scatter the lower triangle.  This path is HBM-bound (about 24 flop per
// byte), so the kernel is organised around memory traffic instead:
//
//   * one wave owns one sample at a time; a workgroup (4 waves) owns 8 consecutive samples,
//     whose outputs form one contiguous, 16-byte aligned run of 8 * (k + m(m-1)/2) elements;
//   * X (m x k, m <= 32) is read once with fully coalesced 128-bit loads (both samples of a
//     wave are requested before either is consumed), parked in LDS with a per-row XOR swizzle,
//     and fed to v_mfma_f32_32x32x16 with the same register as both operands (X X^T): k / 16
//     matrix instructions, one 128-bit LDS read each; lanes of rows >= m feed zeros, which is
//     the 27 -> 32 padding;
//   * the strict lower triangle and the copied first row are assembled in an LDS image of
//     the output and leave with coalesced 128-bit stores.  No global scratch;
//   * up to 16 features, "one sample" above is a block of several consecutive samples, whose
//     rows are contiguous in memory: the products across samples are computed and dropped.
//
// f32 has kernels of its own on v_mfma_f32_16x16x4_f32 (an LDS image of X, or the matrix
// instructions fed straight from the global loads: see dlrmFwdF32Kernel, dlrmFwdF32Direct).
//
// Backward takes the place of test/dlrm/device/dlrm_dot_bwd.hpp:35-176: the symmetric matrix
// of the upstream triangle (trilReconstruct) is formed directly as a matrix-instruction operand
// and multiplied into X, read from LDS with transposing reads, again without global scratch.
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace
{
    using f32x16 = float __attribute__((ext_vector_type(16)));
    using i32x4  = int __attribute__((ext_vector_type(4)));
    using f16x8  = _Float16 __attribute__((ext_vector_type(8)));
    using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));

    constexpr uint32_t WAVES          = 4;
    constexpr uint32_t THREADS        = WAVES * 64;
    constexpr uint32_t SAMPLES_PER_WG = 8; // 8 * out_row_bytes is a multiple of 16 for every (m, k)
    constexpr uint32_t MAX_M          = 32;
    constexpr uint32_t MAX_K          = 256;

    template <bool BF16>
    __device__ inline f32x16 mfma16(f32x16 acc, i32x4 x, i32x4 y)
    {
        if constexpr(BF16)
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8, x), __builtin_bit_cast(bf16x8, y), acc, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_f32_32x32x16_f16(
                __builtin_bit_cast(f16x8, x), __builtin_bit_cast(f16x8, y), acc, 0, 0, 0);
    }

    template <bool BF16>
    __device__ inline uint16_t roundOut(float v)
    {
        if constexpr(BF16)
            return __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
        else
            return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
    }

    // A run of `bytes` bytes at base + offset (wave-uniform) as a raw buffer: a lane whose offset lies beyond it loads zeros
    // (stores nothing) without touching memory.  Loads and stores through it need no branches, so every vector-memory
    // instruction is issued on every path and the compiler can count them: the wait for one sample's loads then leaves
    // the next sample's loads and the previous sample's stores in flight.  (With a branch around each guarded access the
    // number of younger operations is unknown and every wait becomes "until nothing is outstanding".)
    __device__ inline __amdgpu_buffer_rsrc_t runBuffer(const void* base, uint64_t offset, uint32_t bytes)
    {
        const uint64_t addr = reinterpret_cast<uint64_t>(base) + offset;
        const uint32_t lo   = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr));
        const uint32_t hi   = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(addr >> 32));
        return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>((static_cast<uint64_t>(hi) << 32) | lo), 0,
                                                 static_cast<int>(__builtin_amdgcn_readfirstlane(bytes)), 0x00020000);
    }
    // cache-policy bits of the raw buffer builtins (2 = nt): X, the upstream gradient and the results are touched once.
    // Measurement builds (python -m rocwmma_amd.build --variant <name> -D...): R355_DLRM_PLAIN_LOADS / R355_DLRM_PLAIN_STORES
    // take the default policy instead.
#if defined(R355_DLRM_PLAIN_LOADS)
    constexpr int LOAD_POLICY = 0;
#elif defined(R355_DLRM_LOAD_POLICY)
    constexpr int LOAD_POLICY = R355_DLRM_LOAD_POLICY;
#else
    constexpr int LOAD_POLICY = 2;
#endif
#ifdef R355_DLRM_PLAIN_STORES
    constexpr int STORE_POLICY = 0;
#else
#ifdef R355_DLRM_STORE_POLICY
    constexpr int STORE_POLICY = R355_DLRM_STORE_POLICY;
#else
    constexpr int STORE_POLICY = 2;
#endif
#endif
    // 128-bit stores of whole runs of output (a workgroup's output rows, a sample's gradient rows) go through a raw buffer
    // of the run's bytes with cache-policy bits of their own: 16 = sc1, device scope, measured against nt (2) at a batch of
    // 65536 - f32 forward 27 x 128 0.1747 -> 0.1651 ms, f16 forward 0.0833 -> 0.0823, 8 x 64 forward / backward + 3 / + 2 %,
    // the 27 x 128 backward kernels unchanged.  (The 4-byte stores of the kernels that store a row per wave lose 10 % with
    // it and stay nt.)  -DR355_DLRM_RUN_POLICY=<bits> builds another choice.
#if defined(R355_DLRM_PLAIN_STORES)
    constexpr int RUN_POLICY = 0;
#elif defined(R355_DLRM_RUN_POLICY)
    constexpr int RUN_POLICY = R355_DLRM_RUN_POLICY;
#else
    constexpr int RUN_POLICY = 16;
#endif
    template <typename V>
    __device__ __forceinline__ void runStore(const V& v, __amdgpu_buffer_rsrc_t run, uint32_t byteOffset)
    {
        using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
        static_assert(sizeof(V) == 16, "128-bit pieces");
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), run, byteOffset, 0, RUN_POLICY);
    }

    // K is a template parameter (32, 64, 128, 256): rows of X are K * 2 bytes = K / 8 chunks.
    // ROWS (28 or 32) bounds m: the LDS image of a sample holds ROWS rows, which at m <= 28 and
    // K = 128 lets four workgroups share a CU instead of three.
    // Few features: `pack` consecutive samples (pack * m <= ROWS rows, contiguous in memory) are taken as one block of
    // rows.  The Gram matrix of the stacked rows holds each sample's own on its diagonal - the products across samples are
    // computed and dropped - so loads, LDS image and matrix instructions are those of one large sample, and a workgroup's
    // 8 * pack output rows are still one run of bytes.  (m = 8, k = 128 at a batch of 65536: four samples per block.)
    template <bool BF16, uint32_t K, uint32_t ROWS>
    __global__ void __launch_bounds__(THREADS)
        dlrmFwdKernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out, uint32_t m, uint32_t batch, uint32_t pack)
    {
        constexpr uint32_t ROW_CHUNKS = K / 8; // 16-byte chunks per row
        constexpr uint32_t X_BYTES    = ROWS * K * 2; // LDS image of one sample
        constexpr uint32_t MAX_OUT    = K + ROWS * (ROWS - 1) / 2;

        __shared__ __attribute__((aligned(16))) char     xLds[WAVES][X_BYTES];
        __shared__ __attribute__((aligned(16))) uint16_t outLds[SAMPLES_PER_WG * MAX_OUT + 8];

        const uint32_t tid       = threadIdx.x;
        const uint32_t lane      = tid & 63u;
        const uint32_t wave      = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t outStride = K + m * (m - 1) / 2; // elements per sample
        const uint32_t b0        = blockIdx.x * SAMPLES_PER_WG * pack;
        const uint32_t inBytes   = m * K * 2u; // of one sample
        const uint32_t rows      = m * pack; // of one block
        const uint32_t rcpM      = (65536u + m - 1u) / m; // i / m == (i * rcpM) >> 16 for i < 32

        char* xw = xLds[wave];
        // rows m..31 of the 32 x 32 product are padding: their lanes feed zeros (see below)

        // (Tried and dropped: two groups of 8 samples per workgroup with the next group's loads in flight during compute
        // and copy-out - the compiler then keeps 137 instead of 85 registers at k = 128, three workgroups per CU instead
        // of four, 0.0852 against 0.0823 ms at a batch of 65536; and the copy-out through a raw buffer - the same at
        // k <= 128, 0.162 against 0.155 ms at k = 256.)
        // Both samples of this wave are requested from HBM before either is consumed: the kernel is
        // bandwidth-bound, and bytes in flight per CU are what keeps HBM busy.  The loads go through a raw buffer of
        // exactly the sample's bytes (runBuffer; none for a sample beyond the batch), so the first sample is consumed
        // while the second is still arriving.
        constexpr uint32_t PER_WAVE   = SAMPLES_PER_WG / WAVES; // 2
        constexpr uint32_t MAX_CHUNKS = (ROWS * ROW_CHUNKS + 63u) / 64u; // loads per lane per sample
        i32x4              stash[PER_WAVE][MAX_CHUNKS];
#pragma unroll
        for(uint32_t q = 0; q < PER_WAVE; ++q)
        {
            const uint32_t b   = b0 + (wave + q * WAVES) * pack; // the block's first sample
            const uint32_t has = b < batch ? (batch - b < pack ? batch - b : pack) : 0u;
            const auto     src = runBuffer(in, (uint64_t)(has ? b : 0u) * inBytes, has * inBytes);
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
                stash[q][j] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(src, (j * 64u + lane) * 16u, 0, LOAD_POLICY)); // read once
        }

#pragma unroll
        for(uint32_t q = 0; q < PER_WAVE; ++q)
        {
            const uint32_t sIdx = wave + q * WAVES;
            const uint32_t b    = b0 + sIdx * pack;
            if(b >= batch)
                break;
            // ---- X -> LDS: chunk c of the sample goes to row c / ROW_CHUNKS, slot (c % ROW_CHUNKS) ^ (row % 16)
            // (chunks of rows m .. ROWS - 1 arrived as zeros and are written like the others: those rows are never used)
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < ROWS * ROW_CHUNKS)
                {
                    const uint32_t row  = c / ROW_CHUNKS, col = c % ROW_CHUNKS;
                    const uint32_t slot = col ^ (row & (ROW_CHUNKS - 1u) & 15u);
                    *reinterpret_cast<i32x4*>(xw + (row * ROW_CHUNKS + slot) * 16u) = stash[q][j];
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this wave's LDS writes are done
            __builtin_amdgcn_wave_barrier();

            // ---- Gram matrix: acc(i, j) = sum_k X(i, k) X(j, k)
            f32x16         acc   = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            const bool     valid = (lane & 31u) < rows;
            const uint32_t row   = valid ? (lane & 31u) : 0u; // padding lanes read row 0 and discard it
#pragma unroll
            for(uint32_t s = 0; s < K / 16; ++s)
            {
                const uint32_t col  = 2u * s + (lane >> 5);
                const uint32_t slot = col ^ (row & (ROW_CHUNKS - 1u) & 15u);
                i32x4          x    = *reinterpret_cast<const i32x4*>(xw + (row * ROW_CHUNKS + slot) * 16u);
                if(!valid)
                    x = i32x4{0, 0, 0, 0};
                acc = mfma16<BF16>(acc, x, x);
            }

            // ---- output image: first row, then strict lower triangle (i, j < i) row-major
            uint16_t* o = outLds + sIdx * pack * outStride; // the block's samples one after the other
            for(uint32_t e = lane; e < pack * K; e += 64)
            {
                const uint32_t s = e / K, c = e % K, row = s * m; // a sample's first row is the head of its output row
                const uint32_t slot = (c / 8u) ^ (row & (ROW_CHUNKS - 1u) & 15u);
                o[s * outStride + c] = reinterpret_cast<const uint16_t*>(xw)[(row * ROW_CHUNKS + slot) * 8u + c % 8u];
            }
            const uint32_t j = lane & 31u, sj = (j * rcpM) >> 16, lj = j - sj * m;
#pragma unroll
            for(uint32_t r = 0; r < 16; ++r)
            {
                const uint32_t i = 8u * (r >> 2) + 4u * (lane >> 5) + (r & 3u);
                const uint32_t si = (i * rcpM) >> 16, li = i - si * m; // sample within the block, row within the sample
                if(si == sj && lj < li && i < rows)
                    o[si * outStride + K + li * (li - 1u) / 2u + lj] = roundOut<BF16>(acc[r]);
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
        }
        __syncthreads();

        // ---- coalesced copy-out of the workgroup's samples
        const uint32_t nSamples = (batch - b0) < SAMPLES_PER_WG * pack ? (batch - b0) : SAMPLES_PER_WG * pack;
        const uint32_t total    = nSamples * outStride; // elements
        uint16_t*      dst      = out + (uint64_t)b0 * outStride;
        const uint32_t vecs     = total / 8u;
        const auto run = runBuffer(dst, 0u, vecs * 16u);
        for(uint32_t v = tid; v < vecs; v += THREADS)
            runStore(reinterpret_cast<const i32x4*>(outLds)[v], run, v * 16u);
        for(uint32_t e = vecs * 8u + tid; e < total; e += THREADS)
            dst[e] = outLds[e];
    }

    // f32 variant.  An f32 sample is 13.8 KB, so only a few fit in LDS per CU and the matrix core
    // (v_mfma_f32_16x16x4_f32, 96 instructions per sample) is busy a good third of the time.  A wave walks the samples
    // first, first + stride, ... (stride = the launch's waves); a sample's loads are requested as soon as the sample two
    // steps before has been unloaded from its register stash into LDS, and each result row leaves from the wave's own
    // LDS image with coalesced 4-byte stores (a sample's output row is only 4-byte aligned) that are still in flight when
    // the next sample is taken up.  The launch gives every wave F32_STEPS samples: two workgroups share a CU and the
    // older one is served first, so with long walks (one launch-wide round of workgroups) the first half of the
    // workgroups finished after 135 us of 198 and the others ran the rest of the time alone, one wave per SIMD with
    // nothing to overlap its phases; short walks let the dispatcher refill a CU as soon as a workgroup ends
    // (0.196 ms with 32 samples per wave, 0.183 with 4, 0.178 with 2 at a batch of 65536).
    constexpr uint32_t F32_STEPS = 2;

    template <uint32_t K, uint32_t ROWS>
    __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2)))
        dlrmFwdF32Kernel(const float* __restrict__ in, float* __restrict__ out, uint32_t m, uint32_t batch)
    {
        constexpr uint32_t ROW_CHUNKS = K / 4; // 16-byte chunks per row
        constexpr uint32_t MAX_OUT    = K + ROWS * (ROWS - 1) / 2;
        constexpr uint32_t OUT_STEPS  = (MAX_OUT + 63u) / 64u; // 4-byte stores per lane and sample
        constexpr uint32_t MAX_CHUNKS = (ROWS * ROW_CHUNKS + 63u) / 64u;
        // Rows of the LDS image are one chunk longer than the data: (K + 4) / 4 is odd, so the 16 rows x 4 k values that
        // one operand read touches fall into 64 different banks, and a row's chunks keep their order (every read and
        // write of the image is one lane address plus a constant).
        constexpr uint32_t ROWP       = K * 4u + 16u;
        using f32x4                   = float __attribute__((ext_vector_type(4)));

        __shared__ __attribute__((aligned(16))) char  xLds[WAVES][ROWS * ROWP];
        __shared__ __attribute__((aligned(16))) float outLds[WAVES][OUT_STEPS * 64u];

        const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t outStride = K + m * (m - 1) / 2;
        const uint32_t inBytes   = m * K * 4u;
        // a wave walks the samples first, first + stride, ...: what the four waves of a workgroup request at one time is
        // one run of consecutive bytes
        const uint32_t first = blockIdx.x * WAVES + wave, stride = gridDim.x * WAVES;
        char*          xw        = xLds[wave];
        float*         o         = outLds[wave];

        // Two register stashes, used in turn: the loads of the next two samples are in flight while one is computed
        // (a wave holds 2 x 13.8 KB in flight, a CU's eight waves 220 KB).  One stash where two would not fit the 256
        // registers that two waves per SIMD leave each wave (32 rows of 128).
        constexpr bool TWO = MAX_CHUNKS < 16u;
        // (a sample beyond the batch is a buffer of no bytes: the loads are issued and move nothing)
        f32x4 stashA[MAX_CHUNKS], stashB[MAX_CHUNKS];
        auto  request = [&](f32x4 (&stash)[MAX_CHUNKS], uint64_t b) {
            const bool valid = b < batch;
            const auto src   = runBuffer(in, (uint64_t)(valid ? b : 0u) * inBytes, valid ? inBytes : 0u);
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
                stash[j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(src, (j * 64u + lane) * 16u, 0, LOAD_POLICY));
        };
        // sample b from its stash, which then takes the sample two steps further on
        auto process = [&](f32x4 (&stash)[MAX_CHUNKS], uint64_t b) {
            // chunks of rows m .. ROWS - 1 arrive as zeros and are written like the others: those rows are never used
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < ROWS * ROW_CHUNKS)
                {
                    const uint32_t row = c / ROW_CHUNKS, col = c % ROW_CHUNKS;
                    *reinterpret_cast<f32x4*>(xw + row * ROWP + col * 16u) = stash[j];
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
            request(stash, b + (TWO ? 2u : 1u) * stride); // the stash is free again

            // v_mfma_f32_16x16x4_f32 on the three 16 x 16 blocks of the Gram matrix that hold its lower
            // triangle (rows < 16 x rows < 16, rows >= 16 x rows < 16, rows >= 16 x rows >= 16): a quarter
            // fewer matrix-core cycles than the full 32 x 32 product, and three independent accumulator
            // chains keep the pipeline full.  Lane l feeds row l % 16 (+ 16) at k = 4 s + l / 16.
            using f32x4acc = float __attribute__((ext_vector_type(4)));
            f32x4acc       accLL = {0, 0, 0, 0}, accHL = accLL, accHH = accLL;
            const uint32_t r16 = lane & 15u, kq = lane >> 4;
            const bool     validLo = r16 < m, validHi = 16u + r16 < m;
            const uint32_t rowLo = validLo ? r16 : 0u, rowHi = validHi ? 16u + r16 : 0u;
            // eight steps of k (24 matrix instructions, 768 matrix-core clocks) per group; a group's 16 operand reads are
            // issued before the previous group's matrix instructions, so what the reads wait for in the LDS queue (the
            // other waves' 16-byte writes take 13 clocks each) is not what the matrix core waits for
            constexpr uint32_t GROUP = (ROWS > 28u && K > 64u) ? 4u : 8u, GROUPS = K / 4 / GROUP; // (registers: two waves per SIMD)
            float              xl[2][GROUP], xh[2][GROUP];
            auto fetch = [&](uint32_t grp, float (&lo)[GROUP], float (&hi)[GROUP]) {
#pragma unroll
                for(uint32_t u = 0; u < GROUP; ++u)
                {
                    const uint32_t s = grp * GROUP + u;
                    lo[u] = *reinterpret_cast<const float*>(xw + rowLo * ROWP + kq * 4u + s * 16u);
                    hi[u] = *reinterpret_cast<const float*>(xw + rowHi * ROWP + kq * 4u + s * 16u);
                }
            };
            fetch(0, xl[0], xh[0]);
#pragma unroll
            for(uint32_t grp = 0; grp < GROUPS; ++grp)
            {
                if(grp + 1u < GROUPS)
                    fetch(grp + 1u, xl[(grp + 1u) & 1u], xh[(grp + 1u) & 1u]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for(uint32_t u = 0; u < GROUP; ++u)
                {
                    const float lo = validLo ? xl[grp & 1u][u] : 0.0f, hi = validHi ? xh[grp & 1u][u] : 0.0f;
                    accLL          = __builtin_amdgcn_mfma_f32_16x16x4f32(lo, lo, accLL, 0, 0, 0);
                    accHL          = __builtin_amdgcn_mfma_f32_16x16x4f32(hi, lo, accHL, 0, 0, 0);
                    accHH          = __builtin_amdgcn_mfma_f32_16x16x4f32(hi, hi, accHH, 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }

            for(uint32_t e = lane; e < K; e += 64)
                o[e] = reinterpret_cast<const float*>(xw)[e]; // row 0
            // a 16 x 16 result block: lane holds rows 4 (lane / 16) + e, column lane % 16
#pragma unroll
            for(uint32_t e = 0; e < 4; ++e)
            {
                const uint32_t i = 4u * kq + e, j = r16;
                if(j < i && i < m)
                    o[K + i * (i - 1u) / 2u + j] = accLL[e];
                const uint32_t ih = 16u + i;
                if(ih < m)
                {
                    o[K + ih * (ih - 1u) / 2u + j] = accHL[e];
                    if(j < i)
                        o[K + ih * (ih - 1u) / 2u + 16u + j] = accHH[e];
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
            const auto dst = runBuffer(out, (uint64_t)(b < batch ? b : 0u) * outStride * 4u, b < batch ? outStride * 4u : 0u);
#pragma unroll
            for(uint32_t e = 0; e < OUT_STEPS; ++e)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, o[e * 64u + lane]), dst, (e * 64u + lane) * 4u, 0, STORE_POLICY);
            __builtin_amdgcn_s_waitcnt(0xC07F); // the image is rewritten by the next sample
            __builtin_amdgcn_wave_barrier();
        };

        // The first two samples stand outside the loop so that the loop is entered with the same operations in flight
        // as its own trips leave behind (loads, stores, loads, stores): the waits inside are then exact on both paths.
        // (A sample index is 64-bit here: the walk looks two steps beyond the batch.)
        if(first >= batch)
            return;
        request(stashA, first);
        if constexpr(TWO)
        {
            request(stashB, (uint64_t)first + stride);
            process(stashA, first);
            process(stashB, (uint64_t)first + stride);
#pragma unroll 1
            for(uint64_t b = (uint64_t)first + 2u * stride; b < batch; b += 2u * stride)
            {
                process(stashA, b);
                process(stashB, b + stride);
            }
        }
        else
        {
            process(stashA, first);
#pragma unroll 1
            for(uint64_t b = (uint64_t)first + stride; b < batch; b += stride)
                process(stashA, b);
        }
    }

    // f32 forward, k = 64 or 128: a workgroup owns 8 consecutive samples, as in the 16-bit kernel, and their output rows - one
    // run of 8 (k + m (m - 1) / 2) floats, a whole number of 16-byte pieces that starts on one - leave together with
    // 128-bit stores.  (A wave that stores its own sample's row writes 4-byte pieces of a row that starts anywhere: every
    // store instruction and every sample ends inside a cache line that another instruction or wave completes later; taking
    // the stores out of that kernel took a quarter of its time with them, for an eighth of its bytes.)
    // A sample of 128 columns passes through the wave's LDS image in two halves of 64 that accumulate into the same three
    // blocks, each half with a register stash of its own that is requested again (the same half of the wave's second
    // sample) as soon as it has been unloaded: the image of half a sample leaves the LDS for the eight output rows.
    // Rows from m on lie beyond the sample's buffer and cost no traffic, so the time follows m (the matrix work does not).
    template <uint32_t K, uint32_t ROWS>
    __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(ROWS <= 28u ? 3 : 2)))
        dlrmFwdF32Run(const float* __restrict__ in, float* __restrict__ out, uint32_t m, uint32_t batch)
    {
        constexpr uint32_t KH = 64u, HALVES = K / KH; // columns of a half, halves of a sample
        static_assert(K == 64u || K == 128u, "one or two halves");
        constexpr uint32_t ROW_CHUNKS = KH / 4u; // 16-byte chunks per row of a half
        constexpr uint32_t MAX_OUT    = K + ROWS * (ROWS - 1) / 2;
        constexpr uint32_t CHUNKS     = ROWS * ROW_CHUNKS / 64u; // loads per lane and half (ROWS * 16 is a multiple of 64)
        constexpr uint32_t ROWP       = KH * 4u + 16u; // rows one chunk longer than the data: (KH + 4) / 4 is odd (see dlrmFwdF32Kernel)
        constexpr uint32_t PER_WAVE   = SAMPLES_PER_WG / WAVES; // 2
        using f32x4                   = float __attribute__((ext_vector_type(4)));
        static_assert(ROWS * ROW_CHUNKS % 64u == 0u, "whole load instructions");

        __shared__ __attribute__((aligned(16))) char  xLds[WAVES][ROWS * ROWP];
        __shared__ __attribute__((aligned(16))) float outLds[SAMPLES_PER_WG * MAX_OUT + 4u];

        const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t outStride = K + m * (m - 1) / 2;
        const uint32_t inBytes   = m * K * 4u;
        const uint32_t b0        = blockIdx.x * SAMPLES_PER_WG;
        char*          xw = xLds[wave];
        const uint32_t r16 = lane & 15u, kq = lane >> 4;
        const bool     validLo = r16 < m, validHi = 16u + r16 < m;
        const uint32_t rowLo = validLo ? r16 : 0u, rowHi = validHi ? 16u + r16 : 0u;

        f32x4 stash[HALVES][CHUNKS];
        // (a sample beyond the batch is a buffer of no bytes: the loads are issued and move nothing)
        auto request = [&](uint32_t h, uint32_t b) {
            const bool valid = b < batch;
            const auto src   = runBuffer(in, (uint64_t)(valid ? b : 0u) * inBytes, valid ? inBytes : 0u);
#pragma unroll
            for(uint32_t j = 0; j < CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                stash[h][j]      = __builtin_bit_cast(
                    f32x4, __builtin_amdgcn_raw_buffer_load_b128(src, (c / ROW_CHUNKS) * (K * 4u) + h * (KH * 4u) + (c % ROW_CHUNKS) * 16u, 0, LOAD_POLICY));
            }
        };
#pragma unroll
        for(uint32_t h = 0; h < HALVES; ++h)
            request(h, b0 + wave);
#pragma unroll
        for(uint32_t q = 0; q < PER_WAVE; ++q)
        {
            const uint32_t sIdx = wave + q * WAVES, b = b0 + sIdx;
            float*         o    = outLds + sIdx * outStride;
            f32x4 accLL = {0, 0, 0, 0}, accHL = accLL, accHH = accLL;
#pragma unroll
            for(uint32_t h = 0; h < HALVES; ++h)
            {
                // chunks of rows m .. ROWS - 1 arrive as zeros and are written like the others: those rows are never used
#pragma unroll
                for(uint32_t j = 0; j < CHUNKS; ++j)
                {
                    const uint32_t c = j * 64u + lane;
                    *reinterpret_cast<f32x4*>(xw + (c / ROW_CHUNKS) * ROWP + (c % ROW_CHUNKS) * 16u) = stash[h][j];
                }
                __builtin_amdgcn_s_waitcnt(0xC07F);
                __builtin_amdgcn_wave_barrier();
                if(q + 1u < PER_WAVE)
                    request(h, b + WAVES); // this half's stash is free again: the wave's second sample

                // lane l feeds row l % 16 (+ 16) at k = 4 s + l / 16; a group's operand reads are issued before the
                // previous group's matrix instructions (see dlrmFwdF32Kernel)
                constexpr uint32_t GROUP = 4u, GROUPS = KH / 4u / GROUP;
                float              xl[2][GROUP], xh[2][GROUP];
                auto fetch = [&](uint32_t grp, float (&lo)[GROUP], float (&hi)[GROUP]) {
#pragma unroll
                    for(uint32_t u = 0; u < GROUP; ++u)
                    {
                        const uint32_t st = grp * GROUP + u;
                        lo[u] = *reinterpret_cast<const float*>(xw + rowLo * ROWP + kq * 4u + st * 16u);
                        hi[u] = *reinterpret_cast<const float*>(xw + rowHi * ROWP + kq * 4u + st * 16u);
                    }
                };
                fetch(0, xl[0], xh[0]);
#pragma unroll
                for(uint32_t grp = 0; grp < GROUPS; ++grp)
                {
                    if(grp + 1u < GROUPS)
                        fetch(grp + 1u, xl[(grp + 1u) & 1u], xh[(grp + 1u) & 1u]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for(uint32_t u = 0; u < GROUP; ++u)
                    {
                        const float lo = validLo ? xl[grp & 1u][u] : 0.0f, hi = validHi ? xh[grp & 1u][u] : 0.0f;
                        accLL          = __builtin_amdgcn_mfma_f32_16x16x4f32(lo, lo, accLL, 0, 0, 0);
                        accHL          = __builtin_amdgcn_mfma_f32_16x16x4f32(hi, lo, accHL, 0, 0, 0);
                        accHH          = __builtin_amdgcn_mfma_f32_16x16x4f32(hi, hi, accHH, 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                if(b < batch)
                    o[h * KH + lane] = reinterpret_cast<const float*>(xw)[lane]; // row 0: 64 values of this half
                __builtin_amdgcn_s_waitcnt(0xC07F);
                __builtin_amdgcn_wave_barrier(); // every read of this half has returned: the image takes the next one
            }
            // a 16 x 16 result block: lane holds rows 4 (lane / 16) + e, column lane % 16
            if(b < batch)
#pragma unroll
                for(uint32_t e = 0; e < 4; ++e)
                {
                    const uint32_t i = 4u * kq + e, j = r16;
                    if(j < i && i < m)
                        o[K + i * (i - 1u) / 2u + j] = accLL[e];
                    const uint32_t ih = 16u + i;
                    if(ih < m)
                    {
                        o[K + ih * (ih - 1u) / 2u + j] = accHL[e];
                        if(j < i)
                            o[K + ih * (ih - 1u) / 2u + 16u + j] = accHH[e];
                    }
                }
        }
        __syncthreads();

        // ---- coalesced copy-out of the workgroup's samples
        const uint32_t nSamples = (batch - b0) < SAMPLES_PER_WG ? (batch - b0) : SAMPLES_PER_WG;
        const uint32_t total    = nSamples * outStride; // floats
        float*         dst      = out + (uint64_t)b0 * outStride;
        const uint32_t vecs     = total / 4u;
        const auto run = runBuffer(dst, 0u, vecs * 16u);
        for(uint32_t v = tid; v < vecs; v += THREADS)
            runStore(reinterpret_cast<const f32x4*>(outLds)[v], run, v * 16u);
        for(uint32_t e = vecs * 4u + tid; e < total; e += THREADS)
            dst[e] = outLds[e];
    }

    // f32 forward with the matrix instructions fed straight from the global loads: no LDS image of X.  Both operands of
    // v_mfma_f32_16x16x4_f32 hold, in lane l, row l % 16 of a block of rows at k index l / 16 - and which four values of k
    // one instruction sums is free as long as A and B agree.  Lane l therefore loads, for j = 0 .. K / 16 - 1, the 16
    // bytes X[l % 16][16 j + 4 (l / 16) ...] (and, HIGH, the same of row 16 + l % 16; rows from m on lie beyond the
    // sample's buffer and arrive as zeros), and instruction t of step j takes element t of those vectors: it sums
    // k = 16 j + 4 q + t over q.  The registers the loads arrive in are the operand file of the matrix instructions, and
    // the next sample is requested into them as soon as those have issued.  What stays in LDS is the image of the output
    // row, so registers set the occupancy (eight waves per SIMD up to 16 features, four beyond).
    // Every lane's 16 bytes are a memory access of their own here (neighbouring lanes are a row apart), and the other
    // half of each cache line comes with the next instruction: ordinary loads, which keep the line for it, not streaming
    // ones (7 - 15 % faster), and a rate that stops near 0.70 of the HBM peak for k = 64 and 128 whatever m is, where the
    // LDS image's coalesced loads reach 0.72 - 0.80 once m is near 32.  Up to 16 features this kernel does a third of the
    // matrix work of the one above, which always computes three blocks (batch 65536, k = 128: m = 16 0.144 -> 0.109 ms,
    // m = 8 0.136 -> 0.048 ms); which of the two runs beyond 16 is decided by the launcher.
    constexpr uint32_t F32_DIRECT_STEPS = 2; // samples per wave
    template <uint32_t K, bool HIGH = false>
    __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(4)))
        dlrmFwdF32Direct(const float* __restrict__ in, float* __restrict__ out, uint32_t m, uint32_t batch)
    {
        constexpr uint32_t JS        = K / 16u; // 128-bit loads per lane and sample
        constexpr uint32_t ROWS      = HIGH ? 32u : 16u;
        constexpr uint32_t MAX_OUT   = K + ROWS * (ROWS - 1u) / 2u;
        constexpr uint32_t OUT_STEPS = (MAX_OUT + 63u) / 64u; // 4-byte stores per lane and sample
        using f32x4                  = float __attribute__((ext_vector_type(4)));

        __shared__ __attribute__((aligned(16))) float outLds[WAVES][OUT_STEPS * 64u];

        const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t outStride = K + m * (m - 1u) / 2u;
        const uint32_t inBytes   = m * K * 4u;
        const uint32_t first = blockIdx.x * WAVES + wave, stride = gridDim.x * WAVES;
        float*         o     = outLds[wave];
        const uint32_t r16 = lane & 15u, kq = lane >> 4;
        const uint32_t off = r16 * K * 4u + kq * 16u;

        f32x4 x[JS], hi[HIGH ? JS : 1u];
        // (a sample beyond the batch is a buffer of no bytes: the loads are issued and move nothing)
        auto request = [&](uint64_t b) {
            const bool valid = b < batch;
            const auto src   = runBuffer(in, (uint64_t)(valid ? b : 0u) * inBytes, valid ? inBytes : 0u);
#pragma unroll
            for(uint32_t j = 0; j < JS; ++j)
            {
                x[j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(src, off + j * 64u, 0, 0));
                if constexpr(HIGH)
                    hi[j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(src, off + 16u * K * 4u + j * 64u, 0, 0));
            }
        };
        if(first >= batch)
            return;
        request(first);
#pragma unroll 1
        for(uint64_t b = first; b < batch; b += stride)
        {
            f32x4 acc0 = {0, 0, 0, 0}, acc1 = acc0, accHL = acc0, accHH = acc0;
#pragma unroll
            for(uint32_t j = 0; j < JS; ++j)
            {
                if(r16 == 0u) // the sample's first row is the head of its output row
                    *reinterpret_cast<f32x4*>(o + j * 16u + kq * 4u) = x[j];
                if constexpr(HIGH)
                {
#pragma unroll
                    for(uint32_t t = 0; t < 4u; ++t)
                    {
                        acc0  = __builtin_amdgcn_mfma_f32_16x16x4f32(x[j][t], x[j][t], acc0, 0, 0, 0);
                        accHL = __builtin_amdgcn_mfma_f32_16x16x4f32(hi[j][t], x[j][t], accHL, 0, 0, 0);
                        accHH = __builtin_amdgcn_mfma_f32_16x16x4f32(hi[j][t], hi[j][t], accHH, 0, 0, 0);
                    }
                    continue;
                }
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(x[j][0], x[j][0], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(x[j][1], x[j][1], acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(x[j][2], x[j][2], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(x[j][3], x[j][3], acc1, 0, 0, 0);
            }
            acc0 += acc1;
            __builtin_amdgcn_sched_barrier(0);
            request(b + stride); // the registers are free again
            __builtin_amdgcn_sched_barrier(0);

            // the 16 x 16 result block: a lane holds rows 4 (lane / 16) + e of column lane % 16
#pragma unroll
            for(uint32_t e = 0; e < 4; ++e)
            {
                const uint32_t i = 4u * kq + e, j = r16;
                if(j < i && i < m)
                    o[K + i * (i - 1u) / 2u + j] = acc0[e];
                if constexpr(HIGH)
                {
                    const uint32_t ih = 16u + i;
                    if(ih < m)
                    {
                        o[K + ih * (ih - 1u) / 2u + j] = accHL[e];
                        if(j < i)
                            o[K + ih * (ih - 1u) / 2u + 16u + j] = accHH[e];
                    }
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
            const auto dst = runBuffer(out, b * outStride * 4u, outStride * 4u);
#pragma unroll
            for(uint32_t e = 0; e < OUT_STEPS; ++e)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, o[e * 64u + lane]), dst, (e * 64u + lane) * 4u, 0, STORE_POLICY);
            __builtin_amdgcn_s_waitcnt(0xC07F); // the image is rewritten by the next sample
            __builtin_amdgcn_wave_barrier();
        }
    }

    // Backward: S = T + T^T (T = strict lower triangle from the upstream gradient, zero diagonal),
    // grad (m x k) = S X.  Same organisation as the forward kernel: a workgroup owns 8 consecutive
    // samples (their upstream rows form one 16-byte aligned run, staged in LDS with 128-bit loads),
    // a wave owns one sample at a time with the X of both of its samples requested up front.
    // X sits in LDS as [j][c] rows; the matrix instruction wants X^T (lane = column c, 8
    // consecutive j), which the transposing LDS read delivers: 16 lanes address a 4 (j) x 16 (c)
    // block and lane t receives column t.  Per 32-column slab of k: acc(c, i) = sum_j X(j, c) S(j, i),
    // i.e. every lane ends up with runs of 4 consecutive c of one gradient row i.  The gradient
    // image replaces X in LDS (rows < m) and leaves with 128-bit nontemporal stores.
    typedef __fp16 trv4 __attribute__((__vector_size__(4 * sizeof(__fp16))));

    template <bool BF16, uint32_t K, uint32_t ROWS>
    __global__ void __launch_bounds__(THREADS) dlrmBwdKernel(const uint16_t* __restrict__ in,
                                                            const uint16_t* __restrict__ upstream,
                                                            uint16_t* __restrict__ mlpGrad,
                                                            uint16_t* __restrict__ inGrad,
                                                            uint32_t m,
                                                            uint32_t batch,
                                                            uint32_t pack)
    {
        // (`pack` consecutive samples of few features as one block of rows, as in the forward kernel: S of the block is
        // block-diagonal, X and the gradient are the samples' rows one after the other)
        constexpr uint32_t ROW_CHUNKS = K / 8; // 16-byte chunks per row
        constexpr uint32_t ROWB       = K * 2;
        constexpr uint32_t X_BYTES    = MAX_M * ROWB; // always 32 rows: rows >= m stay zero
        constexpr uint32_t SLABS      = K / 32;
        constexpr uint32_t MAX_UP     = K + ROWS * (ROWS - 1) / 2;
        constexpr uint32_t PER_WAVE   = SAMPLES_PER_WG / WAVES;
        constexpr uint32_t MAX_CHUNKS = (ROWS * ROW_CHUNKS + 63u) / 64u;
        constexpr uint32_t SWZ_IN     = 12u & (ROW_CHUNKS - 1u); // (j & 3) << 2: four j rows -> four 64-byte groups
        constexpr uint32_t SWZ_OUT    = 15u & (ROW_CHUNKS - 1u);

        constexpr uint32_t UP_VECS = (SAMPLES_PER_WG * MAX_UP + 7u) / 8u; // 16-byte pieces of the workgroup's upstream run
        constexpr uint32_t UP_LOADS = (UP_VECS + THREADS - 1u) / THREADS; // per thread

        __shared__ __attribute__((aligned(16))) char     xLds[WAVES][X_BYTES];
        __shared__ __attribute__((aligned(16))) uint16_t upLds[UP_LOADS * THREADS * 8u];

        const uint32_t tid      = threadIdx.x;
        const uint32_t lane     = tid & 63u;
        const uint32_t wave     = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t upStride = K + m * (m - 1) / 2;
        const uint32_t b0       = blockIdx.x * SAMPLES_PER_WG * pack;
        const uint32_t rows     = m * pack; // of a block
        const uint32_t inChunks = rows * ROW_CHUNKS;
        const uint32_t inBytes  = m * ROW_CHUNKS * 16u; // of a sample
        const uint32_t rcpM     = (65536u + m - 1u) / m; // i / m == (i * rcpM) >> 16 for i < 32
        char*          xw       = xLds[wave];

        // Everything the workgroup reads is requested at once, through raw buffers of exactly the bytes that exist (runBuffer):
        // X of the wave's two samples, then the workgroup's run of upstream rows.  (With a loop of guarded loads each trip
        // waited for its own load - one memory latency per trip.)
        i32x4 stash[PER_WAVE][MAX_CHUNKS];
#pragma unroll
        for(uint32_t q = 0; q < PER_WAVE; ++q)
        {
            const uint32_t b   = b0 + (wave + q * WAVES) * pack; // the block's first sample
            const uint32_t has = b < batch ? (batch - b < pack ? batch - b : pack) : 0u;
            const auto     src = runBuffer(in, (uint64_t)(has ? b : 0u) * inBytes, has * inBytes);
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
                stash[q][j] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(src, (j * 64u + lane) * 16u, 0, LOAD_POLICY));
        }

        // ---- upstream rows of the workgroup's samples -> LDS; zero rows m..31 of the X image
        const uint32_t nSamples = (batch - b0) < SAMPLES_PER_WG * pack ? (batch - b0) : SAMPLES_PER_WG * pack;
        {
            // the run is a whole number of 16-byte pieces unless the batch ends inside this workgroup; whole 4-byte words go
            // through the buffer (its range check works on words), a last odd element on its own
            const uint32_t total = nSamples * upStride; // elements
            const auto     src   = runBuffer(upstream, (uint64_t)b0 * upStride * 2u, (total & ~1u) * 2u);
            i32x4          upv[UP_LOADS];
#pragma unroll
            for(uint32_t j = 0; j < UP_LOADS; ++j)
                upv[j] = __builtin_bit_cast(i32x4, __builtin_amdgcn_raw_buffer_load_b128(src, (j * THREADS + tid) * 16u, 0, LOAD_POLICY));
#pragma unroll
            for(uint32_t j = 0; j < UP_LOADS; ++j)
                reinterpret_cast<i32x4*>(upLds)[j * THREADS + tid] = upv[j];
            // (by the thread whose own 16-byte piece covers it and has just put a zero there: LDS writes of one wave stay
            // in order, those of different waves do not)
            if((total & 1u) && tid == ((total - 1u) / 8u) % THREADS)
                upLds[total - 1u] = upstream[(uint64_t)b0 * upStride + total - 1u];
            for(uint32_t c = inChunks + lane; c < MAX_M * ROW_CHUNKS; c += 64u)
                *reinterpret_cast<i32x4*>(xw + c * 16u) = i32x4{0, 0, 0, 0};
        }
        __syncthreads();

        // ---- bottom-MLP gradient: the first k values of every upstream row
        const auto mlpRun = runBuffer(mlpGrad, (uint64_t)b0 * K * 2u, nSamples * K * 2u);
        for(uint32_t t = tid; t < nSamples * ROW_CHUNKS; t += THREADS)
        {
            const uint32_t sIdx = t / ROW_CHUNKS, cc = t % ROW_CHUNKS;
            union
            {
                uint16_t h[8];
                i32x4    v;
            } o;
#pragma unroll
            for(uint32_t e = 0; e < 8; ++e)
                o.h[e] = upLds[sIdx * upStride + cc * 8u + e];
            runStore(o.v, mlpRun, t * 16u);
        }

        const uint32_t i = lane & 31u, half = lane >> 5, t16 = lane & 15u;
#pragma unroll
        for(uint32_t q = 0; q < PER_WAVE; ++q)
        {
            const uint32_t sIdx = wave + q * WAVES;
            const uint32_t b    = b0 + sIdx * pack;
            if(b >= batch)
                break;
            const uint32_t has = batch - b < pack ? batch - b : pack; // samples of this block
            // ---- X -> LDS: chunk c goes to row j = c / ROW_CHUNKS, slot (c % ROW_CHUNKS) ^ ((j & 3) << 2)
            // (the rows of samples beyond the batch arrived as zeros and are written like the others)
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < inChunks)
                {
                    const uint32_t row = c / ROW_CHUNKS, col = c % ROW_CHUNKS;
                    *reinterpret_cast<i32x4*>(xw + (row * ROW_CHUNKS + (col ^ ((row << 2) & SWZ_IN))) * 16u) = stash[q][j];
                }
            }
            // ---- S operand: lane holds S(i, j) for its 8-wide runs of j (zero diagonal, zero padding)
            const uint16_t* tril = upLds + sIdx * pack * upStride + K; // of the block's first sample
            const uint32_t  si = (i * rcpM) >> 16, li = i - si * m; // the lane's row: sample within the block, row within it
            i32x4           sReg[2];
#pragma unroll
            for(uint32_t s = 0; s < 2; ++s)
            {
                union
                {
                    uint16_t h[8];
                    i32x4    v;
                } so;
#pragma unroll
                for(uint32_t e = 0; e < 8; ++e)
                {
                    const uint32_t j  = 16u * s + 8u * half + e;
                    const uint32_t sj = (j * rcpM) >> 16, lj = j - sj * m;
                    const uint32_t hi = li > lj ? li : lj, lo = li > lj ? lj : li;
                    uint16_t       v  = 0;
                    if(si == sj && si < has && hi != lo)
                        v = tril[si * upStride + hi * (hi - 1u) / 2u + lo];
                    so.h[e] = v;
                }
                sReg[s] = so.v;
            }
            __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): this wave's LDS writes are done
            __builtin_amdgcn_wave_barrier();

            f32x16 acc[SLABS];
#pragma unroll
            for(uint32_t slab = 0; slab < SLABS; ++slab)
            {
                acc[slab] = f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for(uint32_t s = 0; s < 2; ++s)
                {
                    using lp             = __attribute__((address_space(3))) trv4*;
                    const uint32_t row   = 16u * s + 8u * half + (t16 >> 2);
                    const uint32_t piece = 8u * slab + 4u * ((lane >> 4) & 1u) + (t16 & 3u); // 8-byte pieces
                    const char*    p0    = xw + row * ROWB + (((piece >> 1) ^ ((row << 2) & SWZ_IN)) * 16u) + (piece & 1u) * 8u;
                    using i32x2          = int __attribute__((ext_vector_type(2)));
                    const i32x2 lo = __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((lp)p0));
                    const i32x2 hi = __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4f16((lp)(p0 + 4u * ROWB)));
                    acc[slab]      = mfma16<BF16>(acc[slab], i32x4{lo[0], lo[1], hi[0], hi[1]}, sReg[s]);
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F); // every read of X has returned before rows are overwritten
            __builtin_amdgcn_wave_barrier();

            // ---- gradient image over the block's rows: lane has c = 32 slab + 8 r + 4 half + (0..3) of row i
            if(i < rows)
            {
#pragma unroll
                for(uint32_t slab = 0; slab < SLABS; ++slab)
#pragma unroll
                    for(uint32_t r = 0; r < 4; ++r)
                    {
                        union
                        {
                            uint16_t h[4];
                            uint64_t v;
                        } o;
#pragma unroll
                        for(uint32_t e = 0; e < 4; ++e)
                            o.h[e] = roundOut<BF16>(acc[slab][4 * r + e]);
                        const uint32_t chunk = 4u * slab + r;
                        *reinterpret_cast<uint64_t*>(xw + i * ROWB + ((chunk ^ (i & SWZ_OUT)) * 16u) + half * 8u) = o.v;
                    }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();

            const auto gradRun = runBuffer(inGrad, (uint64_t)b * m * K * 2u, has * m * K * 2u);
#pragma unroll
            for(uint32_t j = 0; j < MAX_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                if(c < has * m * ROW_CHUNKS)
                {
                    const uint32_t row = c / ROW_CHUNKS, col = c % ROW_CHUNKS;
                    const i32x4    v   = *reinterpret_cast<const i32x4*>(xw + (row * ROW_CHUNKS + (col ^ (row & SWZ_OUT))) * 16u);
                    runStore(v, gradRun, c * 16u);
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
        }
    }

    // f32 backward.  grad (m x k) = S X with S = T + T^T from the upstream triangle, on
    // v_mfma_f32_16x16x4_f32: A operand = a 16 x 4 piece of S (lane l: row l % 16, column l / 16), B
    // operand = a 4 x 16 piece of X (lane l: row l / 16, column l % 16), 2 x (k / 16) result blocks, 8
    // steps over the 32 (zero-padded) rows of X.  Every wave walks F32_STEPS samples (first, first + stride, ...) with the
    // loads of the next sample in flight.  Per sample: X goes to an LDS image whose 64-byte column
    // groups are XOR-swizzled with the row (four consecutive rows of one column group land in
    // different banks), the upstream row to a second image from which each lane gathers its 16 values
    // of S; the gradient is written over X and leaves with 128-bit nontemporal stores; the first k
    // upstream values are the bottom-MLP gradient (test/reference_impl.hpp:121-179).
    template <uint32_t K, bool PACK>
    __global__ void __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2))) dlrmBwdF32Kernel(const float* __restrict__ in, const float* __restrict__ upstream,
                                                               float* __restrict__ mlpGrad, float* __restrict__ inGrad,
                                                               uint32_t m, uint32_t batch, uint32_t packArg)
    {
        // (PACK: `pack` consecutive samples of few features as one block of rows, as in the 16-bit kernels: S of the block
        // is block-diagonal, X, the upstream rows and the gradient are the samples' one after the other.  An instance of its
        // own: the index arithmetic of the block-diagonal S would cost the one-sample kernel registers it does not have.)
        const uint32_t pack = PACK ? packArg : 1u;
        constexpr uint32_t ROW_CHUNKS = K / 4; // 16-byte chunks per row
        constexpr uint32_t ROWB       = K * 4;
        constexpr uint32_t MAX_UP     = K + MAX_M * (MAX_M - 1) / 2;
        constexpr uint32_t X_CHUNKS   = (MAX_M * ROW_CHUNKS + 63u) / 64u; // per lane
        constexpr uint32_t UP_WORDS   = (MAX_UP + 63u) / 64u; // per lane
        constexpr uint32_t CBLOCKS    = K / 16; // 64-byte column groups per row
        constexpr uint32_t SWZ        = CBLOCKS >= 4 ? 3u : CBLOCKS - 1u;
        using f32x4                   = float __attribute__((ext_vector_type(4)));

        __shared__ __attribute__((aligned(16))) char  xLds[WAVES][MAX_M * ROWB];
        __shared__ __attribute__((aligned(16))) float upLds[WAVES][UP_WORDS * 64u];

        const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t upStride = K + m * (m - 1) / 2;
        const uint32_t inBytes  = m * ROWB; // of a sample
        const uint32_t rows     = m * pack; // of a block
        const uint32_t rcpM     = (65536u + m - 1u) / m; // i / m == (i * rcpM) >> 16 for i < 32
        const uint32_t blocks   = (batch + pack - 1u) / pack;
        // a wave walks the blocks first, first + stride, ...
        const uint32_t first = blockIdx.x * WAVES + wave, stride = gridDim.x * WAVES;
        char*          xw       = xLds[wave];
        float*         uw       = upLds[wave];
        const uint32_t r16 = lane & 15u, q4 = lane >> 4;

        // byte address of 16-byte chunk c (0 .. ROW_CHUNKS) of row `row` in the swizzled image
        auto chunkAt = [&](uint32_t row, uint32_t c) { return row * ROWB + ((((c >> 2) ^ (row & SWZ)) << 2) + (c & 3u)) * 16u; };

        // where lane l finds S(i, j) in the upstream image: the strict lower triangle is stored row by
        // row behind the first k values; the diagonal is zero (recomputed per sample: registers are
        // scarcer than integer instructions here)
        auto sAt = [&](uint32_t i, uint32_t j) -> float {
            if constexpr(PACK)
            {
                const uint32_t si = (i * rcpM) >> 16, sj = (j * rcpM) >> 16, li = i - si * m, lj = j - sj * m;
                const uint32_t hi = li > lj ? li : lj, lo = li > lj ? lj : li;
                return (si == sj && li != lj && si < pack) ? uw[si * upStride + K + hi * (hi - 1u) / 2u + lo] : 0.0f;
            }
            else
            {
                const uint32_t hi = i > j ? i : j, lo = i > j ? j : i;
                return (i != j && hi < m) ? uw[K + hi * (hi - 1u) / 2u + lo] : 0.0f;
            }
        };

        // one register stash: a sample's loads are requested while the previous sample is computed and
        // unloaded into LDS before the next request reuses the registers.  All loads and stores go through raw
        // buffers of exactly the sample's bytes (runBuffer): no branches, every wait exact.  (A sample beyond the batch
        // is a buffer of no bytes.)  Chunks of rows >= m arrive as zeros, which is what the
        // product needs there.
        f32x4 xs[X_CHUNKS];
        float us[UP_WORDS];
        // (block index -> its first sample and how many of its samples exist)
        auto  request = [&](uint64_t blk) {
            const uint64_t b   = blk * pack;
            const uint32_t has = blk < blocks ? (batch - b < pack ? (uint32_t)(batch - b) : pack) : 0u;
            const auto     src = runBuffer(in, (has ? b : 0u) * inBytes, has * inBytes);
            const auto     up  = runBuffer(upstream, (has ? b : 0u) * upStride * 4u, has * upStride * 4u);
#pragma unroll
            for(uint32_t j = 0; j < X_CHUNKS; ++j)
                xs[j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(src, (j * 64u + lane) * 16u, 0, LOAD_POLICY));
#pragma unroll
            for(uint32_t j = 0; j < UP_WORDS; ++j)
                us[j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(up, (j * 64u + lane) * 4u, 0, LOAD_POLICY));
        };

        auto process = [&](uint64_t blk) {
            const uint64_t b   = blk * pack;
            const uint32_t has = batch - b < pack ? (uint32_t)(batch - b) : pack;
#pragma unroll
            for(uint32_t j = 0; j < X_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane; // (X_CHUNKS * 64 chunks are exactly the 32 rows of the image)
                *reinterpret_cast<f32x4*>(xw + chunkAt(c / ROW_CHUNKS, c % ROW_CHUNKS)) = xs[j];
            }
#pragma unroll
            for(uint32_t j = 0; j < UP_WORDS; ++j)
                uw[j * 64u + lane] = us[j];
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
            request(blk + stride);

            // bottom-MLP gradient: the first k upstream values of every sample of the block
            const auto mg = runBuffer(mlpGrad, b * K * 4u, has * K * 4u);
            for(uint32_t s = 0; s < has; ++s)
#pragma unroll
                for(uint32_t e = 0; e < (K + 63u) / 64u; ++e)
                    if(K >= 64u || lane < K)
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, uw[s * upStride + e * 64u + lane]), mg,
                                                              (s * K + e * 64u + lane) * 4u, 0, STORE_POLICY);

            float sv[2][8];
#pragma unroll
            for(uint32_t ib = 0; ib < 2; ++ib)
#pragma unroll
                for(uint32_t js = 0; js < 8; ++js)
                    sv[ib][js] = sAt(16u * ib + r16, 4u * js + q4);

            f32x4 acc[2][CBLOCKS];
#pragma unroll
            for(uint32_t ib = 0; ib < 2; ++ib)
#pragma unroll
                for(uint32_t cb = 0; cb < CBLOCKS; ++cb)
                    acc[ib][cb] = f32x4{0, 0, 0, 0};
#pragma unroll
            for(uint32_t js = 0; js < 8; ++js)
            {
                const uint32_t row = 4u * js + q4;
#pragma unroll
                for(uint32_t cb = 0; cb < CBLOCKS; ++cb)
                {
                    // X(row, 16 cb + l % 16): 64-byte column group cb, swizzled with the row
                    const float xv = *reinterpret_cast<const float*>(xw + row * ROWB + ((cb ^ (row & SWZ)) << 6) + r16 * 4u);
                    acc[0][cb]     = __builtin_amdgcn_mfma_f32_16x16x4f32(sv[0][js], xv, acc[0][cb], 0, 0, 0);
                    acc[1][cb]     = __builtin_amdgcn_mfma_f32_16x16x4f32(sv[1][js], xv, acc[1][cb], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0); // keeps the LDS reads of later steps from piling up in registers
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier(); // every lane has read X: the gradient goes over it
            // result block (ib, cb): lane holds rows 16 ib + 4 (l / 16) + e, column 16 cb + l % 16
#pragma unroll
            for(uint32_t ib = 0; ib < 2; ++ib)
#pragma unroll
                for(uint32_t cb = 0; cb < CBLOCKS; ++cb)
#pragma unroll
                    for(uint32_t e = 0; e < 4; ++e)
                    {
                        const uint32_t row = 16u * ib + 4u * q4 + e;
                        if(row < rows)
                            *reinterpret_cast<float*>(xw + row * ROWB + ((cb ^ (row & SWZ)) << 6) + r16 * 4u) = acc[ib][cb][e];
                    }
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_wave_barrier();
            const auto dst = runBuffer(inGrad, b * inBytes, has * inBytes);
#pragma unroll
            for(uint32_t j = 0; j < X_CHUNKS; ++j)
            {
                const uint32_t c = j * 64u + lane;
                using u32x4      = uint32_t __attribute__((ext_vector_type(4)));
                __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const u32x4*>(xw + chunkAt(c / ROW_CHUNKS, c % ROW_CHUNKS)), dst,
                                                       c * 16u, 0, RUN_POLICY);
            }
            __builtin_amdgcn_s_waitcnt(0xC07F); // the images are rewritten by the next sample
            __builtin_amdgcn_wave_barrier();
        };

        // The first sample stands outside the loop so that the loop is entered with the same operations in flight as
        // its own trips leave behind: the waits inside are then exact on both paths.
        if(first >= blocks)
            return;
        request(first);
        process(first);
#pragma unroll 1
        for(uint64_t blk = (uint64_t)first + stride; blk < blocks; blk += stride)
            process(blk);
    }

    int checkArgs(const char* what, int32_t dtype, const void* in, const void* out, uint32_t m, uint32_t k, uint32_t batch,
                  bool allowF32)
    {
        if(!in || !out)
            return r355::fail(R355_ERR_BAD_ARG, "%s: null pointer", what);
        if(dtype != R355_F16 && dtype != R355_BF16 && !(allowF32 && dtype == R355_F32))
            return r355::fail(R355_ERR_UNSUPPORTED, "%s: dtype must be R355_F16, R355_BF16%s", what, allowF32 ? " or R355_F32" : "");
        if(m < 2)
            return r355::fail(R355_ERR_BAD_SIZE, "%s: m=%u must be at least 2", what, m);
        if(batch == 0)
            return r355::fail(R355_ERR_BAD_ARG, "%s: batch is zero", what);
        if(!r355::aligned(in, 16) || !r355::aligned(out, 16))
            return r355::fail(R355_ERR_MISALIGNED, "%s: in / out must be 16-byte aligned", what);
        return R355_OK;
    }
    // 16-bit kernels, up to 16 features: the samples that share a block of rows - as many as fit the rows of the LDS image
    // (28 or 32: `small` says which instance) and, with their output / upstream rows, the space of that image's one
    // full-size sample's row.  The 32-row instance where it takes more samples per block - except at k = 128, where the
    // 28-row image lets four workgroups share a CU instead of three and fewer samples per block are still faster
    // (forward, m = 16: 0.79 against 0.73 of the HBM peak, m = 8: 0.77 against 0.74).
    uint32_t samplesPerBlock(uint32_t m, uint32_t k, bool& small)
    {
#ifdef R355_DLRM_NO_PACK // (measurement build: one sample per block whatever m is)
        return 1u;
#endif
        if(m > 16)
            return 1u;
        auto fits = [&](uint32_t rows) {
            const uint32_t byRows = rows / m, byRow = (k + rows * (rows - 1u) / 2u) / (k + m * (m - 1u) / 2u);
            return byRows < byRow ? byRows : byRow;
        };
        const uint32_t p28 = fits(28), p32 = fits(32);
#if defined(R355_DLRM_PACK_PREFER_28) // (measurement builds: always the 28-row image / always the one with more samples)
        small = true;
#elif defined(R355_DLRM_PACK_MORE_SAMPLES)
        small = p28 == p32;
#else
        small = p28 == p32 || k == 128;
#endif
        return small ? p28 : p32;
    }
    // the kernels of this file: up to 32 features and an embedding width they are instantiated for; everything else goes
    // to the kernels of dlrm_general.hip
    bool specialised(int32_t dtype, uint32_t m, uint32_t k)
    {
        return m <= MAX_M && (k == 32 || k == 64 || k == 128 || (k == 256 && dtype != R355_F32));
    }
} // namespace

extern "C" int r355_dlrm_fwd(int32_t dtype, const void* in, void* out, uint32_t m, uint32_t k, uint32_t batch, void* stream)
{
    int rc = checkArgs("dlrm_fwd", dtype, in, out, m, k, batch, true);
    if(rc != R355_OK)
        return rc;
    r355::beginCall();
    hipStream_t s = static_cast<hipStream_t>(stream);
    if(!specialised(dtype, m, k))
        return r355::dlrmGeneralFwd(dtype, in, out, m, k, batch, s);
    if(dtype == R355_F32)
    {
        const uint32_t steps = (batch + WAVES - 1) / WAVES; // of one sample per wave
        auto*      fi = static_cast<const float*>(in);
        auto*      fo = static_cast<float*>(out);
        // Three kernels.  dlrmFwdF32Direct (matrix instructions straight from the loads): up to 16 features, where it runs one
        // block of rows instead of three, and a few more while its scattered 16-byte pieces cost less than what the others
        // pay per sample.  dlrmFwdF32Run (eight samples per workgroup, one run of output rows, the image in halves of k): its
        // time follows m.  dlrmFwdF32Kernel (a wave per sample, the whole sample in the image): k = 64 near 32 features.
        // Chosen per (m, k) from measurements at a batch of 65536 (m = 17 .. 32); measurement builds force one of them.
#if defined(R355_DLRM_F32_LDS_IMAGE)
        const bool direct = false, run = false;
#elif defined(R355_DLRM_F32_DIRECT_ALL)
        const bool direct = true, run = false;
#elif defined(R355_DLRM_F32_RUN_ALL)
        const bool direct = false, run = k >= 64;
#else
        const bool direct = m <= 16 || k == 32 || (k == 64 && m <= 20) || (k == 128 && m <= 17);
        const bool run    = !direct && (k == 128 || (k == 64 && m <= 26));
#endif
        if(direct)
        {
            const dim3 grid((steps + F32_DIRECT_STEPS - 1) / F32_DIRECT_STEPS), block(THREADS);
#define R355_FWD32D(KK)                                                                              \
    do                                                                                               \
    {                                                                                                \
        if(m <= 16)                                                                                  \
            hipLaunchKernelGGL((dlrmFwdF32Direct<KK, false>), grid, block, 0, s, fi, fo, m, batch);  \
        else                                                                                         \
            hipLaunchKernelGGL((dlrmFwdF32Direct<KK, true>), grid, block, 0, s, fi, fo, m, batch);   \
    } while(0)
            switch(k)
            {
            case 32: R355_FWD32D(32); break;
            case 64: R355_FWD32D(64); break;
            default: R355_FWD32D(128); break;
            }
#undef R355_FWD32D
            return r355::checkLaunch("dlrm_fwd");
        }
        const dim3     grid32((steps + F32_STEPS - 1) / F32_STEPS), block32(THREADS);
        if(run)
        {
            const dim3 gridRun((batch + SAMPLES_PER_WG - 1) / SAMPLES_PER_WG);
            if(k == 64 && m <= 28)
                hipLaunchKernelGGL((dlrmFwdF32Run<64, 28>), gridRun, block32, 0, s, fi, fo, m, batch);
            else if(k == 64)
                hipLaunchKernelGGL((dlrmFwdF32Run<64, 32>), gridRun, block32, 0, s, fi, fo, m, batch);
            else if(m <= 28)
                hipLaunchKernelGGL((dlrmFwdF32Run<128, 28>), gridRun, block32, 0, s, fi, fo, m, batch);
            else
                hipLaunchKernelGGL((dlrmFwdF32Run<128, 32>), gridRun, block32, 0, s, fi, fo, m, batch);
            return r355::checkLaunch("dlrm_fwd");
        }
#define R355_FWD32(KK)                                                                                \
    do                                                                                                \
    {                                                                                                 \
        if(m <= 28)                                                                                   \
            hipLaunchKernelGGL((dlrmFwdF32Kernel<KK, 28>), grid32, block32, 0, s, fi, fo, m, batch);  \
        else                                                                                          \
            hipLaunchKernelGGL((dlrmFwdF32Kernel<KK, 32>), grid32, block32, 0, s, fi, fo, m, batch);  \
    } while(0)
        switch(k)
        {
        case 32: R355_FWD32(32); break;
        case 64: R355_FWD32(64); break;
        default: R355_FWD32(128); break;
        }
#undef R355_FWD32
        return r355::checkLaunch("dlrm_fwd");
    }
    bool           small = m <= 28;
    const uint32_t pack  = samplesPerBlock(m, k, small);
    const dim3 grid((batch + SAMPLES_PER_WG * pack - 1) / (SAMPLES_PER_WG * pack)), block(THREADS);
    auto*       pi = static_cast<const uint16_t*>(in);
    auto*       po = static_cast<uint16_t*>(out);
#define R355_FWD(BF, KK)                                                                               \
    do                                                                                                  \
    {                                                                                                   \
        if(small)                                                                                       \
            hipLaunchKernelGGL((dlrmFwdKernel<BF, KK, 28>), grid, block, 0, s, pi, po, m, batch, pack); \
        else                                                                                            \
            hipLaunchKernelGGL((dlrmFwdKernel<BF, KK, 32>), grid, block, 0, s, pi, po, m, batch, pack); \
    } while(0)
#define R355_FWD_K(BF)   \
    switch(k)            \
    {                    \
    case 32: R355_FWD(BF, 32); break;   \
    case 64: R355_FWD(BF, 64); break;   \
    case 128: R355_FWD(BF, 128); break; \
    default: R355_FWD(BF, 256); break;  \
    }
    if(dtype == R355_BF16)
    {
        R355_FWD_K(true)
    }
    else
    {
        R355_FWD_K(false)
    }
#undef R355_FWD_K
#undef R355_FWD
    return r355::checkLaunch("dlrm_fwd");
}

extern "C" int r355_dlrm_bwd(int32_t dtype, const void* in, const void* upstream, void* mlp_grad, void* in_grad,
                             uint32_t m, uint32_t k, uint32_t batch, void* stream)
{
    int rc = checkArgs("dlrm_bwd", dtype, in, in_grad, m, k, batch, true);
    if(rc != R355_OK)
        return rc;
    if(!upstream || !mlp_grad)
        return r355::fail(R355_ERR_BAD_ARG, "dlrm_bwd: null pointer");
    r355::beginCall();
    if(!specialised(dtype, m, k))
        return r355::dlrmGeneralBwd(dtype, in, upstream, mlp_grad, in_grad, m, k, batch, static_cast<hipStream_t>(stream));
    if(dtype == R355_F32)
    {
        if(!r355::aligned(upstream, 4) || !r355::aligned(mlp_grad, 4))
            return r355::fail(R355_ERR_MISALIGNED, "dlrm_bwd: upstream and mlp_grad must be 4-byte aligned");
        // up to 16 features several samples share a block of rows, as many as fit the 32 rows of the image and, with
        // their upstream rows, the space of one 32-feature sample's
        uint32_t pack = 1;
#ifndef R355_DLRM_NO_PACK
        if(m <= 16)
        {
            const uint32_t byRows = 32u / m, byRow = (k + 32u * 31u / 2u) / (k + m * (m - 1u) / 2u);
            pack = byRows < byRow ? byRows : byRow;
        }
#endif
        const uint32_t blocks = (batch + pack - 1) / pack;
        const uint32_t steps  = (blocks + WAVES - 1) / WAVES; // of one block per wave
        const dim3     grid32((steps + F32_STEPS - 1) / F32_STEPS), block32(THREADS);
        hipStream_t    s32 = static_cast<hipStream_t>(stream);
        auto*          fi  = static_cast<const float*>(in);
        auto*          fu  = static_cast<const float*>(upstream);
        auto*          fm  = static_cast<float*>(mlp_grad);
        auto*          fg  = static_cast<float*>(in_grad);
#define R355_BWD32(KK)                                                                                                   \
    do                                                                                                                   \
    {                                                                                                                    \
        if(pack > 1)                                                                                                     \
            hipLaunchKernelGGL((dlrmBwdF32Kernel<KK, true>), grid32, block32, 0, s32, fi, fu, fm, fg, m, batch, pack);   \
        else                                                                                                             \
            hipLaunchKernelGGL((dlrmBwdF32Kernel<KK, false>), grid32, block32, 0, s32, fi, fu, fm, fg, m, batch, pack);  \
    } while(0)
        switch(k)
        {
        case 32: R355_BWD32(32); break;
        case 64: R355_BWD32(64); break;
        default: R355_BWD32(128); break;
        }
#undef R355_BWD32
        return r355::checkLaunch("dlrm_bwd");
    }
    if(!r355::aligned(upstream, 16) || !r355::aligned(mlp_grad, 16))
        return r355::fail(R355_ERR_MISALIGNED, "dlrm_bwd: upstream and mlp_grad must be 16-byte aligned");
    bool           small = m <= 28;
    const uint32_t pack  = samplesPerBlock(m, k, small);
    const dim3     grid((batch + SAMPLES_PER_WG * pack - 1) / (SAMPLES_PER_WG * pack)), block(THREADS);
    hipStream_t s  = static_cast<hipStream_t>(stream);
    auto*       pi = static_cast<const uint16_t*>(in);
    auto*       pu = static_cast<const uint16_t*>(upstream);
    auto*       pm = static_cast<uint16_t*>(mlp_grad);
    auto*       pg = static_cast<uint16_t*>(in_grad);
#define R355_BWD(BF, KK)                                                                                          \
    do                                                                                                            \
    {                                                                                                             \
        if(small)                                                                                                 \
            hipLaunchKernelGGL((dlrmBwdKernel<BF, KK, 28>), grid, block, 0, s, pi, pu, pm, pg, m, batch, pack);    \
        else                                                                                                      \
            hipLaunchKernelGGL((dlrmBwdKernel<BF, KK, 32>), grid, block, 0, s, pi, pu, pm, pg, m, batch, pack);    \
    } while(0)
#define R355_BWD_K(BF)   \
    switch(k)            \
    {                    \
    case 32: R355_BWD(BF, 32); break;   \
    case 64: R355_BWD(BF, 64); break;   \
    case 128: R355_BWD(BF, 128); break; \
    default: R355_BWD(BF, 256); break;  \
    }
    if(dtype == R355_BF16)
    {
        R355_BWD_K(true);
    }
    else
    {
        R355_BWD_K(false);
    }
#undef R355_BWD_K
#undef R355_BWD
    return r355::checkLaunch("dlrm_bwd");
}
