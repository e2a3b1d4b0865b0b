// C++ host bench for the C ABI: allocates device buffers, fills them from a seeded generator,
// times the kernel with the reference's protocol (warm-up launches, then N launches between two
// hipEvents: test/gemm/gemm_kernel_base_impl.hpp:647-676) and reports throughput the way the
// reference does (2 m n k flop, test/performance.hpp:424-442), plus the fraction of MI355X's
// published peak.  Usage:
//   host_bench gemm  [--type f16|bf16|i8|e4m3|f32|f64] [--out f16|bf16|f32|i32|f64] [--layout nt|tn|nn|tt]
//                    [--m M --n N --k K] [--kernel auto|simple|tiled|tiled128|deep] [--warmup W --iters I]
//                    [--sparse 1]   A is 2:4 structured sparse (compressed values + index nibbles)
//                    [--workspace MiB]  device workspace offered for split-K (few tiles, long K); 0 = none
//                    [--zero 1]     all-zero operands (no switching power: the engine clock stays at its maximum)
//                    [--ldpad E]    lda and ldb grow by E elements (power-of-two strides cost L2 efficiency)
//   host_bench dlrm  [--type f16|bf16|f32] [--bwd 1] [--batch B --m M --k K] [--warmup W --iters I]
//   host_bench gemv  [--m M --k K --layout n|t] [--split 1]   (--split 1: r355_gemv_ws with the workspace its query asks for)
//   host_bench copy  [--bytes N]      plain device copy of known size (counter calibration)
//   host_bench mix                    a bare kernel at the DLRM forward's read / write mix (7 KiB read, 1 KiB written per
//                                     unit and wave, 65536 units): what plain streaming code reaches at that mix
//   host_bench lds   [--iters I]      LDS read and write instructions from fixed conflict-free addresses with 4, 2 and 1 waves per CU:
//                                     shader clocks per wave-level read and bytes per clock per CU
//   host_bench fill                   direct global -> LDS loads alone, in the access stream of the 8192^3 1-byte GEMM
//                                     (1024 tiles x 64 stages x 64 KiB), 1 - 3 stages in flight: aggregate TB/s
//   host_bench store                  global stores alone in the shape of the macro-tile epilogue (256 KiB per workgroup)
//   host_bench mfma  [--iters I]      register-resident MFMA loops, one wave per SIMD, 16 independent
//                                     accumulators: the rate the matrix cores sustain under the board's
//                                     power limit with all-zero and with random operands
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include <hip/hip_runtime.h>

#include "../../include/r355_wmma.h"
#include "lds_dma.hpp"
#include "tile_map.hpp"

#define HIP_OK(expr)                                                                       \
    do                                                                                     \
    {                                                                                      \
        hipError_t e_ = (expr);                                                            \
        if(e_ != hipSuccess)                                                               \
        {                                                                                  \
            fprintf(stderr, "hip error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            return 1;                                                                      \
        }                                                                                  \
    } while(0)

namespace
{
    uint64_t splitmix(uint64_t seed, uint64_t i)
    {
        uint64_t z = (i + 1) * 0x9E3779B97F4A7C15ull + seed * 0xD1B54A32D192ED03ull;
        z          = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z          = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }

    // seeded values in a sane range for each type, no NaN / inf
    void fillBytes(std::vector<uint8_t>& buf, int dtype, uint64_t seed)
    {
        const size_t es = (dtype == R355_F16 || dtype == R355_BF16) ? 2 : (dtype == R355_F32 ? 4 : (dtype == R355_F64 ? 8 : 1));
        const size_t n  = buf.size() / es;
        for(size_t i = 0; i < n; ++i)
        {
            const uint64_t r = splitmix(seed, i);
            switch(dtype)
            {
            case R355_F16: // U[-1, 1) rounded to the type, like bench.py's operands
            {
                const _Float16 h = static_cast<_Float16>(static_cast<float>(r >> 40) * (2.0f / 16777216.0f) - 1.0f);
                memcpy(buf.data() + 2 * i, &h, 2);
                break;
            }
            case R355_BF16:
            {
                const float f = static_cast<float>(r >> 40) * (2.0f / 16777216.0f) - 1.0f;
                uint32_t    u;
                memcpy(&u, &f, 4);
                u += 0x7FFFu + ((u >> 16) & 1u); // round to nearest even
                reinterpret_cast<uint16_t*>(buf.data())[i] = static_cast<uint16_t>(u >> 16);
                break;
            }
            case R355_E4M3: // exponent 3..6: |x| in [1/16, 1)
                buf[i] = static_cast<uint8_t>(((r & 1) << 7) | ((3 + ((r >> 1) & 3)) << 3) | ((r >> 8) & 7));
                break;
            case R355_I8: buf[i] = static_cast<uint8_t>(r >> 32); break;
            case R355_F64: reinterpret_cast<double*>(buf.data())[i] = static_cast<double>(r >> 11) * (2.0 / 9007199254740992.0) - 1.0; break;
            default: reinterpret_cast<float*>(buf.data())[i] = static_cast<float>((r >> 40) & 0xFFFF) / 65536.0f - 0.5f;
            }
        }
    }

    int parseType(const std::string& s)
    {
        if(s == "f16") return R355_F16;
        if(s == "bf16") return R355_BF16;
        if(s == "e4m3" || s == "fp8") return R355_E4M3;
        if(s == "i8") return R355_I8;
        if(s == "f32") return R355_F32;
        if(s == "f64") return R355_F64;
        if(s == "i32") return R355_I32;
        return -1;
    }

    size_t bytesOf(int t)
    {
        return (t == R355_F16 || t == R355_BF16) ? 2 : ((t == R355_F32 || t == R355_I32) ? 4 : (t == R355_F64 ? 8 : 1));
    }

    using f32x16 = float __attribute__((ext_vector_type(16)));
    using i32x16 = int __attribute__((ext_vector_type(16)));
    using i32x4  = int __attribute__((ext_vector_type(4)));
    using i32x8  = int __attribute__((ext_vector_type(8)));
    using f16x8  = _Float16 __attribute__((ext_vector_type(8)));
    using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));

    enum MfmaKind { MF_F16, MF_BF16, MF_I8, MF_FP8_K64, MF_SPARSE_I8, MF_F16_16, MF_I8_16, MF_FP8_16, MF_SPARSE_I8_16, MF_SPARSE_FP8_16, MF_KINDS };

    // 16 MFMAs per loop trip on 4 x 4 operand registers; no memory traffic inside the loop.
    template <int T>
    __global__ void __launch_bounds__(256) mfmaLoop(const i32x4* __restrict__ in, float* __restrict__ out, int iters)
    {
        i32x4 a[4], b[4];
        for(int i = 0; i < 4; ++i)
        {
            a[i] = in[(threadIdx.x + i * 256) % 1024];
            b[i] = in[(threadIdx.x * 3 + i * 131) % 1024];
        }
        f32x16 acc[16];
        i32x16 iacc[16];
        for(int i = 0; i < 16; ++i)
            for(int e = 0; e < 16; ++e)
                acc[i][e] = 0.0f, iacc[i][e] = 0;
        for(int it = 0; it < iters; ++it)
        {
#pragma unroll
            for(int i = 0; i < 4; ++i)
#pragma unroll
                for(int j = 0; j < 4; ++j)
                {
                    const int  x  = i * 4 + j;
                    const auto a8 = __builtin_shufflevector(a[i], a[(i + 1) & 3], 0, 1, 2, 3, 4, 5, 6, 7);
                    const auto b8 = __builtin_shufflevector(b[j], b[(j + 1) & 3], 0, 1, 2, 3, 4, 5, 6, 7);
                    if constexpr(T == MF_F16)
                        acc[x] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a[i]),
                                                                        __builtin_bit_cast(f16x8, b[j]), acc[x], 0, 0, 0);
                    else if constexpr(T == MF_BF16)
                        acc[x] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[i]),
                                                                         __builtin_bit_cast(bf16x8, b[j]), acc[x], 0, 0, 0);
                    else if constexpr(T == MF_I8)
                        iacc[x] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], iacc[x], 0, 0, 0);
                    else if constexpr(T == MF_FP8_K64)
                        acc[x] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a8, b8, acc[x], 0, 0, 0, 0x7F7F7F7F, 0,
                                                                                 0x7F7F7F7F);
                    else
                        iacc[x] = __builtin_amdgcn_smfmac_i32_32x32x64_i8(a[i], b8, iacc[x], 0x84848484, 0, 0);
                }
        }
        float s = 0.0f;
        for(int i = 0; i < 16; ++i)
            for(int e = 0; e < 16; ++e)
                s += acc[i][e] + static_cast<float>(iacc[i][e]);
        out[blockIdx.x * 256 + threadIdx.x] = s;
    }

    // The 16 x 16 shapes of the same types: 64 independent 4-register accumulators (same register
    // footprint and flop per loop trip as the 32 x 32 loop above).
    using f32x4 = float __attribute__((ext_vector_type(4)));
    template <int T>
    __global__ void __launch_bounds__(256) mfmaLoop16(const i32x4* __restrict__ in, float* __restrict__ out, int iters)
    {
        i32x4 a[4], b[4];
        for(int i = 0; i < 4; ++i)
        {
            a[i] = in[(threadIdx.x + i * 256) % 1024];
            b[i] = in[(threadIdx.x * 3 + i * 131) % 1024];
        }
        f32x4 acc[64];
        i32x4 iacc[64];
        for(int i = 0; i < 64; ++i)
            for(int e = 0; e < 4; ++e)
                acc[i][e] = 0.0f, iacc[i][e] = 0;
        for(int it = 0; it < iters; ++it)
        {
#pragma unroll
            for(int x = 0; x < 64; ++x)
            {
                const int  i = x & 3, j = (x >> 2) & 3;
                const auto a8 = __builtin_shufflevector(a[i], a[(i + 1) & 3], 0, 1, 2, 3, 4, 5, 6, 7);
                const auto b8 = __builtin_shufflevector(b[j], b[(j + 1) & 3], 0, 1, 2, 3, 4, 5, 6, 7);
                if constexpr(T == MF_F16_16)
                    acc[x] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a[i]),
                                                                    __builtin_bit_cast(f16x8, b[j]), acc[x], 0, 0, 0);
                else if constexpr(T == MF_I8_16)
                    iacc[x] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i], b[j], iacc[x], 0, 0, 0);
                else if constexpr(T == MF_FP8_16)
                    acc[x] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, acc[x], 0, 0, 0, 0x7F7F7F7F, 0,
                                                                              0x7F7F7F7F);
                else if constexpr(T == MF_SPARSE_I8_16) // 2:4 sparse A: 16 kept bytes + one index word per lane, 32 dense bytes of B
                    iacc[x] = __builtin_amdgcn_smfmac_i32_16x16x128_i8(a[i], b8, iacc[x], 0x84848484, 0, 0);
                else
                    acc[x] = __builtin_amdgcn_smfmac_f32_16x16x128_fp8_fp8(a[i], b8, acc[x], 0x84848484, 0, 0);
            }
        }
        float s = 0.0f;
        for(int i = 0; i < 64; ++i)
            for(int e = 0; e < 4; ++e)
                s += acc[i][e] + static_cast<float>(iacc[i][e]);
        out[blockIdx.x * 256 + threadIdx.x] = s;
    }

    void launchMfma(int kind, int cus, const i32x4* in, float* out, int iters)
    {
        const dim3 g(cus), b(256);
        switch(kind)
        {
        case MF_F16: hipLaunchKernelGGL(mfmaLoop<MF_F16>, g, b, 0, 0, in, out, iters); break;
        case MF_BF16: hipLaunchKernelGGL(mfmaLoop<MF_BF16>, g, b, 0, 0, in, out, iters); break;
        case MF_I8: hipLaunchKernelGGL(mfmaLoop<MF_I8>, g, b, 0, 0, in, out, iters); break;
        case MF_FP8_K64: hipLaunchKernelGGL(mfmaLoop<MF_FP8_K64>, g, b, 0, 0, in, out, iters); break;
        case MF_SPARSE_I8: hipLaunchKernelGGL(mfmaLoop<MF_SPARSE_I8>, g, b, 0, 0, in, out, iters); break;
        case MF_F16_16: hipLaunchKernelGGL(mfmaLoop16<MF_F16_16>, g, b, 0, 0, in, out, iters); break;
        case MF_I8_16: hipLaunchKernelGGL(mfmaLoop16<MF_I8_16>, g, b, 0, 0, in, out, iters); break;
        case MF_FP8_16: hipLaunchKernelGGL(mfmaLoop16<MF_FP8_16>, g, b, 0, 0, in, out, iters); break;
        case MF_SPARSE_I8_16: hipLaunchKernelGGL(mfmaLoop16<MF_SPARSE_I8_16>, g, b, 0, 0, in, out, iters); break;
        default: hipLaunchKernelGGL(mfmaLoop16<MF_SPARSE_FP8_16>, g, b, 0, 0, in, out, iters); break;
        }
    }

    // LDS read rate with nothing else in the loop: 16 reads per trip from fixed addresses (consecutive lanes,
    // consecutive pieces: conflict-free), 8 always in flight.  MODE: 0 ds_read_b128, 1 ds_read_b64, 2 ds_read_b64_tr_b16,
    // 3 ds_read_b32, 4 ds_read_b64_tr_b8.
#define R355_RD8(OP, R0, OFFB)                                                                                          \
    asm volatile(OP " %0, %8 offset:" #OFFB "+0\n\t" OP " %1, %8 offset:" #OFFB "+2048\n\t" OP " %2, %8 offset:" #OFFB      \
                    "+4096\n\t" OP " %3, %8 offset:" #OFFB "+6144\n\t" OP " %4, %8 offset:" #OFFB "+8192\n\t" OP          \
                    " %5, %8 offset:" #OFFB "+10240\n\t" OP " %6, %8 offset:" #OFFB "+12288\n\t" OP " %7, %8 offset:" #OFFB \
                    "+14336\n\t"                                                                                        \
                 : "=v"(R0[0]), "=v"(R0[1]), "=v"(R0[2]), "=v"(R0[3]), "=v"(R0[4]), "=v"(R0[5]), "=v"(R0[6]), "=v"(R0[7])  \
                 : "v"(addr))
#define R355_WR8(OP, R0, OFFB)                                                                                          \
    asm volatile(OP " %8, %0 offset:" #OFFB "+0\n\t" OP " %8, %1 offset:" #OFFB "+2048\n\t" OP " %8, %2 offset:" #OFFB      \
                    "+4096\n\t" OP " %8, %3 offset:" #OFFB "+6144\n\t" OP " %8, %4 offset:" #OFFB "+8192\n\t" OP          \
                    " %8, %5 offset:" #OFFB "+10240\n\t" OP " %8, %6 offset:" #OFFB "+12288\n\t" OP " %8, %7 offset:" #OFFB \
                    "+14336\n\t"                                                                                        \
                 :                                                                                                      \
                 : "v"(R0[0]), "v"(R0[1]), "v"(R0[2]), "v"(R0[3]), "v"(R0[4]), "v"(R0[5]), "v"(R0[6]), "v"(R0[7]), "v"(addr) \
                 : "memory")
    using i32x2 = int __attribute__((ext_vector_type(2)));
    // Direct global -> LDS loads and nothing else: every workgroup walks the K stages of a 256 x 256 tile of the 8192^3
    // 1-byte GEMM (64 KiB per stage: 8 + 8 loads of 1 KiB per wave), the tiles in the library's own order, DEPTH stages in
    // flight.  PATTERN 0: K-contiguous operands with `pitch` bytes per row (a load touches 8 rows x 128 bytes);
    // 1: K-blocked operands (a tile's share of a stage is 32 KiB of consecutive bytes); 2: pattern 0 with every workgroup on
    // tile (0, 0) (no L2 misses).
    // SOLO: 96 KiB of LDS per workgroup, so that a CU holds one workgroup and DEPTH x 64 KiB is all it has in flight.
    template <int DEPTH, int PATTERN, bool SOLO = false>
    __global__ void __launch_bounds__(256) fillLoop(const char* a, const char* b, uint32_t pitch, uint32_t stages, uint32_t tiles)
    {
        __shared__ __attribute__((aligned(1024))) char lds[SOLO ? 98304 : 65536];
        uint32_t tm = 0, tn = 0;
        if(!r355::tileCoordRange(blockIdx.x, tiles, tiles, 0u, tiles * tiles, false, tm, tn))
            return;
        if(PATTERN == 2)
            tm = tn = 0;
        const uint32_t tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) char*)lds));
        uint32_t       off[8];
        uint32_t       stageStride;
        uint64_t       panel;
        if(PATTERN == 1)
        {
            for(uint32_t j = 0; j < 8; ++j)
                off[j] = j * 4096u + tid * 16u;
            stageStride = 32768u;
            panel       = (uint64_t)stages * 32768u; // a tile row's K stages, one after the other
        }
        else
        {
            for(uint32_t j = 0; j < 8; ++j)
                off[j] = ((tid >> 3) + 32u * j) * pitch + (tid & 7u) * 16u;
            stageStride = 128u;
            panel       = 256ull * pitch;
        }
        const r355::dma_i32x4 ra = r355::rawBuffer(r355::uniformAddress(a + tm * panel));
        const r355::dma_i32x4 rb = r355::rawBuffer(r355::uniformAddress(b + tn * panel));
        for(uint32_t st = 0; st < stages; ++st)
        {
#pragma unroll
            for(uint32_t j = 0; j < 8; ++j)
                r355::loadToLds(ra, off[j], st * stageStride, ldsBase + wave * 1024u + j * 4096u);
#pragma unroll
            for(uint32_t j = 0; j < 8; ++j)
                r355::loadToLds(rb, off[j], st * stageStride, ldsBase + 32768u + wave * 1024u + j * 4096u);
            r355::waitVmcnt<16 * (DEPTH - 1)>();
        }
        r355::waitVmcnt<0>();
    }


    // Global stores alone, in the shape of the macro-tile epilogue: every workgroup of 4 waves writes a 256 x 256 tile of
    // 4-byte elements (256 KiB) of a row-major matrix with `pitch` bytes per row, 16 bytes per lane; a wave owns a
    // 128 x 128 quarter and one store instruction covers SEG consecutive bytes of 1024 / SEG rows.  NT: nontemporal.
    template <uint32_t SEG, bool NT>
    __global__ void __launch_bounds__(256) storeLoop(char* d, uint32_t pitch, uint32_t tiles, unsigned long long* cyc)
    {
        uint32_t tm = 0, tn = 0;
        if(!r355::tileCoordRange(blockIdx.x, tiles, tiles, 0u, tiles * tiles, false, tm, tn))
            return;
        using v4            = int __attribute__((ext_vector_type(4)));
        const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
        const uint32_t wm = wave >> 1, wn = wave & 1u;
        constexpr uint32_t LPR = SEG / 16u, ROWS = 64u / LPR; // lanes per row, rows per instruction
        char* base = d + ((uint64_t)tm * 256u + wm * 128u) * pitch + (tn * 256u + wn * 128u) * 4u;
        const v4 v = {(int)lane, (int)wave, (int)tm, (int)tn};
        const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
#pragma unroll 8
        for(uint32_t it = 0; it < 65536u / 1024u; ++it)
        {
            // 512 bytes per row of the wave tile: SEG-byte segment s of row r
            const uint32_t unit = it * ROWS + lane / LPR; // (row, segment) pairs in row-major order
            const uint32_t row = unit / (512u / SEG), seg = unit % (512u / SEG);
            v4* at = reinterpret_cast<v4*>(base + (uint64_t)row * pitch + seg * SEG + (lane % LPR) * 16u);
            if(NT)
                __builtin_nontemporal_store(v, at);
            else
                *at = v;
        }
        __builtin_amdgcn_s_waitcnt(0);
        const unsigned long long t1 = __builtin_amdgcn_s_memrealtime();
        if(threadIdx.x == 0)
            atomicMax(cyc, t1 - t0);
    }


    template <int MODE>
    __global__ void __launch_bounds__(256) ldsReadLoop(int* out, int iters, unsigned long long* cyc)
    {
        __shared__ __attribute__((aligned(16))) char lds[65536];
        const int t = threadIdx.x;
        for(int i = t; i < 65536 / 4; i += blockDim.x)
            reinterpret_cast<int*>(lds)[i] = i;
        __syncthreads();
        const uint32_t           addr = ((MODE == 0 || MODE == 5) ? t * 16 : ((MODE == 3 || MODE == 7) ? t * 4 : t * 8)) & 2047;
        const unsigned long long c0   = __builtin_readcyclecounter();
        int                      s    = 0;
        if constexpr(MODE == 0)
        {
            i32x4 x[8], y[8];
            for(int it = 0; it < iters; ++it)
            {
                R355_RD8("ds_read_b128", x, 0);
                asm volatile("s_waitcnt lgkmcnt(8)");
                R355_RD8("ds_read_b128", y, 16384);
                asm volatile("s_waitcnt lgkmcnt(8)");
            }
            asm volatile("s_waitcnt lgkmcnt(0)");
            for(int i = 0; i < 8; ++i)
                s ^= x[i][0] ^ y[i][3];
        }
        else if constexpr(MODE >= 5)
        {
            // writes: the same addresses and pacing, data from registers that never change
            using W = std::conditional_t<MODE == 5, i32x4, std::conditional_t<MODE == 6, i32x2, int>>;
            W x[8];
            for(int i = 0; i < 8; ++i)
                x[i] = W{} + (t + i);
            for(int it = 0; it < iters; ++it)
            {
                if constexpr(MODE == 5)
                {
                    R355_WR8("ds_write_b128", x, 0);
                    asm volatile("s_waitcnt lgkmcnt(8)");
                    R355_WR8("ds_write_b128", x, 16384);
                }
                else if constexpr(MODE == 6)
                {
                    R355_WR8("ds_write_b64", x, 0);
                    asm volatile("s_waitcnt lgkmcnt(8)");
                    R355_WR8("ds_write_b64", x, 16384);
                }
                else
                {
                    R355_WR8("ds_write_b32", x, 0);
                    asm volatile("s_waitcnt lgkmcnt(8)");
                    R355_WR8("ds_write_b32", x, 16384);
                }
                asm volatile("s_waitcnt lgkmcnt(8)");
            }
            asm volatile("s_waitcnt lgkmcnt(0)");
            __syncthreads();
            s = reinterpret_cast<const int*>(lds)[t];
        }
        else if constexpr(MODE == 3)
        {
            int x[8], y[8];
            for(int it = 0; it < iters; ++it)
            {
                R355_RD8("ds_read_b32", x, 0);
                asm volatile("s_waitcnt lgkmcnt(8)");
                R355_RD8("ds_read_b32", y, 16384);
                asm volatile("s_waitcnt lgkmcnt(8)");
            }
            asm volatile("s_waitcnt lgkmcnt(0)");
            for(int i = 0; i < 8; ++i)
                s ^= x[i] ^ y[i];
        }
        else
        {
            i32x2 x[8], y[8];
            for(int it = 0; it < iters; ++it)
            {
                if constexpr(MODE == 1)
                {
                    R355_RD8("ds_read_b64", x, 0);
                    asm volatile("s_waitcnt lgkmcnt(8)");
                    R355_RD8("ds_read_b64", y, 16384);
                }
                else if constexpr(MODE == 2)
                {
                    R355_RD8("ds_read_b64_tr_b16", x, 0);
                    asm volatile("s_waitcnt lgkmcnt(8)");
                    R355_RD8("ds_read_b64_tr_b16", y, 16384);
                }
                else
                {
                    R355_RD8("ds_read_b64_tr_b8", x, 0);
                    asm volatile("s_waitcnt lgkmcnt(8)");
                    R355_RD8("ds_read_b64_tr_b8", y, 16384);
                }
                asm volatile("s_waitcnt lgkmcnt(8)");
            }
            asm volatile("s_waitcnt lgkmcnt(0)");
            for(int i = 0; i < 8; ++i)
                s ^= x[i][0] ^ y[i][1];
        }
        const unsigned long long c1 = __builtin_readcyclecounter();
        out[blockIdx.x * 256 + t]   = s;
        if(t == 0 && blockIdx.x == 0)
            cyc[0] = c1 - c0;
    }

    // A wave reads seven 1 KiB pieces of a unit with nontemporal loads, adds them up and writes 1 KiB; UNITS consecutive units
    // per wave, the next one requested before (AHEAD) or after the current one is written.
    template <int UNITS, bool AHEAD>
    __global__ void __launch_bounds__(256) mixKernel(const f32x4* __restrict__ in, f32x4* __restrict__ out, uint32_t units)
    {
        const uint32_t lane = threadIdx.x & 63u, first = (blockIdx.x * 4u + (threadIdx.x >> 6)) * UNITS;
        f32x4          cur[7], nxt[7];
        auto           load = [&](f32x4(&d)[7], uint32_t u) {
#pragma unroll
            for(int i = 0; i < 7; ++i)
                d[i] = __builtin_nontemporal_load(in + (size_t)u * 448u + i * 64u + lane);
        };
        if(first >= units)
            return;
        load(cur, first);
        for(int i = 0; i < UNITS && first + i < units; ++i)
        {
            const uint32_t u    = first + i;
            const bool     more = i + 1 < UNITS && u + 1u < units;
            if(AHEAD && more)
                load(nxt, u + 1u);
            f32x4 acc = cur[0];
#pragma unroll
            for(int j = 1; j < 7; ++j)
                acc += cur[j];
            __builtin_nontemporal_store(acc, out + (size_t)u * 64u + lane);
            if(!AHEAD && more)
                load(nxt, u + 1u);
#pragma unroll
            for(int j = 0; j < 7; ++j)
                cur[j] = nxt[j];
        }
    }

    __global__ void copyKernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n)
    {
        for(size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
            dst[i] = src[i];
    }
} // namespace

int main(int argc, char** argv)
{
    if(argc < 2)
    {
        fprintf(stderr, "usage: host_bench gemm|dlrm|gemv|copy|mix|mfma|lds|fill|store [options]\n");
        return 2;
    }
    const std::string op = argv[1];
    std::string       type = "f16", out = "", layout = "nt", kernel = "auto";
    bool              sparse = false, itersSet = false, bwd = false, zeroFill = false, split = false;
    uint32_t          m = 8192, n = 8192, k = 8192, batch = 65536, ldpad = 0;
    bool              mSet = false, kSet = false;
    int               warmup = 2, iters = 10;
    size_t            bytes = 1ull << 30, workspaceMiB = 0;
    for(int i = 2; i + 1 < argc; i += 2)
    {
        const std::string a = argv[i], v = argv[i + 1];
        if(a == "--type") type = v;
        else if(a == "--out") out = v;
        else if(a == "--layout") layout = v;
        else if(a == "--kernel") kernel = v;
        else if(a == "--m") m = atoi(v.c_str()), mSet = true;
        else if(a == "--n") n = atoi(v.c_str());
        else if(a == "--k") k = atoi(v.c_str()), kSet = true;
        else if(a == "--batch") batch = atoi(v.c_str());
        else if(a == "--ldpad") ldpad = atoi(v.c_str()); // elements added to lda and ldb (dense GEMM)
        else if(a == "--warmup") warmup = atoi(v.c_str());
        else if(a == "--iters") iters = atoi(v.c_str()), itersSet = true;
        else if(a == "--sparse") sparse = atoi(v.c_str()) != 0;
        else if(a == "--split") split = atoi(v.c_str()) != 0;
        else if(a == "--bwd") bwd = atoi(v.c_str()) != 0;
        else if(a == "--zero") zeroFill = atoi(v.c_str()) != 0;
        else if(a == "--workspace") workspaceMiB = strtoull(v.c_str(), nullptr, 10);
        else if(a == "--bytes") bytes = strtoull(v.c_str(), nullptr, 10);
        else
        {
            fprintf(stderr, "unknown option %s\n", a.c_str());
            return 2;
        }
    }
    r355_device_info dev;
    if(r355_get_device_info(&dev) != R355_OK)
    {
        fprintf(stderr, "%s\n", r355_last_error());
        return 1;
    }
    float ms = 0.0f;

    if(op == "gemm")
    {
        const int inT = parseType(type);
        if(out.empty())
            out = inT == R355_I8 ? "i32" : (inT == R355_E4M3 ? "f32" : type);
        const int outT = parseType(out);
        r355_gemm_args g;
        memset(&g, 0, sizeof(g));
        g.in_type = inT, g.out_type = outT;
        g.layout_a = layout[0] == 't' ? R355_ROW_MAJOR : R355_COL_MAJOR; // BLAS letters: T = row-major A
        g.layout_b = layout[1] == 't' ? R355_ROW_MAJOR : R355_COL_MAJOR;
        g.layout_c = g.layout_d = R355_ROW_MAJOR;
        g.m = m, g.n = n, g.k = k;
        g.lda = (g.layout_a == R355_ROW_MAJOR ? k : m) + ldpad;
        g.ldb = (g.layout_b == R355_ROW_MAJOR ? n : k) + ldpad;
        g.ldc = g.ldd = n;
        g.alpha = 1.0, g.beta = 0.0;
        g.kernel = kernel == "simple"     ? R355_KERNEL_SIMPLE
                   : kernel == "tiled"    ? R355_KERNEL_TILED
                   : kernel == "tiled128" ? R355_KERNEL_TILED_128
                   : kernel == "deep"     ? R355_KERNEL_TILED_DEEP
                                          : R355_KERNEL_AUTO;
        const size_t rowsA = g.layout_a == R355_ROW_MAJOR ? m : k, rowsB = g.layout_b == R355_ROW_MAJOR ? k : n;
        std::vector<uint8_t> ha(sparse ? (size_t)m * k * bytesOf(inT) / 2 : rowsA * g.lda * bytesOf(inT)),
            hb(rowsB * g.ldb * bytesOf(inT));
        if(!zeroFill)
        {
            fillBytes(ha, inT, 1);
            fillBytes(hb, inT, 2);
        }
        void *da, *db, *dd, *dmeta = nullptr;
        if(sparse)
        {
            // compressed A: m * k/2 kept values in the K-blocked storage (any bytes are valid values); one index nibble per group of four dense columns:
            // 0x4 keeps positions (0, 1), 0x8 keeps positions (0, 2)
            g.sparse24 = 1;
            g.lda      = k / 2;
            std::vector<uint8_t> hm((size_t)m * k / 8, 0x84);
            HIP_OK(hipMalloc(&dmeta, hm.size()));
            HIP_OK(hipMemcpy(dmeta, hm.data(), hm.size(), hipMemcpyHostToDevice));
            g.a_meta = dmeta;
        }
        HIP_OK(hipMalloc(&da, ha.size()));
        HIP_OK(hipMalloc(&db, hb.size()));
        HIP_OK(hipMalloc(&dd, (size_t)m * n * bytesOf(outT)));
        HIP_OK(hipMemcpy(da, ha.data(), ha.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(db, hb.data(), hb.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemset(dd, 0xFF, (size_t)m * n * bytesOf(outT))); // NaN-prefill as the reference does
        g.a = da, g.b = db, g.d = dd;
        if(workspaceMiB)
        {
            HIP_OK(hipMalloc(&g.workspace, workspaceMiB << 20));
            g.workspace_bytes = workspaceMiB << 20;
        }
        r355_gemm_plan plan;
        if(r355_gemm_query(&g, &plan) != R355_OK || r355_gemm_timed(&g, nullptr, warmup, iters, &ms) != R355_OK)
        {
            fprintf(stderr, "%s\n", r355_last_error());
            return 1;
        }
        const double flop   = 2.0 * m * n * k;
        const double tflops = flop / ms / 1e9;
        const double vendor = (inT == R355_F64   ? 78.6
                               : inT == R355_F32 ? 157.3
                               : (inT == R355_I8 || inT == R355_E4M3) ? 5000.0
                                                                      : 2500.0)
                              * (sparse ? 2.0 : 1.0);
        const double perClk = inT == R355_F64 ? 128.0 : inT == R355_F32 ? 256.0 : (inT == R355_I8 || inT == R355_E4M3) ? 8192.0 : 4096.0; // flop / CU / clk
        const double model  = perClk * dev.compute_units * dev.clock_mhz * 1e-6; // TFLOP/s at the reported clock
        printf("{\"op\": \"%s\", \"type\": \"%s\", \"out\": \"%s\", \"layout\": \"%s\", \"m\": %u, \"n\": %u, \"k\": %u, "
               "\"kernel\": %d, \"macro_tile\": [%u, %u, %u], \"split_k\": %u, \"lds_bytes\": %u, \"ms\": %.4f, \"tflops\": %.1f, "
               "\"frac_vendor_peak\": %.4f, \"frac_clock_model_peak\": %.4f, \"cus\": %d, \"clock_mhz\": %d}\n",
               sparse ? "gemm_sparse24" : "gemm", type.c_str(), out.c_str(), layout.c_str(), m, n, k, plan.kernel, plan.macro_tile_m, plan.macro_tile_n,
               plan.macro_tile_k, plan.split_k, plan.lds_bytes, ms, tflops, tflops / vendor, tflops / model, dev.compute_units,
               dev.clock_mhz);
    }
    else if(op == "dlrm")
    {
        if(!mSet) m = 27;
        if(!kSet) k = 128;
        const size_t inElems = (size_t)batch * m * k, outElems = (size_t)batch * (k + m * (m - 1) / 2);
        const int    dt = parseType(type);
        const size_t es = bytesOf(dt);
        std::vector<uint8_t> hx(inElems * es);
        fillBytes(hx, dt, 3);
        void *dx, *dout;
        HIP_OK(hipMalloc(&dx, hx.size()));
        HIP_OK(hipMalloc(&dout, outElems * es));
        HIP_OK(hipMemcpy(dx, hx.data(), hx.size(), hipMemcpyHostToDevice));
        if(bwd)
        {
            // upstream gradient has the forward output's shape; outputs: mlp gradient [batch][k]
            // and input gradient [batch][m][k]
            std::vector<uint8_t> hu(outElems * es);
            fillBytes(hu, dt, 9);
            void *dmlp, *dgrad;
            HIP_OK(hipMemcpy(dout, hu.data(), hu.size(), hipMemcpyHostToDevice));
            HIP_OK(hipMalloc(&dmlp, (size_t)batch * k * es));
            HIP_OK(hipMalloc(&dgrad, inElems * es));
            hipEvent_t e0, e1;
            HIP_OK(hipEventCreate(&e0));
            HIP_OK(hipEventCreate(&e1));
            for(int i = 0; i < warmup + iters; ++i)
            {
                if(i == warmup)
                    HIP_OK(hipEventRecord(e0));
                if(r355_dlrm_bwd(dt, dx, dout, dmlp, dgrad, m, k, batch, nullptr) != R355_OK)
                {
                    fprintf(stderr, "%s\n", r355_last_error());
                    return 1;
                }
            }
            HIP_OK(hipEventRecord(e1));
            HIP_OK(hipEventSynchronize(e1));
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
            ms /= iters;
            const double byts = (double)(2 * inElems + outElems + (size_t)batch * k) * es;
            printf("{\"op\": \"dlrm_bwd\", \"type\": \"%s\", \"batch\": %u, \"m\": %u, \"k\": %u, \"ms\": %.4f, \"gbps\": %.1f, "
                   "\"frac_hbm_peak\": %.4f}\n",
                   type.c_str(), batch, m, k, ms, byts / ms / 1e6, byts / ms / 1e6 / 8000.0);
            return 0;
        }
        if(r355_dlrm_fwd_timed(dt, dx, dout, m, k, batch, nullptr, warmup, iters, &ms) != R355_OK)
        {
            fprintf(stderr, "%s\n", r355_last_error());
            return 1;
        }
        const double byts = (double)(inElems + outElems) * es;
        printf("{\"op\": \"dlrm_fwd\", \"type\": \"%s\", \"batch\": %u, \"m\": %u, \"k\": %u, \"ms\": %.4f, \"gbps\": %.1f, "
               "\"frac_hbm_peak\": %.4f, \"gflops_ref_convention\": %.1f}\n",
               type.c_str(), batch, m, k, ms, byts / ms / 1e6, byts / ms / 1e6 / 8000.0,
               2.0 * m * m * k * batch / ms / 1e6);
    }
    else if(op == "gemv")
    {
        if(!mSet) m = 8192;
        if(!kSet) k = 8192;
        std::vector<uint8_t> ha((size_t)m * k * 4), hx((size_t)k * 4);
        fillBytes(ha, R355_F32, 4);
        fillBytes(hx, R355_F32, 5);
        void *da, *dx, *dy;
        HIP_OK(hipMalloc(&da, ha.size()));
        HIP_OK(hipMalloc(&dx, hx.size()));
        HIP_OK(hipMalloc(&dy, (size_t)m * 4));
        HIP_OK(hipMemcpy(da, ha.data(), ha.size(), hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dx, hx.data(), hx.size(), hipMemcpyHostToDevice));
        const int    lay = layout[0] == 't' ? R355_ROW_MAJOR : R355_COL_MAJOR;
        const size_t wsBytes = split ? r355_gemv_workspace_bytes(lay, m, k, 4) : 0;
        if(wsBytes)
        {
            void* ws = nullptr;
            HIP_OK(hipMalloc(&ws, wsBytes));
            hipEvent_t e0, e1;
            HIP_OK(hipEventCreate(&e0));
            HIP_OK(hipEventCreate(&e1));
            for(int it = 0; it < warmup + iters; ++it)
            {
                if(it == warmup)
                    HIP_OK(hipEventRecord(e0));
                if(r355_gemv_ws(lay, m, k, (const float*)da, lay == R355_ROW_MAJOR ? k : m, (const float*)dx, nullptr, (float*)dy, 1.0f,
                                0.0f, ws, wsBytes, nullptr)
                   != R355_OK)
                {
                    fprintf(stderr, "%s\n", r355_last_error());
                    return 1;
                }
            }
            HIP_OK(hipEventRecord(e1));
            HIP_OK(hipEventSynchronize(e1));
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
            ms /= (float)iters;
        }
        else if(r355_gemv_timed(lay, m, k, (const float*)da, lay == R355_ROW_MAJOR ? k : m, (const float*)dx, nullptr,
                                (float*)dy, 1.0f, 0.0f, nullptr, warmup, iters, &ms)
                != R355_OK)
        {
            fprintf(stderr, "%s\n", r355_last_error());
            return 1;
        }
        const double byts = (double)m * k * 4.0 + (double)(m + k) * 4.0;
        printf("{\"op\": \"gemv\", \"m\": %u, \"k\": %u, \"layout\": \"%s\", \"workspace_bytes\": %zu, \"ms\": %.4f, \"gbps\": %.1f, "
               "\"frac_hbm_peak\": %.4f}\n",
               m, k, lay == R355_ROW_MAJOR ? "row" : "col", wsBytes, ms, byts / ms / 1e6, byts / ms / 1e6 / 8000.0);
    }
    else if(op == "mfma")
    {
        const int loops = itersSet ? iters : 20000;
        i32x4*    in;
        float*    outBuf;
        HIP_OK(hipMalloc(&in, 1024 * sizeof(i32x4)));
        HIP_OK(hipMalloc(&outBuf, (size_t)dev.compute_units * 256 * sizeof(float)));
        hipEvent_t e0, e1;
        HIP_OK(hipEventCreate(&e0));
        HIP_OK(hipEventCreate(&e1));
        static const char*  names[MF_KINDS] = {"f16 32x32x16", "bf16 32x32x16", "i8 32x32x32", "fp8 f8f6f4 32x32x64",
                                               "sparse i8 smfmac 32x32x64 (dense-equivalent ops)", "f16 16x16x32",
                                               "i8 16x16x64", "fp8 f8f6f4 16x16x128",
                                               "sparse i8 smfmac 16x16x128 (dense-equivalent ops)",
                                               "sparse fp8 smfmac 16x16x128 (dense-equivalent ops)"};
        // flop per loop trip and wave: 16 instructions of the 32 x 32 shapes, 64 of the 16 x 16 shapes
        static const double flopPer[MF_KINDS]
            = {2.0 * 32 * 32 * 16, 2.0 * 32 * 32 * 16, 2.0 * 32 * 32 * 32, 2.0 * 32 * 32 * 64, 2.0 * 32 * 32 * 64,
               4 * 2.0 * 16 * 16 * 32, 4 * 2.0 * 16 * 16 * 64, 4 * 2.0 * 16 * 16 * 128, 4 * 2.0 * 16 * 16 * 128,
               4 * 2.0 * 16 * 16 * 128};
        static const double vendorPeak[MF_KINDS] = {2500.0, 2500.0, 5000.0, 5000.0, 10000.0, 2500.0, 5000.0, 5000.0, 10000.0, 10000.0};
        printf("[");
        for(int random = 0; random < 2; ++random)
            for(int kind = 0; kind < MF_KINDS; ++kind)
            {
                std::vector<uint32_t> h(4096, 0u);
                for(size_t i = 0; random && i < h.size(); ++i)
                {
                    const uint32_t r = static_cast<uint32_t>(splitmix(7 + kind, i));
                    h[i] = kind == MF_F16    ? ((r & 0x8FFF8FFFu) | 0x30003000u)  // |x| in [1/8, 1)
                           : kind == MF_BF16 ? ((r & 0x807F807Fu) | 0x3E003E00u)  // |x| in [1/8, 1/4)
                           : kind == MF_F16_16 ? ((r & 0x8FFF8FFFu) | 0x30003000u)
                           : (kind == MF_FP8_K64 || kind == MF_FP8_16 || kind == MF_SPARSE_FP8_16) ? ((r & 0x87878787u) | 0x30303030u) // |x| in [1/2, 1)
                                                : r;
                }
                HIP_OK(hipMemcpy(in, h.data(), h.size() * 4, hipMemcpyHostToDevice));
                launchMfma(kind, dev.compute_units, in, outBuf, 1000);
                HIP_OK(hipDeviceSynchronize());
                HIP_OK(hipEventRecord(e0));
                launchMfma(kind, dev.compute_units, in, outBuf, loops);
                HIP_OK(hipEventRecord(e1));
                HIP_OK(hipEventSynchronize(e1));
                HIP_OK(hipEventElapsedTime(&ms, e0, e1));
                const double tf = (double)dev.compute_units * 4 * loops * 16 * flopPer[kind] / ms / 1e9;
                printf("%s\n {\"op\": \"mfma\", \"instr\": \"%s\", \"operands\": \"%s\", \"ms\": %.3f, \"tflops\": %.1f, "
                       "\"frac_vendor_peak\": %.4f}",
                       (random || kind) ? "," : "", names[kind], random ? "random" : "zero", ms, tf, tf / vendorPeak[kind]);
            }
        printf("\n]\n");
    }
    else if(op == "lds")
    {
        // wave-level read instructions per shader clock and bytes per clock per CU, with 4, 2 and 1 waves per CU reading
        int*                out;
        unsigned long long* cyc;
        HIP_OK(hipMalloc(&out, (size_t)dev.compute_units * 256 * sizeof(int)));
        HIP_OK(hipMalloc(&cyc, 64));
        const int          loops   = itersSet ? iters : 4000;
        static const char* names[] = {"ds_read_b128", "ds_read_b64", "ds_read_b64_tr_b16", "ds_read_b32", "ds_read_b64_tr_b8",
                                      "ds_write_b128", "ds_write_b64", "ds_write_b32"};
        static const int   width[] = {16, 8, 8, 4, 8, 16, 8, 4};
        printf("[");
        for(int waves = 4; waves >= 1; waves /= 2)
            for(int mode = 0; mode < 8; ++mode)
            {
                for(int rep = 0; rep < 2; ++rep)
                {
                    const dim3 g(dev.compute_units), b(64 * waves);
                    switch(mode)
                    {
                    case 0: hipLaunchKernelGGL(ldsReadLoop<0>, g, b, 0, 0, out, loops, cyc); break;
                    case 1: hipLaunchKernelGGL(ldsReadLoop<1>, g, b, 0, 0, out, loops, cyc); break;
                    case 2: hipLaunchKernelGGL(ldsReadLoop<2>, g, b, 0, 0, out, loops, cyc); break;
                    case 3: hipLaunchKernelGGL(ldsReadLoop<3>, g, b, 0, 0, out, loops, cyc); break;
                    case 4: hipLaunchKernelGGL(ldsReadLoop<4>, g, b, 0, 0, out, loops, cyc); break;
                    case 5: hipLaunchKernelGGL(ldsReadLoop<5>, g, b, 0, 0, out, loops, cyc); break;
                    case 6: hipLaunchKernelGGL(ldsReadLoop<6>, g, b, 0, 0, out, loops, cyc); break;
                    default: hipLaunchKernelGGL(ldsReadLoop<7>, g, b, 0, 0, out, loops, cyc); break;
                    }
                    HIP_OK(hipDeviceSynchronize());
                }
                unsigned long long clocks = 0;
                HIP_OK(hipMemcpy(&clocks, cyc, 8, hipMemcpyDeviceToHost));
                const double reads = 16.0 * loops * waves; // wave-level instructions per CU
                printf("%s\n {\"op\": \"lds\", \"instr\": \"%s\", \"waves_per_cu\": %d, \"clocks_per_wave_read\": %.2f, "
                       "\"bytes_per_clock_per_cu\": %.1f}",
                       (waves == 4 && mode == 0) ? "" : ",", names[mode], waves, clocks / reads, reads * 64 * width[mode] / clocks);
            }
        printf("\n]\n");
    }
    else if(op == "fill")
    {
        // aggregate rate of direct global -> LDS loads in the access stream of the 8192^3 1-byte GEMM (no matrix instructions,
        // no LDS reads, no stores): 1024 tiles x 64 stages x 64 KiB
        const uint32_t tiles = 32, stages = 64;
        const size_t   pitchMax = 8192 + 128;
        void *         pa, *pb;
        HIP_OK(hipMalloc(&pa, 8192 * pitchMax));
        HIP_OK(hipMalloc(&pb, 8192 * pitchMax));
        HIP_OK(hipMemset(pa, 1, 8192 * pitchMax));
        HIP_OK(hipMemset(pb, 2, 8192 * pitchMax));
        hipEvent_t e0, e1;
        HIP_OK(hipEventCreate(&e0));
        HIP_OK(hipEventCreate(&e1));
        const char* names[5] = {"K-contiguous rows, pitch 8192", "K-contiguous rows, pitch 8320", "K-blocked (32 KiB runs)",
                                "every workgroup on tile (0, 0)", "K-contiguous rows, pitch 8192, one workgroup per CU"};
        printf("[");
        for(int pat = 0; pat < 5; ++pat)
            for(int depth = 1; depth <= 3; ++depth)
            {
                const uint32_t pitch = pat == 1 ? 8320u : 8192u;
                auto           go    = [&] {
                    const dim3 g(tiles * tiles), blk(256);
                    const char *a = static_cast<const char*>(pa), *b = static_cast<const char*>(pb);
#define R355_FILL(D, P) hipLaunchKernelGGL((fillLoop<D, P>), g, blk, 0, 0, a, b, pitch, stages, tiles)
                    const int p = pat == 0 || pat == 1 ? 0 : pat - 1;
                    if(pat == 4)
                    {
                        if(depth == 1)
                            hipLaunchKernelGGL((fillLoop<1, 0, true>), g, blk, 0, 0, a, b, pitch, stages, tiles);
                        else if(depth == 2)
                            hipLaunchKernelGGL((fillLoop<2, 0, true>), g, blk, 0, 0, a, b, pitch, stages, tiles);
                        else
                            hipLaunchKernelGGL((fillLoop<3, 0, true>), g, blk, 0, 0, a, b, pitch, stages, tiles);
                    }
                    else if(depth == 1) { if(p == 0) R355_FILL(1, 0); else if(p == 1) R355_FILL(1, 1); else R355_FILL(1, 2); }
                    else if(depth == 2) { if(p == 0) R355_FILL(2, 0); else if(p == 1) R355_FILL(2, 1); else R355_FILL(2, 2); }
                    else { if(p == 0) R355_FILL(3, 0); else if(p == 1) R355_FILL(3, 1); else R355_FILL(3, 2); }
#undef R355_FILL
                };
                for(int i = 0; i < 20; ++i)
                    go();
                HIP_OK(hipEventRecord(e0));
                for(int i = 0; i < 20; ++i)
                    go();
                HIP_OK(hipEventRecord(e1));
                HIP_OK(hipEventSynchronize(e1));
                HIP_OK(hipEventElapsedTime(&ms, e0, e1));
                ms /= 20;
                const double bytes = (double)tiles * tiles * stages * 65536.0;
                const double rounds = (double)tiles * tiles / dev.compute_units;
                printf("%s\n {\"op\": \"fill\", \"pattern\": \"%s\", \"stages_in_flight\": %d, \"ms\": %.4f, \"tb_per_s\": %.2f, "
                       "\"us_per_64KiB_stage_per_cu\": %.3f}",
                       (pat == 0 && depth == 1) ? "" : ",", names[pat], depth, ms, bytes / ms / 1e9, ms * 1e3 / (rounds * stages));
            }
        printf("\n]\n");
    }
    else if(op == "store")
    {
        // epilogue-shaped global stores alone: 1, 64, 256 or 1024 tiles of 256 KiB
        void* pd;
        const size_t pitch = 8192 * 4;
        HIP_OK(hipMalloc(&pd, 8192 * pitch));
        unsigned long long* cyc;
        HIP_OK(hipMalloc(&cyc, 8));
        hipEvent_t e0, e1;
        HIP_OK(hipEventCreate(&e0));
        HIP_OK(hipEventCreate(&e1));
        printf("[");
        bool first = true;
        for(uint32_t tiles : {1u, 8u, 16u, 32u})
            for(int var = 0; var < 6; ++var)
            {
                auto go = [&] {
                    const dim3 g(((tiles * tiles + 7u) / 8u) * 8u), blk(256);
                    char*      d = static_cast<char*>(pd);
                    switch(var)
                    {
                    case 0: hipLaunchKernelGGL((storeLoop<512, true>), g, blk, 0, 0, d, (uint32_t)pitch, tiles, cyc); break;
                    case 1: hipLaunchKernelGGL((storeLoop<512, false>), g, blk, 0, 0, d, (uint32_t)pitch, tiles, cyc); break;
                    case 2: hipLaunchKernelGGL((storeLoop<256, true>), g, blk, 0, 0, d, (uint32_t)pitch, tiles, cyc); break;
                    case 3: hipLaunchKernelGGL((storeLoop<128, true>), g, blk, 0, 0, d, (uint32_t)pitch, tiles, cyc); break;
                    case 4: hipLaunchKernelGGL((storeLoop<64, true>), g, blk, 0, 0, d, (uint32_t)pitch, tiles, cyc); break;
                    default: hipLaunchKernelGGL((storeLoop<64, false>), g, blk, 0, 0, d, (uint32_t)pitch, tiles, cyc); break;
                    }
                };
                const char* names[6] = {"512 B x 2 rows, nontemporal", "512 B x 2 rows, plain", "256 B x 4 rows, nontemporal",
                                        "128 B x 8 rows, nontemporal", "64 B x 16 rows, nontemporal", "64 B x 16 rows, plain"};
                for(int i = 0; i < 10; ++i)
                    go();
                HIP_OK(hipMemset(cyc, 0, 8));
                HIP_OK(hipEventRecord(e0));
                for(int i = 0; i < 20; ++i)
                    go();
                HIP_OK(hipEventRecord(e1));
                HIP_OK(hipEventSynchronize(e1));
                HIP_OK(hipEventElapsedTime(&ms, e0, e1));
                ms /= 20;
                unsigned long long worst = 0;
                HIP_OK(hipMemcpy(&worst, cyc, 8, hipMemcpyDeviceToHost));
                printf("%s\n {\"op\": \"store\", \"tiles\": %u, \"instruction\": \"%s\", \"ms_per_launch\": %.4f, "
                       "\"slowest_workgroup_us\": %.2f, \"tb_per_s\": %.2f}",
                       first ? "" : ",", tiles * tiles, names[var], ms, worst / 100.0, tiles * tiles * 262144.0 / ms / 1e9);
                first = false;
            }
        printf("\n]\n");
    }
    else if(op == "copy")
    {
        void *src, *dst;
        HIP_OK(hipMalloc(&src, bytes));
        HIP_OK(hipMalloc(&dst, bytes));
        HIP_OK(hipMemset(src, 1, bytes));
        hipEvent_t e0, e1;
        HIP_OK(hipEventCreate(&e0));
        HIP_OK(hipEventCreate(&e1));
        for(int i = 0; i < warmup; ++i)
            hipLaunchKernelGGL(copyKernel, dim3(4096), dim3(256), 0, 0, (const uint4*)src, (uint4*)dst, bytes / 16);
        HIP_OK(hipEventRecord(e0));
        for(int i = 0; i < iters; ++i)
            hipLaunchKernelGGL(copyKernel, dim3(4096), dim3(256), 0, 0, (const uint4*)src, (uint4*)dst, bytes / 16);
        HIP_OK(hipEventRecord(e1));
        HIP_OK(hipEventSynchronize(e1));
        HIP_OK(hipEventElapsedTime(&ms, e0, e1));
        ms /= iters;
        printf("{\"op\": \"copy\", \"bytes_read\": %zu, \"bytes_written\": %zu, \"ms\": %.4f, \"gbps\": %.1f}\n", bytes,
               bytes, ms, 2.0 * bytes / ms / 1e6);
    }
    else if(op == "mix")
    {
        const uint32_t units = 65536;
        void *         src, *dst;
        HIP_OK(hipMalloc(&src, (size_t)units * 7168));
        HIP_OK(hipMalloc(&dst, (size_t)units * 1024));
        HIP_OK(hipMemset(src, 1, (size_t)units * 7168));
        hipEvent_t e0, e1;
        HIP_OK(hipEventCreate(&e0));
        HIP_OK(hipEventCreate(&e1));
        auto run = [&](auto unitsPerWave, auto ahead) {
            constexpr int  U = decltype(unitsPerWave)::value;
            constexpr bool A = decltype(ahead)::value;
            const dim3     grid((units + 4 * U - 1) / (4 * U));
            for(int i = 0; i < warmup; ++i)
                hipLaunchKernelGGL((mixKernel<U, A>), grid, dim3(256), 0, 0, (const f32x4*)src, (f32x4*)dst, units);
            HIP_OK(hipEventRecord(e0));
            for(int i = 0; i < iters; ++i)
                hipLaunchKernelGGL((mixKernel<U, A>), grid, dim3(256), 0, 0, (const f32x4*)src, (f32x4*)dst, units);
            HIP_OK(hipEventRecord(e1));
            HIP_OK(hipEventSynchronize(e1));
            HIP_OK(hipEventElapsedTime(&ms, e0, e1));
            ms /= iters;
            printf("{\"op\": \"mix\", \"units_per_wave\": %d, \"next_requested_first\": %d, \"ms\": %.4f, \"gbps\": %.1f, "
                   "\"frac_hbm_peak\": %.4f}\n",
                   U, (int)A, ms, units * 8192.0 / ms / 1e6, units * 8192.0 / ms / 1e6 / 8000.0);
            return 0;
        };
        run(std::integral_constant<int, 1>{}, std::false_type{});
        run(std::integral_constant<int, 2>{}, std::true_type{});
        run(std::integral_constant<int, 2>{}, std::false_type{});
        run(std::integral_constant<int, 8>{}, std::true_type{});
        run(std::integral_constant<int, 8>{}, std::false_type{});
    }
    else
    {
        fprintf(stderr, "unknown op %s\n", op.c_str());
        return 2;
    }
    return 0;
}
