// Matrix-core dispatch for gfx950: one MFMA per K-chunk of an A/B fragment pair.
//
// The reference wraps gfx908/90a/94x instructions (mfma_impl.hpp:53-928) and unrolls
// BlockK / KPerMfma calls (mfma.hpp:49-132).  This version issues the gfx950
// double-K forms whenever the fragment's K extent allows it and falls back to the
// short-K forms for fragments declared with the reference's smaller BlockK:
//   f16   8/lane: v_mfma_f32_32x32x16_f16   / 16x16x32_f16    4/lane: 32x32x8f16 / 16x16x16f16
//   bf16  8/lane: v_mfma_f32_32x32x16_bf16  / 16x16x32_bf16   4/lane: 32x32x8bf16_1k / 16x16x16bf16_1k
//   int8 16/lane: v_mfma_i32_32x32x32_i8    / 16x16x64_i8     8/lane: 32x32x16_i8 / 16x16x32_i8
//   e4m3  8/lane: v_mfma_f32_32x32x16_fp8_fp8 / 16x16x32_fp8_fp8   (OCP encoding on gfx950); 16/lane: two of them,
//   e5m2  8/lane: v_mfma_f32_32x32x16_bf8_bf8 / 16x16x32_bf8_bf8   one per 8-byte half of the lane's K bytes
//   f32   1/lane: v_mfma_f32_32x32x2f32     / 16x16x4f32
//   f64   1/lane: v_mfma_f64_16x16x4f64 (16x16 blocks only)
#ifndef ROCWMMA_MFMA_HPP
#define ROCWMMA_MFMA_HPP

#include "layout.hpp"

namespace rocwmma
{
    namespace detail
    {
        template <uint32_t BlockDim>
        using acc_f32_t = vec_t<float, BlockDim == 32u ? 16u : 4u>;
        template <uint32_t BlockDim>
        using acc_i32_t = vec_t<int32_t, BlockDim == 32u ? 16u : 4u>;

        // One matrix instruction: acc += A(chunk) * B(chunk).  `a` / `b` point at the KW
        // elements of the chunk in the fragment's unpacked storage.
        template <typename InputT, uint32_t BlockDim, uint32_t KW>
        struct MfmaChunk
        {
            static_assert(BlockDim == 16u || BlockDim == 32u, "MFMA blocks are 16x16 or 32x32");

            using AccT = std::conditional_t<
                is_i8_v<InputT>,
                acc_i32_t<BlockDim>,
                std::conditional_t<std::is_same_v<InputT, float64_t>, vec_t<double, 4>, acc_f32_t<BlockDim>>>;

            ROCWMMA_DEVICE static inline void exec(AccT& acc, InputT const* a, InputT const* b)
            {
#if ROCWMMA_DEVICE_COMPILE
                if constexpr(is_f16_v<InputT> && KW == 8u)
                {
                    using V = vec_t<_Float16, 8>;
                    V av, bv;
                    __builtin_memcpy(&av, a, sizeof(V));
                    __builtin_memcpy(&bv, b, sizeof(V));
                    if constexpr(BlockDim == 32u)
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, bv, acc, 0, 0, 0);
                    else
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, acc, 0, 0, 0);
                }
                else if constexpr(is_f16_v<InputT> && KW == 4u)
                {
                    using V = vec_t<_Float16, 4>;
                    V av, bv;
                    __builtin_memcpy(&av, a, sizeof(V));
                    __builtin_memcpy(&bv, b, sizeof(V));
                    if constexpr(BlockDim == 32u)
                        acc = __builtin_amdgcn_mfma_f32_32x32x8f16(av, bv, acc, 0, 0, 0);
                    else
                        acc = __builtin_amdgcn_mfma_f32_16x16x16f16(av, bv, acc, 0, 0, 0);
                }
                else if constexpr(is_bf16_v<InputT> && KW == 8u)
                {
                    using V = vec_t<__bf16, 8>;
                    V av, bv;
                    __builtin_memcpy(&av, a, sizeof(V));
                    __builtin_memcpy(&bv, b, sizeof(V));
                    if constexpr(BlockDim == 32u)
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
                    else
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, acc, 0, 0, 0);
                }
                else if constexpr(is_bf16_v<InputT> && KW == 4u)
                {
                    using V = vec_t<short, 4>;
                    V av, bv;
                    __builtin_memcpy(&av, a, sizeof(V));
                    __builtin_memcpy(&bv, b, sizeof(V));
                    if constexpr(BlockDim == 32u)
                        acc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(av, bv, acc, 0, 0, 0);
                    else
                        acc = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(av, bv, acc, 0, 0, 0);
                }
                else if constexpr(is_i8_v<InputT> && KW == 16u)
                {
                    using V = vec_t<int, 4>;
                    V av, bv;
                    __builtin_memcpy(&av, a, sizeof(V));
                    __builtin_memcpy(&bv, b, sizeof(V));
                    if constexpr(BlockDim == 32u)
                        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bv, acc, 0, 0, 0);
                    else
                        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, acc, 0, 0, 0);
                }
                else if constexpr(is_i8_v<InputT> && KW == 8u)
                {
                    long av, bv;
                    __builtin_memcpy(&av, a, 8);
                    __builtin_memcpy(&bv, b, 8);
                    if constexpr(BlockDim == 32u)
                        acc = __builtin_amdgcn_mfma_i32_32x32x16_i8(av, bv, acc, 0, 0, 0);
                    else
                        acc = __builtin_amdgcn_mfma_i32_16x16x32_i8(av, bv, acc, 0, 0, 0);
                }
                else if constexpr((is_fp8_v<InputT> || is_bf8_v<InputT>) && KW == 16u)
                {
                    // K is a sum: the low 8 bytes of every lane of A meet the low 8 bytes of every lane of B in one
                    // instruction, the high 8 bytes in the next
                    MfmaChunk<InputT, BlockDim, 8u>::exec(acc, a, b);
                    MfmaChunk<InputT, BlockDim, 8u>::exec(acc, a + 8, b + 8);
                }
                else if constexpr(is_fp8_v<InputT> && KW == 8u)
                {
                    long av, bv;
                    __builtin_memcpy(&av, a, 8);
                    __builtin_memcpy(&bv, b, 8);
                    if constexpr(BlockDim == 32u)
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(av, bv, acc, 0, 0, 0);
                    else
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(av, bv, acc, 0, 0, 0);
                }
                else if constexpr(is_bf8_v<InputT> && KW == 8u)
                {
                    long av, bv;
                    __builtin_memcpy(&av, a, 8);
                    __builtin_memcpy(&bv, b, 8);
                    if constexpr(BlockDim == 32u)
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(av, bv, acc, 0, 0, 0);
                    else
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf8_bf8(av, bv, acc, 0, 0, 0);
                }
                else if constexpr(std::is_same_v<InputT, float32_t> && KW == 1u)
                {
                    if constexpr(BlockDim == 32u)
                        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(*a, *b, acc, 0, 0, 0);
                    else
                        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(*a, *b, acc, 0, 0, 0);
                }
                else if constexpr(std::is_same_v<InputT, float64_t> && KW == 1u)
                {
                    static_assert(BlockDim == 16u, "f64 matrix instructions exist for 16x16 blocks only");
                    acc = __builtin_amdgcn_mfma_f64_16x16x4f64(*a, *b, acc, 0, 0, 0);
                }
                else
                {
                    static_assert(sizeof(InputT) == 0, "no gfx950 matrix instruction for this input type / K width");
                }
#else
                (void)acc;
                (void)a;
                (void)b;
#endif
            }
        };
    } // namespace detail
} // namespace rocwmma

#endif // ROCWMMA_MFMA_HPP
