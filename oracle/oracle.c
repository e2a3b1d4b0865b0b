/*
 * CPU oracle for the fragment -> MFMA -> store hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithms of the reference's CPU
 * validators.  It is linked only by the test-suite, the smoke check and the
 * benchmark's cpu_baseline leg; the product library never links or calls it.
 *
 * Functions and the reference text they follow:
 *   orc_gemm       test/reference_impl.hpp:36-81   (gemm_CPU)
 *   orc_dlrm_fwd   test/reference_impl.hpp:83-119  (dlrm_fwd_CPU)
 *   orc_dlrm_bwd   test/reference_impl.hpp:121-179 (dlrm_bwd_CPU)
 *   orc_compare    test/common.hpp:350-444, test/device/common.hpp:111-124
 *   orc_fill_ref   test/device/common.hpp:203-220  (fillKernel input pattern)
 *   orc_e4m3_*     OCP FP8 E4M3 (bias 7, max 448, no inf, NaN = S.1111.111);
 *                  the reference takes this arithmetic from <hip/hip_fp8.h>
 *                  (library/include/rocwmma/internal/float8.hpp:118) which is
 *                  not part of the reference tree.
 *   orc_compress24 / orc_decompress24   build-defined 2:4 format; the
 *                  reference has no structured-sparse path.
 *
 * Pinning status (what checks each function against something other than
 * itself; the checks live in tests/test_oracle.py):
 *   orc_gemm      int8: numpy int64 matmul, all 16 layout combinations;
 *                 f16/bf16/f32: numpy float64 matmul on the reference's own
 *                 integer input pattern (every partial sum exact), and the
 *                 sequential-in-k f32 summation order against numpy's
 *                 sequential np.add.accumulate; alpha/beta epilogue with
 *                 power-of-two and non-power-of-two scalars against float64.
 *   orc_dlrm_fwd  the reference-held fixtures test/dlrm/data/input_fp16 ->
 *                 output_fp16 and input_fp32 -> output_fp32.
 *   orc_dlrm_bwd  the reference-held fixtures input_grad_* ->
 *                 output_input_grad_* / output_mlp_input_grad_*.
 *   orc_compare   closed-form cases (identical, one-off, inf, NaN).
 *   orc_e4m3_*    parity unpinned by the reference (its tests feed {0,-1,-2}
 *                 only); pinned by the OCP closed form over all 256 codes and
 *                 every rounding midpoint, and by agreement with torch's
 *                 independent float8_e4m3fn cast on 4e5 seeded values.
 *   orc_compress24  parity unpinned (absent from the reference); pinned by
 *                 format invariants and decompress(compress(x)) == x.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { ORC_F16 = 0, ORC_BF16 = 1, ORC_E4M3 = 2, ORC_I8 = 3, ORC_F32 = 4, ORC_I32 = 5, ORC_F64 = 6, ORC_E5M2 = 7 };
enum { ORC_ROW_MAJOR = 0, ORC_COL_MAJOR = 1 };

/* ---------------------------------------------------------------- scalars */

static inline float bits_to_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint32_t f32_to_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp  = (h >> 10) & 0x1Fu;
    uint32_t man  = h & 0x3FFu;
    if(exp == 0)
    {
        if(man == 0)
            return bits_to_f32(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return (sign ? -v : v);
    }
    if(exp == 31)
        return bits_to_f32(sign | 0x7F800000u | (man << 13));
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even, overflow -> inf (what a C cast to _Float16 does) */
uint16_t orc_f32_to_f16(float f)
{
    uint32_t u    = f32_to_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t abs  = u & 0x7FFFFFFFu;
    if(abs > 0x7F800000u)
        return (uint16_t)(sign | 0x7E00u | ((abs >> 13) & 0x3FFu)); /* NaN */
    if(abs >= 0x47800000u) /* >= 65536 -> inf (65520 rounds up below) */
        return (uint16_t)(sign | 0x7C00u);
    if(abs < 0x38800000u) /* < 2^-14: subnormal or zero */
    {
        if(abs < 0x33000000u) /* < 2^-25 -> 0 */
            return sign;
        /* value = m * 2^(e-150); target unit 2^-24 */
        uint32_t e     = abs >> 23;
        uint32_t m     = (abs & 0x7FFFFFu) | 0x800000u;
        uint32_t shift = 126u - e; /* 14..24 */
        uint32_t q     = m >> shift;
        uint32_t rem   = m & ((1u << shift) - 1u);
        uint32_t half  = 1u << (shift - 1u);
        if(rem > half || (rem == half && (q & 1u)))
            q++;
        return (uint16_t)(sign | q);
    }
    {
        uint32_t e   = (abs >> 23) - 112u;
        uint32_t m   = abs & 0x7FFFFFu;
        uint32_t q   = (e << 10) | (m >> 13);
        uint32_t rem = m & 0x1FFFu;
        if(rem > 0x1000u || (rem == 0x1000u && (q & 1u)))
            q++; /* carries into the exponent correctly, up to inf */
        return (uint16_t)(sign | q);
    }
}

float orc_bf16_to_f32(uint16_t h)
{
    return bits_to_f32((uint32_t)h << 16);
}

/* round-to-nearest-even as in hip_bfloat16(float) */
uint16_t orc_f32_to_bf16(float f)
{
    uint32_t u = f32_to_bits(f);
    if((u & 0x7FFFFFFFu) > 0x7F800000u)
        return (uint16_t)((u >> 16) | 0x40u); /* quiet NaN */
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* OCP FP8 E4M3: 1-4-3, bias 7, no infinities, NaN = 0x7F / 0xFF, max 448 */
float orc_e4m3_to_f32(uint8_t v)
{
    uint32_t sign = v >> 7;
    uint32_t exp  = (v >> 3) & 0xFu;
    uint32_t man  = v & 0x7u;
    float    r;
    if(exp == 0xFu && man == 0x7u)
        return bits_to_f32(0x7FC00000u | (sign << 31));
    if(exp == 0)
        r = (float)man * 0.001953125f; /* man * 2^-9 */
    else
        r = ldexpf((float)(8u + man), (int)exp - 10);
    return sign ? -r : r;
}

/* round-to-nearest-even, saturate-to-finite (HIP's default __HIP_SATFINITE) */
uint8_t orc_f32_to_e4m3(float f)
{
    uint32_t u    = f32_to_bits(f);
    uint8_t  sign = (uint8_t)((u >> 24) & 0x80u);
    float    a    = fabsf(f);
    if(a != a)
        return (uint8_t)(sign | 0x7Fu);
    if(a >= 448.0f)
        return (uint8_t)(sign | 0x7Eu);
    if(a < 0.015625f) /* below 2^-6: subnormal grid of 2^-9 */
    {
        float    q = a * 512.0f;
        uint32_t n = (uint32_t)q;
        float    r = q - (float)n;
        if(r > 0.5f || (r == 0.5f && (n & 1u)))
            n++;
        return (uint8_t)(sign | n); /* n == 8 lands on the first normal code */
    }
    {
        int      e;
        float    m    = frexpf(a, &e); /* a = m * 2^e, m in [0.5,1) */
        float    q    = m * 16.0f;     /* [8,16) */
        uint32_t n    = (uint32_t)q;
        float    r    = q - (float)n;
        int      bexp = e - 1 + 7;
        if(r > 0.5f || (r == 0.5f && (n & 1u)))
            n++;
        if(n == 16u)
        {
            n = 8u;
            bexp++;
        }
        if(bexp > 15 || (bexp == 15 && n == 15u))
            return (uint8_t)(sign | 0x7Eu);
        return (uint8_t)(sign | ((uint32_t)bexp << 3) | (n - 8u));
    }
}

static inline float load_as_f32(const void* p, size_t idx, int dtype)
{
    switch(dtype)
    {
    case ORC_F16:
        return orc_f16_to_f32(((const uint16_t*)p)[idx]);
    case ORC_BF16:
        return orc_bf16_to_f32(((const uint16_t*)p)[idx]);
    case ORC_E4M3:
        return orc_e4m3_to_f32(((const uint8_t*)p)[idx]);
    case ORC_E5M2: /* OCP e5m2 is binary16 cut after two mantissa bits: the code is the f16's high byte */
        return orc_f16_to_f32((uint16_t)(((const uint8_t*)p)[idx] << 8));
    case ORC_I8:
        return (float)((const int8_t*)p)[idx];
    case ORC_F32:
        return ((const float*)p)[idx];
    case ORC_I32:
        return (float)((const int32_t*)p)[idx];
    default:
        return 0.0f;
    }
}

static inline void store_from_f32(void* p, size_t idx, int dtype, float v)
{
    switch(dtype)
    {
    case ORC_F16:
        ((uint16_t*)p)[idx] = orc_f32_to_f16(v);
        break;
    case ORC_BF16:
        ((uint16_t*)p)[idx] = orc_f32_to_bf16(v);
        break;
    case ORC_F32:
        ((float*)p)[idx] = v;
        break;
    default:
        break;
    }
}

static inline size_t mat_index(uint32_t row, uint32_t col, uint32_t ld, int layout)
{
    /* test/reference_impl.hpp:57-58 */
    return layout == ORC_ROW_MAJOR ? (size_t)row * ld + col : (size_t)col * ld + row;
}

/* ------------------------------------------------------------------ GEMM */

/*
 * D = alpha * A * B + beta * C, following gemm_CPU (test/reference_impl.hpp:36-81):
 * leading dimensions are derived from the layouts (lines 52-55), the
 * accumulator starts at 0 in the compute type and sums k sequentially
 * (lines 70-75), each operand is converted to the compute type before the
 * multiply, and the epilogue alpha*accum + beta*C is rounded once to the
 * output type (lines 76-77).  Rows are spread over OpenMP threads (line 65).
 *
 * Floating inputs (f16, bf16, e4m3, f32) compute in f32, f64 in f64; int8 computes in
 * int32 with int32 alpha/beta passed as integers-in-double.  Returns 0, or
 * -1 for an unsupported type combination.
 */
int orc_gemm(int         in_type,
             int         out_type,
             int         layout_a,
             int         layout_b,
             int         layout_c,
             int         layout_d,
             uint32_t    m,
             uint32_t    n,
             uint32_t    k,
             const void* a,
             const void* b,
             const void* c,
             void*       d,
             double      alpha_c,
             double      beta_c)
{
    /* the scalars arrive wide enough for every compute type (gemm_CPU takes ComputeT alpha, beta:
     * test/reference_impl.hpp:44-45) and are narrowed to it here: int32 for int8 inputs, double for f64,
     * float for everything else */
    const float alpha = (float)alpha_c, beta = (float)beta_c;
    uint32_t lda = layout_a == ORC_ROW_MAJOR ? k : m;
    uint32_t ldb = layout_b == ORC_ROW_MAJOR ? n : k;
    uint32_t ldc = layout_c == ORC_ROW_MAJOR ? n : m;
    uint32_t ldd = layout_d == ORC_ROW_MAJOR ? n : m;

    if(in_type == ORC_I8)
    {
        const int8_t*  pa = (const int8_t*)a;
        const int8_t*  pb = (const int8_t*)b;
        const int32_t* pc = (const int32_t*)c;
        int32_t*       pd = (int32_t*)d;
        int32_t        ia = (int32_t)alpha_c, ib = (int32_t)beta_c;
        if(out_type == ORC_I8)
        {
            /* (int8, int8, int32) of test/gemm/gemm_common_test_params.hpp:52: C and D are int8, the
             * arithmetic is int32 and the result is narrowed by static_cast (test/reference_impl.hpp:74-77),
             * i.e. its low 8 bits */
            const int8_t* qc = (const int8_t*)c;
            int8_t*       qd = (int8_t*)d;
#pragma omp parallel for schedule(static)
            for(int64_t i = 0; i < (int64_t)m; ++i)
            {
                for(uint32_t j = 0; j < n; ++j)
                {
                    int32_t accum = 0;
                    for(uint32_t h = 0; h < k; ++h)
                    {
                        accum += (int32_t)pa[mat_index((uint32_t)i, h, lda, layout_a)]
                                 * (int32_t)pb[mat_index(h, j, ldb, layout_b)];
                    }
                    const uint32_t cterm
                        = ib == 0 ? 0u : (uint32_t)ib * (uint32_t)(int32_t)qc[mat_index((uint32_t)i, j, ldc, layout_c)];
                    qd[mat_index((uint32_t)i, j, ldd, layout_d)] = (int8_t)(uint8_t)((uint32_t)ia * (uint32_t)accum + cterm);
                }
            }
            return 0;
        }
        if(out_type != ORC_I32)
            return -1;
#pragma omp parallel for schedule(static)
        for(int64_t i = 0; i < (int64_t)m; ++i)
        {
            for(uint32_t j = 0; j < n; ++j)
            {
                int32_t accum = 0;
                for(uint32_t h = 0; h < k; ++h)
                {
                    accum += (int32_t)pa[mat_index((uint32_t)i, h, lda, layout_a)]
                             * (int32_t)pb[mat_index(h, j, ldb, layout_b)];
                }
                /* unsigned arithmetic: same bits as the reference's wrapping int32 */
                pd[mat_index((uint32_t)i, j, ldd, layout_d)]
                    = (int32_t)((uint32_t)ia * (uint32_t)accum
                                + (uint32_t)ib
                                      * (uint32_t)pc[mat_index((uint32_t)i, j, ldc, layout_c)]);
            }
        }
        return 0;
    }

    if(in_type == ORC_F64)
    {
        /* f64 in, f64 compute, f64 out (the reference's dgemm instantiation) */
        const double* pa = (const double*)a;
        const double* pb = (const double*)b;
        const double* pc = (const double*)c;
        double*       pd = (double*)d;
        if(out_type != ORC_F64)
            return -1;
#pragma omp parallel for schedule(static)
        for(int64_t i = 0; i < (int64_t)m; ++i)
        {
            for(uint32_t j = 0; j < n; ++j)
            {
                double accum = 0.0;
                for(uint32_t h = 0; h < k; ++h)
                    accum += pa[mat_index((uint32_t)i, h, lda, layout_a)] * pb[mat_index(h, j, ldb, layout_b)];
                pd[mat_index((uint32_t)i, j, ldd, layout_d)]
                    = alpha_c * accum + beta_c * pc[mat_index((uint32_t)i, j, ldc, layout_c)];
            }
        }
        return 0;
    }

    if(in_type != ORC_F16 && in_type != ORC_BF16 && in_type != ORC_E4M3 && in_type != ORC_E5M2 && in_type != ORC_F32)
        return -1;
    if(out_type != ORC_F16 && out_type != ORC_BF16 && out_type != ORC_F32)
        return -1;

#pragma omp parallel for schedule(static)
    for(int64_t i = 0; i < (int64_t)m; ++i)
    {
        for(uint32_t j = 0; j < n; ++j)
        {
            float accum = 0.0f;
            for(uint32_t h = 0; h < k; ++h)
            {
                float av = load_as_f32(a, mat_index((uint32_t)i, h, lda, layout_a), in_type);
                float bv = load_as_f32(b, mat_index(h, j, ldb, layout_b), in_type);
                accum += av * bv;
            }
            float cv = load_as_f32(c, mat_index((uint32_t)i, j, ldc, layout_c), out_type);
            store_from_f32(
                d, mat_index((uint32_t)i, j, ldd, layout_d), out_type, alpha * accum + beta * cv);
        }
    }
    return 0;
}

/*
 * The same arithmetic for a chosen set of complete rows of D only: row r of
 * the result goes to d_rows[r * n ...] (row-major, tightly packed).  Every
 * element of gemm_CPU depends only on its own row of A and column of B
 * (test/reference_impl.hpp:66-79), so these values equal the full oracle's.
 * beta must be 0 (C is not read).
 */
int orc_gemm_rows(int             in_type,
                  int             out_type,
                  int             layout_a,
                  int             layout_b,
                  uint32_t        m,
                  uint32_t        n,
                  uint32_t        k,
                  const void*     a,
                  const void*     b,
                  const uint32_t* rows,
                  uint32_t        nrows,
                  void*           d_rows,
                  double          alpha_c)
{
    const float alpha = (float)alpha_c;
    uint32_t lda = layout_a == ORC_ROW_MAJOR ? k : m;
    uint32_t ldb = layout_b == ORC_ROW_MAJOR ? n : k;
    int      rc  = 0;
#pragma omp parallel for schedule(dynamic, 64) collapse(2)
    for(uint32_t r = 0; r < nrows; ++r)
    {
        for(uint32_t j = 0; j < n; ++j)
        {
            uint32_t i = rows[r];
            if(i >= m)
            {
                rc = -1;
                continue;
            }
            if(in_type == ORC_I8)
            {
                int32_t accum = 0;
                for(uint32_t h = 0; h < k; ++h)
                    accum += (int32_t)((const int8_t*)a)[mat_index(i, h, lda, layout_a)]
                             * (int32_t)((const int8_t*)b)[mat_index(h, j, ldb, layout_b)];
                ((int32_t*)d_rows)[(size_t)r * n + j]
                    = (int32_t)((uint32_t)(int32_t)alpha_c * (uint32_t)accum);
            }
            else
            {
                float accum = 0.0f;
                for(uint32_t h = 0; h < k; ++h)
                    accum += load_as_f32(a, mat_index(i, h, lda, layout_a), in_type)
                             * load_as_f32(b, mat_index(h, j, ldb, layout_b), in_type);
                store_from_f32(d_rows, (size_t)r * n + j, out_type, alpha * accum + 0.0f);
            }
        }
    }
    return rc;
}

/* ------------------------------------------------------------------ DLRM */

/*
 * dlrm_fwd_CPU (test/reference_impl.hpp:83-119): per sample, the first k
 * outputs copy row 0 (the bottom-MLP vector); then for i in 0..m-1, j < i,
 * in row-major order, the f32-accumulated dot product of rows i and j cast
 * to the data type.  Output stride m(m-1)/2 + k.  dtype is ORC_F16 or ORC_F32.
 */
int orc_dlrm_fwd(
    int dtype, const void* input, void* output, uint32_t m, uint32_t k, uint32_t batch)
{
    size_t in_stride  = (size_t)m * k;
    size_t out_stride = ((size_t)m * (m - 1)) / 2 + k;
    if(dtype != ORC_F16 && dtype != ORC_F32 && dtype != ORC_BF16)
        return -1;
#pragma omp parallel for schedule(static)
    for(int64_t b = 0; b < (int64_t)batch; ++b)
    {
        size_t o    = (size_t)b * out_stride;
        size_t base = (size_t)b * in_stride;
        for(uint32_t i = 0; i < k; ++i)
        {
            if(dtype == ORC_F32)
                ((float*)output)[o] = ((const float*)input)[base + i];
            else
                ((uint16_t*)output)[o] = ((const uint16_t*)input)[base + i];
            o++;
        }
        for(uint32_t i = 0; i < m; ++i)
        {
            for(uint32_t j = 0; j < i; ++j)
            {
                float accum = 0.0f;
                for(uint32_t h = 0; h < k; ++h)
                    accum += load_as_f32(input, base + (size_t)i * k + h, dtype)
                             * load_as_f32(input, base + (size_t)j * k + h, dtype);
                store_from_f32(output, o, dtype, accum);
                o++;
            }
        }
    }
    return 0;
}

/*
 * dlrm_bwd_CPU (test/reference_impl.hpp:121-179): the upstream gradient's
 * first k values are the bottom-MLP gradient; the remaining m(m-1)/2 values
 * fill the strict lower triangle of an m x m matrix T (zero elsewhere);
 * S = T + T^T; grad[i][:] = sum_j S[i][j] * X[j][:], f32 accumulation.
 */
int orc_dlrm_bwd(int         dtype,
                 const void* input,
                 const void* upstream,
                 void*       mlp_grad,
                 void*       output,
                 uint32_t    m,
                 uint32_t    k,
                 uint32_t    batch)
{
    size_t in_stride = (size_t)m * k;
    size_t up_stride = ((size_t)m * (m - 1)) / 2 + k;
    if(dtype != ORC_F16 && dtype != ORC_F32 && dtype != ORC_BF16)
        return -1;
#pragma omp parallel for schedule(static)
    for(int64_t b = 0; b < (int64_t)batch; ++b)
    {
        float* tril = (float*)calloc((size_t)m * m, sizeof(float));
        size_t up   = (size_t)b * up_stride;
        for(uint32_t i = 0; i < k; ++i)
        {
            if(dtype == ORC_F32)
                ((float*)mlp_grad)[(size_t)b * k + i] = ((const float*)upstream)[up + i];
            else
                ((uint16_t*)mlp_grad)[(size_t)b * k + i] = ((const uint16_t*)upstream)[up + i];
        }
        up += k;
        for(uint32_t i = 0; i < m; ++i)
            for(uint32_t j = 0; j < i; ++j)
                tril[(size_t)i * m + j] = load_as_f32(upstream, up++, dtype);
        /* symmetrise: S = T + T^T, values kept in the data type as the reference does */
        for(uint32_t i = 0; i < m; ++i)
            for(uint32_t j = i + 1; j < m; ++j)
                tril[(size_t)i * m + j] = tril[(size_t)j * m + i];
        for(uint32_t i = 0; i < m; ++i)
        {
            for(uint32_t h = 0; h < k; ++h)
            {
                float accum = 0.0f;
                for(uint32_t j = 0; j < m; ++j)
                    accum += tril[(size_t)i * m + j]
                             * load_as_f32(input, (size_t)b * in_stride + (size_t)j * k + h, dtype);
                store_from_f32(output, (size_t)b * in_stride + (size_t)i * k + h, dtype, accum);
            }
        }
        free(tril);
    }
    return 0;
}

/* ------------------------------------------------------------ comparator */

/*
 * compareEqual (test/common.hpp:350-444): metric |a-b| / (|a|+|b|+1) in
 * double, maximum over all elements; any inf or NaN fails.  Pass iff
 * max <= eps(type) * tolerance.  Both arrays are contiguous with `count`
 * elements of `dtype`.  *max_rel receives the maximum (inf / NaN on those
 * failures).  Returns 1 on pass, 0 on fail, -1 on a bad dtype.
 */
int orc_compare(
    int dtype, const void* x, const void* y, size_t count, double tolerance, double* max_rel)
{
    double eps;
    double mx     = 0.0;
    int    is_inf = 0, is_nan = 0;
    switch(dtype)
    {
    case ORC_F16:
        eps = 0.0009765625;
        break; /* 2^-10 */
    case ORC_BF16:
        eps = 0.0078125;
        break; /* 2^-7 */
    case ORC_F32:
        eps = 1.1920928955078125e-07;
        break;
    case ORC_I32:
    case ORC_I8:
        eps = 0.0;
        break; /* numeric_limits<int>::epsilon() == 0 */
    case ORC_E4M3:
        eps = 0.125;
        break; /* float8.hpp:549-580: epsilon code 0x20 = 2^-3 */
    case ORC_F64:
        eps = 2.220446049250313e-16;
        break;
    default:
        return -1;
    }
#pragma omp parallel for reduction(max : mx) reduction(| : is_inf, is_nan)
    for(int64_t i = 0; i < (int64_t)count; ++i)
    {
        double a   = dtype == ORC_F64 ? ((const double*)x)[i] : (double)load_as_f32(x, (size_t)i, dtype);
        double b   = dtype == ORC_F64 ? ((const double*)y)[i] : (double)load_as_f32(y, (size_t)i, dtype);
        double num = fabs(a - b);
        double den = fabs(a) + fabs(b) + 1.0;
        if(isinf(num) || isinf(den))
            is_inf |= 1;
        else
        {
            double r = num / den;
            if(isnan(r))
                is_nan |= 1;
            else if(r > mx)
                mx = r;
        }
    }
    if(is_inf)
    {
        *max_rel = INFINITY;
        return 0;
    }
    if(is_nan)
    {
        *max_rel = NAN;
        return 0;
    }
    *max_rel = mx;
    return mx <= eps * tolerance ? 1 : 0;
}

/*
 * The reference's deterministic GEMM test input (test/device/common.hpp:203-220):
 * value = (row*n + col) % 3, negated when non-zero, written at the layout's index
 * with ld = n (row-major) or m (col-major).  Values are exact in every type.
 */
int orc_fill_ref(int dtype, void* mat, uint32_t m, uint32_t n, int layout)
{
    uint32_t ld = layout == ORC_ROW_MAJOR ? n : m;
    for(uint32_t r = 0; r < m; ++r)
    {
        for(uint32_t c = 0; c < n; ++c)
        {
            int    v   = (int)(((uint64_t)r * n + c) % 3u);
            float  fv  = (float)(-v);
            size_t idx = mat_index(r, c, ld, layout);
            switch(dtype)
            {
            case ORC_F16:
                ((uint16_t*)mat)[idx] = orc_f32_to_f16(fv);
                break;
            case ORC_BF16:
                ((uint16_t*)mat)[idx] = orc_f32_to_bf16(fv);
                break;
            case ORC_E4M3:
                ((uint8_t*)mat)[idx] = orc_f32_to_e4m3(fv);
                break;
            case ORC_I8:
                ((int8_t*)mat)[idx] = (int8_t)(-v);
                break;
            case ORC_F32:
                ((float*)mat)[idx] = fv;
                break;
            case ORC_I32:
                ((int32_t*)mat)[idx] = -v;
                break;
            case ORC_F64:
                ((double*)mat)[idx] = (double)fv;
                break;
            default:
                return -1;
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------ 2:4 format */

/*
 * Build-defined 2:4 structured-sparse storage for a row-major m x k matrix of
 * 1-byte elements (int8 or e4m3): every aligned group of 4 along k keeps 2
 * values, in increasing position order, plus a nibble (idx0 | idx1 << 2) with
 * idx0 < idx1.  A group with fewer than 2 non-zeros keeps the non-zeros plus
 * the lowest unused positions.
 *
 * The storage is K-blocked.  A stage is 128 dense k; within a stage a row's 32
 * groups belong to 4 lane groups of 8.  Kept values:
 *   values[stage][row / 16][lane group][row % 16][16]   (16 = 8 groups x 2 kept bytes)
 * and, with the same first four indices, 4 metadata bytes (two nibbles per byte,
 * the even group in the low nibble):
 *   meta[stage][row / 16][lane group][row % 16][4]
 * m must be a multiple of 16 and k of 128.  Returns -1 for other sizes or if a
 * group has more than 2 non-zeros.
 */
static size_t orc24_value_at(uint32_t r, uint32_t g, uint32_t m)
{
    /* g: group of four along k */
    return ((((size_t)(g / 32u) * (m / 16u) + r / 16u) * 4u + (g % 32u) / 8u) * 16u + r % 16u) * 16u + 2u * (g % 8u);
}

static size_t orc24_meta_at(uint32_t r, uint32_t g, uint32_t m)
{
    return ((((size_t)(g / 32u) * (m / 16u) + r / 16u) * 4u + (g % 32u) / 8u) * 16u + r % 16u) * 4u + (g % 8u) / 2u;
}

int orc_compress24(const uint8_t* dense, uint32_t m, uint32_t k, uint8_t* values, uint8_t* meta)
{
    if(k % 128u || m % 16u)
        return -1;
    for(uint32_t r = 0; r < m; ++r)
    {
        for(uint32_t g = 0; g < k / 4u; ++g)
        {
            const uint8_t* p  = dense + (size_t)r * k + 4u * g;
            int            nz = 0, pos[4];
            for(int e = 0; e < 4; ++e)
                if(p[e] != 0)
                    pos[nz++] = e;
            if(nz > 2)
                return -1;
            for(int e = 0; e < 4 && nz < 2; ++e)
            {
                int used = 0;
                for(int q = 0; q < nz; ++q)
                    used |= (pos[q] == e);
                if(!used)
                    pos[nz++] = e;
            }
            if(pos[0] > pos[1])
            {
                int t  = pos[0];
                pos[0] = pos[1];
                pos[1] = t;
            }
            values[orc24_value_at(r, g, m)]      = p[pos[0]];
            values[orc24_value_at(r, g, m) + 1u] = p[pos[1]];
            uint8_t  nib                          = (uint8_t)(pos[0] | (pos[1] << 2));
            uint8_t* mb                           = meta + orc24_meta_at(r, g, m);
            if(g & 1u)
                *mb = (uint8_t)((*mb & 0x0Fu) | (nib << 4));
            else
                *mb = (uint8_t)((*mb & 0xF0u) | nib);
        }
    }
    return 0;
}

int orc_decompress24(
    const uint8_t* values, const uint8_t* meta, uint32_t m, uint32_t k, uint8_t* dense)
{
    if(k % 128u || m % 16u)
        return -1;
    memset(dense, 0, (size_t)m * k);
    for(uint32_t r = 0; r < m; ++r)
    {
        for(uint32_t g = 0; g < k / 4u; ++g)
        {
            uint8_t mb  = meta[orc24_meta_at(r, g, m)];
            uint8_t nib = (g & 1u) ? (uint8_t)(mb >> 4) : (uint8_t)(mb & 0xFu);
            dense[(size_t)r * k + 4u * g + (nib & 3u)]        = values[orc24_value_at(r, g, m)];
            dense[(size_t)r * k + 4u * g + ((nib >> 2) & 3u)] = values[orc24_value_at(r, g, m) + 1u];
        }
    }
    return 0;
}

int orc_num_threads(void)
{
    int n = 1;
#ifdef _OPENMP
#pragma omp parallel
    {
#pragma omp single
        n = omp_get_num_threads();
    }
#endif
    return n;
}
