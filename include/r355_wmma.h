/*
 * C ABI of the MI355X (gfx950) matrix-fragment hot path: GEMM, DLRM dot interaction and
 * GEMV kernels built on MFMA.  Plain pointers and sizes only; every device pointer is
 * caller-owned HIP device memory; `stream` is a hipStream_t passed as void* (NULL = the
 * null stream).  Calls are asynchronous on `stream`, re-entrant, and allocate nothing.
 * Every entry point returns R355_OK or a negative r355_status; r355_last_error() gives
 * the message of the calling thread's most recent failure.
 *
 * The reference is a header-only device library whose host boundary is the kernel
 * launch itself; each entry point below names the reference launch it stands in for.
 */
#ifndef R355_WMMA_H
#define R355_WMMA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum
{
    R355_OK                 = 0,
    R355_ERR_BAD_ARG        = -1, /* null pointer, zero size, unknown enum value          */
    R355_ERR_UNSUPPORTED    = -2, /* type / layout combination has no kernel              */
    R355_ERR_BAD_SIZE       = -3, /* dimension not a multiple of the block the kernel needs
                                     (the reference kernels leave D untouched in that case:
                                     samples/perf_hgemm.cpp:549-553,757-762)               */
    R355_ERR_MISALIGNED     = -4, /* pointer or leading dimension breaks vector alignment */
    R355_ERR_LAUNCH         = -5, /* hipGetLastError() after the launch                   */
    R355_ERR_NOT_24_SPARSE  = -6  /* r355_compress_24: a group of 4 holds > 2 non-zeros   */
} r355_status;

/* element types (storage) */
typedef enum
{
    R355_F16  = 0, /* IEEE binary16                      */
    R355_BF16 = 1, /* bfloat16                           */
    R355_E4M3 = 2, /* OCP FP8 E4M3 (gfx950 native)       */
    R355_I8   = 3, /* signed 8-bit integer               */
    R355_F32  = 4,
    R355_I32  = 5,
    R355_F64  = 6,
    R355_E5M2 = 7 /* OCP FP8 E5M2 ("bf8", the reference's bfloat8_t): GEMM operands, f32 result */
} r355_dtype;

/* memory orientation; BLAS letters: row-major = "T", col-major = "N" for A (m x k) */
typedef enum
{
    R355_ROW_MAJOR = 0,
    R355_COL_MAJOR = 1
} r355_layout;

typedef enum
{
    R355_KERNEL_AUTO   = 0, /* macro-tile kernel when shapes allow, else block-per-wave      */
    R355_KERNEL_SIMPLE = 1, /* one MFMA block per wave through the fragment API, no LDS
                               (samples/simple_hgemm.cpp:81-139,
                                test/gemm/gemm_PGR0_LB0_MP0_SB_NC/device/kernel_device_func.hpp:50-175) */
    R355_KERNEL_TILED  = 2, /* LDS-staged 256 x 256 macro tile (m, n multiples of 16; k of 8 for 16-bit, 16 for 8-bit operands)
                               (samples/perf_hgemm.cpp:515-711,
                                test/gemm/gemm_PGR1_LB2_MP0_MB_CP/device/kernel_device_func.hpp:52-283) */
    R355_KERNEL_TILED_128 = 3, /* the same kernels with a 128 x 128 macro tile (the only one for f64): what AUTO
                               picks when the 256 x 256 tiles of a problem would leave most CUs idle */
    R355_KERNEL_TILED_128_SPLITK = 4, /* 128 x 128 tiles with K split over several workgroups per tile and a reduction
                               (needs `workspace`; what AUTO picks for few tiles and a long K when a workspace is given).
                               No counterpart in the reference. */
    R355_KERNEL_TILED_DEEP = 5 /* the 256 x 256 macro tile with its K loop on five LDS buffers filled two to three stages ahead.
                               8-bit and f32 operands always run that way (the selector then equals R355_KERNEL_TILED); for
                               f16 / bf16 it is what AUTO and R355_KERNEL_TILED take once A and B together exceed the 256 MiB
                               memory-side cache, where the default two-buffer loop no longer hides the HBM latency, and for
                               k <= 1536. */
} r355_gemm_kernel;

/*
 * D = alpha * A * B + beta * C.  A is m x k, B is k x n, C and D are m x n.
 * Argument order and meaning follow the reference kernel signature
 * (test/gemm/gemm_kernel_base.hpp:101-114): leading dimensions in elements.
 * Supported (in -> out, accumulate): f16 -> f32|f16 (f32), bf16 -> f32|bf16 (f32),
 * e4m3 -> f32 (f32), e5m2 -> f32 (f32), i8 -> i32|i8 (i32, alpha/beta truncated to int32; an i8 result is the low 8 bits, as the
 * reference's static_cast narrows it), f32 -> f32 (f32), f64 -> f64 (f64).
 * beta == 0 means C is never read and may be NULL.  C may be D itself (same pointer, leading dimension and orientation:
 * D = alpha * A * B + beta * D in place); any other overlap of D with A, B or C is undefined.
 *
 * sparse24 != 0: A is 2:4 structured-sparse along k (i8 -> i32, e4m3 | f16 | bf16 -> f32; from m, n >= 128 on a macro-tile
 * kernel of 256 x 256 or 128 x 128 - R355_KERNEL_TILED / R355_KERNEL_TILED_128 force one, AUTO takes the faster by a timing
 * model - and a block-per-wave kernel below that; B in either orientation; no split along K):
 * `a` holds the m * k/2 kept values and `a_meta` the m * k/8 index bytes in the K-blocked storage that
 * r355_compress_24 / r355_compress_24_16 write (layout_a = R355_ROW_MAJOR, lda = k / 2: the storage has no padding);
 * m, n multiples of 16, k of 128 bytes' worth of elements (128 for 1-byte, 64 for 2-byte elements).
 * The reference has no sparse path; this form has no counterpart there.
 */
typedef struct
{
    int32_t     in_type;  /* r355_dtype of A and B */
    int32_t     out_type; /* r355_dtype of C and D */
    int32_t     layout_a, layout_b, layout_c, layout_d; /* r355_layout */
    uint32_t    m, n, k;
    const void* a;
    const void* b;
    const void* c;
    void*       d;
    uint32_t    lda, ldb, ldc, ldd;
    /* The reference passes the scalars in the compute type (ComputeT alpha, beta: test/gemm/gemm_kernel_base.hpp:112-113).
     * A double carries each of them unrounded: it is narrowed to float for f16 / bf16 / fp8 / f32 inputs, truncated to
     * int32 for i8 inputs (every int32 is exact in a double) and used as it is for f64. */
    double      alpha, beta;
    int32_t     sparse24;
    const void* a_meta;
    int32_t     kernel; /* r355_gemm_kernel */
    /* Optional device scratch for split-K (dense GEMM only): problems whose 128 x 128 tiles would occupy at most half of
     * the CUs while k spans at least 16 stages of 128 bytes run `split_k` workgroups per tile, each over its own range of
     * K, into workspace[split][m][n] (accumulator type: 4 bytes, f64: 8), followed by a reduction kernel that adds the
     * partial results in split order and applies alpha, beta and C.  r355_gemm_query reports split_k and the bytes it
     * needs for the workspace_bytes offered (to learn the size, offer UINT64_MAX; the query accepts workspace = NULL with
     * it).  A launch with workspace = NULL, one that is not 16-byte aligned or one that is too small does not split.
     * The library never allocates; calls that share a workspace must not overlap. */
    void*       workspace;
    uint64_t    workspace_bytes;
} r355_gemm_args;

/* Replaces: hipExtLaunchKernelGGL(gemm_rocwmma_d, ...) in samples/perf_hgemm.cpp:820-842 and
 * test/gemm/gemm_kernel_base_impl.hpp:622-645. */
int r355_gemm(const r355_gemm_args* args, void* stream);

/* Launch description the AUTO/TILED/SIMPLE choice resolves to, without launching
 * (the values the reference computes on the host: samples/perf_hgemm.cpp:807-817).
 * R355_KERNEL_AUTO may split a problem of several rounds of 256 x 256 tiles into two launches on the
 * same stream - whole rounds on that tile, the rest (at most half a round) on 128 x 128 tiles; the
 * plan then describes the first launch. */
typedef struct
{
    int32_t  kernel;                       /* r355_gemm_kernel actually selected */
    uint32_t macro_tile_m, macro_tile_n, macro_tile_k;
    uint32_t grid_x, grid_y, block_x, block_y;
    uint32_t lds_bytes;
    uint32_t split_k;         /* workgroups per tile along K (1: no split) */
    uint64_t workspace_bytes; /* bytes of `workspace` the plan uses (0 without split-K) */
} r355_gemm_plan;
int r355_gemm_query(const r355_gemm_args* args, r355_gemm_plan* plan);

/* r355_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc) and have no workspace to pass.  No counterpart in the reference.
 * Identical to r355_gemm, except that args->workspace / workspace_bytes are ignored and split-K keeps its partial
 * results in a 16 MiB buffer that is part of the library's device image (one per GPU, held until the process ends);
 * the call allocates and frees nothing.  A problem whose split-K plan needs more than 16 MiB (r355_gemm_query with
 * workspace_bytes = UINT64_MAX reports the need) is refused with R355_ERR_BAD_SIZE; with 4-byte accumulators no plan
 * on 256 CUs needs more.  Nothing in the buffer has to start at zero (every partial result is written before it is
 * read), but all calls on one GPU share it: calls that overlap in time on one GPU (two streams, two threads) race.
 * The first call on a device looks up the buffer's address (hipGetSymbolAddress, which may load the library's device
 * image): it must be made outside stream capture - r355_get_device_info() on that device performs the same look-up and
 * serves as the set-up call.  A first call that arrives while its stream is capturing is refused with
 * R355_ERR_UNSUPPORTED and records nothing. */
int r355_gemm_noalloc(const r355_gemm_args* args, void* stream);

/* Timing helper in the reference's protocol (test/gemm/gemm_kernel_base_impl.hpp:647-676):
 * `warmup` untimed launches, then `iters` launches between two hipEvents on `stream`;
 * *avg_ms = elapsed / iters.  Synchronises the stream. */
int r355_gemm_timed(const r355_gemm_args* args, void* stream, int warmup, int iters, float* avg_ms);

/*
 * DLRM dot-interaction forward.  in: [batch][m][k], out: [batch][k + m(m-1)/2]:
 * out[b][0:k] = in[b][0][:], then the strict lower triangle of X X^T in row-major (i, j<i)
 * order, f32 accumulation, rounded to dtype (R355_F16, R355_BF16 or R355_F32).  Bandwidth-bound kernels for
 * 2 <= m <= 32 with k in {32, 64, 128, 256} (R355_F32: up to 128); any other m and k that are multiples of 16 - the
 * reference's own constraint, test/dlrm/dlrm_kernel_base_impl.hpp:146-151; its tests run m = 128, k = 128 and m = k = 1024 -
 * run kernels written on the fragment API (a 16 x 16 block per wave for small launches, several blocks per wave otherwise;
 * any batch).  No scratch buffer either way (the reference's `acc` argument is gone).
 * Replaces: dlrmDotFwd launch, test/dlrm/dlrm_kernel_base_impl.hpp:78-96,
 * test/dlrm/device/dlrm_dot_fwd.hpp:35-138, samples/simple_dlrm.cpp:184-284.
 */
int r355_dlrm_fwd(int32_t dtype, const void* in, void* out, uint32_t m, uint32_t k, uint32_t batch, void* stream);
int r355_dlrm_fwd_timed(int32_t dtype, const void* in, void* out, uint32_t m, uint32_t k, uint32_t batch,
                        void* stream, int warmup, int iters, float* avg_ms);

/*
 * DLRM dot-interaction backward.  upstream: [batch][k + m(m-1)/2]; mlp_grad: [batch][k];
 * in_grad: [batch][m][k].  dtype R355_F16, R355_BF16 (all four pointers 16-byte aligned) or R355_F32
 * (in / in_grad 16-byte, upstream / mlp_grad 4-byte aligned).  Shapes as for the forward call; the general kernels form S = T + T^T
 * block by block from the packed triangle instead of reconstructing it in memory.  Replaces: dlrmDotBwd +
 * trilReconstruct launches, test/dlrm/device/dlrm_dot_bwd.hpp:35-176.
 */
int r355_dlrm_bwd(int32_t dtype, const void* in, const void* upstream, void* mlp_grad, void* in_grad,
                  uint32_t m, uint32_t k, uint32_t batch, void* stream);

/*
 * y_out = alpha * A * x + beta * y_in.  A is m x k f32 (layout_a), x has k elements, y m.
 * Replaces: sgemv_rocwmma_d launch, samples/simple_sgemv.cpp:103-150,240-262.
 */
int r355_gemv(int32_t layout_a, uint32_t m, uint32_t k, const float* a, uint32_t lda, const float* x,
              const float* y_in, float* y_out, float alpha, float beta, void* stream);
int r355_gemv_timed(int32_t layout_a, uint32_t m, uint32_t k, const float* a, uint32_t lda, const float* x,
                    const float* y_in, float* y_out, float alpha, float beta, void* stream, int warmup,
                    int iters, float* avg_ms);
/* The f64 twin (samples/simple_dgemv.cpp:103): m, k multiples of 2, lda % 2 == 0, 16-byte aligned pointers. */
int r355_dgemv(int32_t layout_a, uint32_t m, uint32_t k, const double* a, uint32_t lda, const double* x,
               const double* y_in, double* y_out, double alpha, double beta, void* stream);

/*
 * The same products with K split over several workgroups per block of rows, for shapes that leave most CUs idle
 * with one workgroup per block: a col-major A with few rows (256 x 262144) or a row count just above a multiple of
 * what fills the CUs (8256 rows), a row-major A with few very long rows.  The splits' partial sums go to `workspace`
 * (the caller's device memory, 16-byte aligned; its contents before the call do not matter) and a second kernel adds
 * them in split order, so the result depends on the shape alone, never on scheduling.
 * r355_gemv_workspace_bytes: what the split form wants for a shape (elem_bytes 4: f32, 8: f64; an unpadded A is
 * assumed: lda = m col-major, k row-major); 0 where the plain kernels do as well.  With a null or smaller workspace r355_gemv_ws / r355_dgemv_ws run the plain kernels
 * (the same as r355_gemv / r355_dgemv).  No counterpart in the reference (its sample has one kernel for all shapes).
 */
size_t r355_gemv_workspace_bytes(int32_t layout_a, uint32_t m, uint32_t k, uint32_t elem_bytes);
int    r355_gemv_ws(int32_t layout_a, uint32_t m, uint32_t k, const float* a, uint32_t lda, const float* x,
                    const float* y_in, float* y_out, float alpha, float beta, void* workspace, size_t workspace_bytes,
                    void* stream);
int    r355_dgemv_ws(int32_t layout_a, uint32_t m, uint32_t k, const double* a, uint32_t lda, const double* x,
                     const double* y_in, double* y_out, double alpha, double beta, void* workspace,
                     size_t workspace_bytes, void* stream);

/*
 * Host-side 2:4 compressor for a row-major m x k matrix of 1-byte elements (host pointers); m % 16 == 0, k % 128 == 0.
 * Every aligned group of 4 along k keeps 2 elements (in position order) and a nibble idx0 | idx1 << 2 (idx0 < idx1).
 * The storage is K-blocked so that a kernel's share of one K stage is contiguous and in matrix-instruction order.
 * With a stage = 128 dense k and a lane group = 32 of them (8 groups of 4):
 *   values [k / 128][m / 16][4 lane groups][16 rows][16 kept bytes]     m * k / 2 bytes
 *   meta   [k / 128][m / 16][4 lane groups][16 rows][4 index bytes]     m * k / 8 bytes, two nibbles per byte, the even
 *                                                                       group in the low nibble
 * (a 32-bit word of `meta` is the index register of v_smfmac_*_16x16x128 for the 16 bytes of `values` beside it).
 * r355_decompress_24 is the inverse.  R355_ERR_BAD_SIZE for sizes off that grid, R355_ERR_NOT_24_SPARSE if a group holds
 * more than 2 non-zeros.  No counterpart in the reference.
 */
int r355_compress_24(const uint8_t* dense, uint32_t m, uint32_t k, uint8_t* values, uint8_t* meta);
int r355_decompress_24(const uint8_t* values, const uint8_t* meta, uint32_t m, uint32_t k, uint8_t* dense);
/* The same for 2-byte elements (f16 / bf16 bit patterns; an element is zero when all its bits are): a stage is 64 dense
 * k (128 bytes), a lane group 16 of them: values [k / 64][m / 16][4][16][8 kept elements], meta [k / 64][m / 16][4][16][2 bytes];
 * k % 64 == 0. */
int r355_compress_24_16(const uint16_t* dense, uint32_t m, uint32_t k, uint16_t* values, uint8_t* meta);
int r355_decompress_24_16(const uint16_t* values, const uint8_t* meta, uint32_t m, uint32_t k, uint16_t* dense);

/* Device facts used by the roofline report (test/hip_device.hpp:101-119 in the reference). */
typedef struct
{
    char     arch[64];
    int32_t  compute_units;
    int32_t  wave_size;
    int32_t  clock_mhz;         /* peak engine clock reported by HIP */
    int32_t  memory_clock_mhz;
    int32_t  lds_bytes_per_block;
    uint64_t hbm_bytes;
} r355_device_info;
int r355_get_device_info(r355_device_info* info);

/* Message for the calling thread's last non-OK status ("" if none). */
const char* r355_last_error(void);

/* Library version string. */
const char* r355_version(void);

#ifdef __cplusplus
}
#endif

#endif /* R355_WMMA_H */
