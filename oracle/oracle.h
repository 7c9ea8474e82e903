/*
 * CPU oracle for the IMEX tile-pipeline hot path -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of what the reference computes for relu / silu /
 * softmax / reduce / transpose / GEMM (+bias, +SiLU epilogue), of its host-side
 * checking helpers (allclose, max error, profiler statistics) and of the seeded
 * input generators the parity tests and the benchmark use.  Nothing that ships
 * (the HIP runtime library, the kernels, the runner utilities) links or calls
 * this file; only tests, the smoke check and the CPU-baseline leg of the
 * benchmark do, and only as the checker.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the intel/mlir-extensions checkout).
 *
 * Pinning status (what independent evidence each function is tested against):
 *   relu, softmax, row-sum, transpose, gemm (f32 / f16 / bf16 inputs), bias add,
 *   half->float, bfloat->float, allclose, stats   : reference golden vectors
 *       and closed forms (tests/golden, tests/test_oracle.py);
 *   silu / outer reduction on f16, bf16           : defined as widen -> f32 function -> one
 *       rounding; pinned as that composition of the f32 oracle with the checked conversions;
 *   row mean                                      : closed forms (the reference's test draws
 *       random inputs and holds no vector): exact dyadic rows, sequential-order witnesses,
 *       a true division;
 *   stats (reference median formula)              : also the reference's own
 *       ExecutionEngineUtils.cpp compiled into oracle/_ref;
 *   float->half / float->bfloat rounding          : exhaustive comparison with
 *       the compiler's _Float16 / numpy; NaN payload behaviour parity unpinned;
 *   silu                                          : parity unpinned by reference
 *       tests (the reference holds no SiLU vector); pinned by closed forms only;
 *   expf, logf                                    : host libm, as the reference's
 *       CPU lowering calls it; parity unpinned beyond 1 ulp;
 *   flash attention                                : the reference's own check input
 *       (every element 0.625 -> every output 0.625, flash_attention_fwd.mlir:481-485)
 *       and closed forms (one-hot scores, uniform scores = mean of V);
 *   maximumf                                      : closed forms (order, signed zeros, NaN if either
 *       operand is; which NaN comes back is parity unpinned -- the reference's test draws no NaN);
 *   loop fusion / input fusion chains             : parity unpinned by reference
 *       tests (the benchmarks feed constants and check nothing); pinned by closed
 *       forms against an f64 evaluation.
 */
#ifndef IMEX_ORACLE_H
#define IMEX_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- 16-bit float conversions -------------------------------------------- */
float oracle_half_to_float(uint16_t h);      /* ImexRunnerUtils.cpp:137-159 */
float oracle_bfloat_to_float(uint16_t b);    /* ImexRunnerUtils.cpp:165-169 */
uint16_t oracle_float_to_half(float f);      /* RNE; upstream Float16bits (call sites ImexRunnerUtils.cpp:34,48,324) */
uint16_t oracle_float_to_bfloat(float f);    /* RNE; upstream Float16bits (call sites ImexRunnerUtils.cpp:34,48,327) */
void oracle_half_to_float_n(const uint16_t *in, float *out, size_t n);
void oracle_bfloat_to_float_n(const uint16_t *in, float *out, size_t n);
void oracle_float_to_half_n(const float *in, uint16_t *out, size_t n);
void oracle_float_to_bfloat_n(const float *in, uint16_t *out, size_t n);

/* ---- seeded generators (std::mt19937 raw stream) ------------------------- */
typedef struct { uint32_t mt[624]; int idx; } oracle_mt19937;
void oracle_mt_seed(oracle_mt19937 *g, uint32_t seed);
uint32_t oracle_mt_next(oracle_mt19937 *g);
/* dtype codes used by the generators and element-wise helpers */
enum { ORACLE_F32 = 0, ORACLE_F16 = 1, ORACLE_BF16 = 2 };
void oracle_fill_uniform(void *out, size_t n, int dtype, uint32_t seed, double lo, double hi);
void oracle_fill_normal(void *out, size_t n, int dtype, uint32_t seed, double mu, double sigma);
void oracle_fill_bits_no_nan(void *out, size_t n, int dtype, uint32_t seed);
void oracle_fill_int_uniform(void *out, size_t n, int dtype, uint32_t seed, int lo, int hi);

/* ---- element-wise --------------------------------------------------------- */
void oracle_relu_f32(const float *x, float *y, size_t n);              /* benchmarks/relu/relu_gpu.mlir.in:8-10 */
void oracle_relu_16(const uint16_t *x, uint16_t *y, size_t n, int dtype);
void oracle_relu_olt_f32(const float *x, float *y, size_t n);          /* test/PlaidML/OpTest.Relu.mlir:29-35 */
void oracle_silu_f32(const float *x, float *y, size_t n);              /* benchmarks/silu/silu_gpu.mlir.in:8-18 */
void oracle_silu_16(const uint16_t *x, uint16_t *y, size_t n, int dtype);   /* widen, silu_f32, round once */
float oracle_silu_scalar_f32(float x);
void oracle_loop_fusion_f32(const float *a, const float *b, float *out, size_t n);                    /* benchmarks/kLoopFusion/kLoopFusion.mlir.in:6-29 */
void oracle_input_fusion_f32(const float *a, const float *b, float *out, int64_t rows, int64_t cols); /* benchmarks/kInputFusion/kInputFusion.mlir.in:8-39 */
void oracle_flash_attention_rows(const uint16_t *Q, const uint16_t *K, const uint16_t *V, uint16_t *out_rows,
                                 int64_t n_ctx, int64_t d_head, float sm_scale, const int64_t *rows,
                                 int64_t nrows); /* WG/flash_attention_fwd.mlir:332-421 */
void oracle_logf_n(const float *in, float *out, size_t n);              /* the host libm logf the fused chains call */
void oracle_maximum_f32(const float *a, const float *b, float *out, size_t n);   /* WG/arith_maximumf.mlir:122-129 (arith.maximumf) */
float oracle_expf_cr(float x);                                          /* correctly rounded exp via f64 */
void oracle_expf_n(const float *in, float *out, size_t n);              /* the host libm expf the oracle's silu/softmax call */

/* ---- softmax --------------------------------------------------------------- */
void oracle_softmax_f32(const float *x, float *y, int64_t rows, int64_t cols);        /* benchmarks/softmax/softmax_gpu.mlir.in:4-44 */
void oracle_softmax_3pass_f32(const float *x, float *y, int64_t rows, int64_t cols);  /* WG/softmax_intra_sg_cross_lane.mlir:85-117 */
void oracle_softmax_16(const uint16_t *x, uint16_t *y, int64_t rows, int64_t cols, int dtype);

/* ---- reductions ------------------------------------------------------------ */
void oracle_rowsum_f32(const float *x, float *out, int64_t rows, int64_t cols, float init);       /* WG/reduction_2D_1D_cross_sg_cross_lane.mlir:31-37 */
void oracle_rowmean_f32(const float *x, float *out, int64_t rows, int64_t cols);                      /* WG/reduction_4D_3D_mean_intra_sg_intra_lane.mlir:115-127 */
void oracle_reduce_outer_f32(const float *x, float *out, int64_t outer, int64_t inner, float init); /* benchmarks/reduce/reduce_gpu.mlir.in:4-21 */
void oracle_reduce_outer_16(const uint16_t *x, uint16_t *out, int64_t outer, int64_t inner, float init, int dtype); /* same, 16-bit in/out, f32 accumulation */
float oracle_sum_all_f32(const float *x, int64_t n, float init);                                   /* test/PlaidML/OpTest.Sum.mlir:18-26 */

/* ---- transpose ------------------------------------------------------------- */
void oracle_transpose2d(const void *in, void *out, int64_t rows, int64_t cols, int elem_bytes);    /* benchmarks/transpose/transpose2d_gpu.mlir.in:4-11 */
void oracle_transpose3d(const void *in, void *out, int64_t d0, int64_t d1, int64_t d2, int elem_bytes); /* benchmarks/transpose/transpose3d_gpu.mlir.in:4-11 */

/* ---- GEMM ------------------------------------------------------------------- */
/* C[M,N] += A[M,K] . B[K,N], f32 accumulate, i-k-j order (ImexRunnerUtils.cpp:308-317).
   ab_dtype selects how A and B are read (f32 / f16 / bf16 bits); C is f32.
   out_round: ORACLE_F32 keeps f32, ORACLE_F16 / ORACLE_BF16 round the final sum
   to that type and widen it back (ImexRunnerUtils.cpp:322-333). */
void oracle_gemm(const void *A, const void *B, float *C, int64_t M, int64_t N, int64_t K,
                 int ab_dtype, int out_round);
/* Same arithmetic restricted to the listed rows of C (C_rows is [nrows, N]). */
void oracle_gemm_rows(const void *A, const void *B, float *C_rows, const int64_t *rows, int64_t nrows,
                      int64_t N, int64_t K, int ab_dtype);
void oracle_bias_add_rows(float *C, const float *bias, int64_t M, int64_t N);  /* WG/gemm_4kx4kx4k_f16_f16_f32_bias.mlir:164-172 */
/* out = bf16( silu( acc + bias[n] ) ) on an [M,N] f32 accumulator */
void oracle_bias_silu_bf16(const float *acc, const float *bias, uint16_t *out, int64_t M, int64_t N);

/* ---- checking helpers ------------------------------------------------------ */
int oracle_allclose_f32(const float *a, const float *ref, size_t n);  /* ImexRunnerUtils.cpp:185-205 */
void oracle_max_error_f32(const float *a, const float *b, size_t n, double *max_abs, double *max_rel); /* :217-255 */

/* ---- profiler statistics (ExecutionEngineUtils.cpp:18-150) ------------------ */
float oracle_stat_min(const float *v, size_t n);
float oracle_stat_max(const float *v, size_t n);
float oracle_stat_avg(const float *v, size_t n);
float oracle_stat_median_textbook(const float *v, size_t n);
float oracle_stat_median_reference(const float *v, size_t n); /* n >= 3 only (reference indexes n/2+1) */
float oracle_stat_stddev(const float *v, size_t n);
float oracle_stat_variance(const float *v, size_t n);
float oracle_stat_p95(const float *v, size_t n);
float oracle_stat_p5(const float *v, size_t n);
float oracle_stat_middle_third_avg(const float *v, size_t n);

/* ---- CPU-baseline timing legs (result buffer allocated inside each call,
        as in benchmarks/relu/relu_cpu.mlir.in:36-51) -------------------------- */
double oracle_time_relu_f32(const float *x, size_t n, int warmup, int runs);
double oracle_time_silu_f32(const float *x, size_t n, int warmup, int runs);
double oracle_time_softmax_f16(const uint16_t *x, int64_t rows, int64_t cols, int warmup, int runs);
double oracle_time_rowsum_f32(const float *x, int64_t rows, int64_t cols, int warmup, int runs);
double oracle_time_transpose2d(const void *x, int64_t rows, int64_t cols, int elem_bytes, int warmup, int runs);
double oracle_time_gemm_rows(const void *A, const void *B, int64_t nrows, int64_t N, int64_t K, int ab_dtype);
double oracle_time_mlp_rows(const void *A, const void *B, const float *bias, int64_t nrows, int64_t N, int64_t K);

#ifdef __cplusplus
}
#endif
#endif
