/*
 * CPU oracle -- TEST INFRASTRUCTURE ONLY (see oracle.h for scope and pinning).
 *
 * Build: -O1 -fno-tree-vectorize -ffp-contract=off, so the loop nests stay the
 * scalar, separately-rounded code the reference's linalg->loops->LLVM lowering
 * produces (benchmarks/pipelines/linalg-to-cpu.pp:12-19).
 */
#include "oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

/* ======================================================================== */
/* 16-bit float conversions                                                  */
/* ======================================================================== */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ImexRunnerUtils.cpp:137-159: shift exponent+mantissa into place, rebias,
   fix up Inf/NaN (second rebias) and zero/subnormal (renormalise by
   subtracting the 2^-14 magic), then or-in the sign. */
float oracle_half_to_float(uint16_t h) {
  const uint32_t shifted_exp = 0x7c00u << 13;
  uint32_t u = ((uint32_t)(h & 0x7fffu)) << 13;
  uint32_t e = u & shifted_exp;
  u += (127u - 15u) << 23;
  if (e == shifted_exp) {
    u += (127u - 15u) << 23;
  } else if (e == 0) {
    u += 1u << 23;
    u = f2u(u2f(u) - u2f(113u << 23));
  }
  u |= ((uint32_t)(h & 0x8000u)) << 16;
  return u2f(u);
}

/* ImexRunnerUtils.cpp:165-169 */
float oracle_bfloat_to_float(uint16_t b) { return u2f(((uint32_t)b) << 16); }

/* Round-to-nearest-even f32 -> f16.  NaN -> quiet NaN 0x7e00 | sign. */
uint16_t oracle_float_to_half(float f) {
  uint32_t u = f2u(f);
  uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  u &= 0x7fffffffu;
  uint16_t o;
  if (u >= 0x47800000u) {              /* |f| >= 65536: Inf or NaN */
    o = (u > 0x7f800000u) ? 0x7e00u : 0x7c00u;
  } else if (u < 0x38800000u) {        /* |f| < 2^-14: subnormal half or zero */
    /* adding 0.5f aligns the mantissa so the low bits are the half subnormal,
       with the hardware's RNE doing the rounding */
    float t = u2f(u) + 0.5f;
    o = (uint16_t)(f2u(t) - 0x3f000000u);
  } else {
    uint32_t mant_odd = (u >> 13) & 1u;
    u += ((uint32_t)(15 - 127) << 23) + 0xfffu;
    u += mant_odd;
    o = (uint16_t)(u >> 13);
  }
  return (uint16_t)(o | sign);
}

/* Round-to-nearest-even f32 -> bf16.  NaN -> 0x7fc0 | sign. */
uint16_t oracle_float_to_bfloat(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u)
    return (u & 0x80000000u) ? 0xffc0u : 0x7fc0u;
  uint32_t bias = ((u >> 16) & 1u) + 0x7fffu;
  u += bias;
  return (uint16_t)(u >> 16);
}

void oracle_half_to_float_n(const uint16_t *in, float *out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = oracle_half_to_float(in[i]);
}
void oracle_bfloat_to_float_n(const uint16_t *in, float *out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = oracle_bfloat_to_float(in[i]);
}
void oracle_float_to_half_n(const float *in, uint16_t *out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = oracle_float_to_half(in[i]);
}
void oracle_float_to_bfloat_n(const float *in, uint16_t *out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = oracle_float_to_bfloat(in[i]);
}

static inline float load_as_f32(const void *p, size_t i, int dtype) {
  switch (dtype) {
  case ORACLE_F16: return oracle_half_to_float(((const uint16_t *)p)[i]);
  case ORACLE_BF16: return oracle_bfloat_to_float(((const uint16_t *)p)[i]);
  default: return ((const float *)p)[i];
  }
}
static inline void store_from_f64(void *p, size_t i, int dtype, double x) {
  /* f64 -> f32 -> 16-bit, the route ImexRunnerUtils.cpp:44,48 takes
     (uniform_real_distribution<double> value handed to T(float)). */
  float f = (float)x;
  switch (dtype) {
  case ORACLE_F16: ((uint16_t *)p)[i] = oracle_float_to_half(f); break;
  case ORACLE_BF16: ((uint16_t *)p)[i] = oracle_float_to_bfloat(f); break;
  default: ((float *)p)[i] = f; break;
  }
}

/* ======================================================================== */
/* Seeded generators.  The reference seeds from std::random_device            */
/* (ImexRunnerUtils.cpp:42-43), so there is no stream to match; these use the  */
/* standardised raw output of std::mt19937 and transforms defined here.        */
/* ======================================================================== */

void oracle_mt_seed(oracle_mt19937 *g, uint32_t seed) {
  g->mt[0] = seed;
  for (int i = 1; i < 624; ++i)
    g->mt[i] = 1812433253u * (g->mt[i - 1] ^ (g->mt[i - 1] >> 30)) + (uint32_t)i;
  g->idx = 624;
}

uint32_t oracle_mt_next(oracle_mt19937 *g) {
  if (g->idx >= 624) {
    uint32_t *mt = g->mt;
    for (int i = 0; i < 624; ++i) {
      uint32_t y = (mt[i] & 0x80000000u) | (mt[(i + 1) % 624] & 0x7fffffffu);
      uint32_t v = mt[(i + 397) % 624] ^ (y >> 1);
      if (y & 1u) v ^= 0x9908b0dfu;
      mt[i] = v;
    }
    g->idx = 0;
  }
  uint32_t y = g->mt[g->idx++];
  y ^= y >> 11;
  y ^= (y << 7) & 0x9d2c5680u;
  y ^= (y << 15) & 0xefc60000u;
  y ^= y >> 18;
  return y;
}

/* u = (w >> 8) * 2^-24 in [0,1); x = lo + (hi - lo) * u in f64, then narrowed. */
void oracle_fill_uniform(void *out, size_t n, int dtype, uint32_t seed, double lo, double hi) {
  oracle_mt19937 g;
  oracle_mt_seed(&g, seed);
  for (size_t i = 0; i < n; ++i) {
    double u = (double)(oracle_mt_next(&g) >> 8) * (1.0 / 16777216.0);
    store_from_f64(out, i, dtype, lo + (hi - lo) * u);
  }
}

/* Box-Muller in f64: u1 = ((w1 >> 8) + 1) * 2^-24 in (0,1], u2 = (w2 >> 8) * 2^-24;
   element 2i takes r*cos(2 pi u2), element 2i+1 takes r*sin(2 pi u2). */
void oracle_fill_normal(void *out, size_t n, int dtype, uint32_t seed, double mu, double sigma) {
  oracle_mt19937 g;
  oracle_mt_seed(&g, seed);
  const double two_pi = 6.283185307179586476925286766559;
  for (size_t i = 0; i < n; i += 2) {
    double u1 = (double)((oracle_mt_next(&g) >> 8) + 1u) * (1.0 / 16777216.0);
    double u2 = (double)(oracle_mt_next(&g) >> 8) * (1.0 / 16777216.0);
    double r = sqrt(-2.0 * log(u1));
    store_from_f64(out, i, dtype, mu + sigma * (r * cos(two_pi * u2)));
    if (i + 1 < n)
      store_from_f64(out, i + 1, dtype, mu + sigma * (r * sin(two_pi * u2)));
  }
}

/* Raw words masked to the element width; NaN encodings are redrawn. */
void oracle_fill_bits_no_nan(void *out, size_t n, int dtype, uint32_t seed) {
  oracle_mt19937 g;
  oracle_mt_seed(&g, seed);
  for (size_t i = 0; i < n; ++i) {
    for (;;) {
      uint32_t w = oracle_mt_next(&g);
      if (dtype == ORACLE_F32) {
        if ((w & 0x7f800000u) == 0x7f800000u && (w & 0x007fffffu)) continue;
        ((uint32_t *)out)[i] = w;
      } else if (dtype == ORACLE_F16) {
        uint16_t h = (uint16_t)(w & 0xffffu);
        if ((h & 0x7c00u) == 0x7c00u && (h & 0x03ffu)) continue;
        ((uint16_t *)out)[i] = h;
      } else {
        uint16_t h = (uint16_t)(w & 0xffffu);
        if ((h & 0x7f80u) == 0x7f80u && (h & 0x007fu)) continue;
        ((uint16_t *)out)[i] = h;
      }
      break;
    }
  }
}

/* Integers uniform in [lo, hi] (inclusive), exactly representable in every
   dtype for the small ranges the exact-sum tests use. */
void oracle_fill_int_uniform(void *out, size_t n, int dtype, uint32_t seed, int lo, int hi) {
  oracle_mt19937 g;
  oracle_mt_seed(&g, seed);
  uint32_t span = (uint32_t)(hi - lo + 1);
  for (size_t i = 0; i < n; ++i) {
    uint32_t w = oracle_mt_next(&g);
    int v = lo + (int)(((uint64_t)w * span) >> 32);
    store_from_f64(out, i, dtype, (double)v);
  }
}

/* ======================================================================== */
/* Element-wise                                                               */
/* ======================================================================== */

/* benchmarks/relu/relu_gpu.mlir.in:8-10: %2 = cmpf ugt %in, 0 ; select %2, %in, 0.
   "ugt" is unordered-or-greater: NaN passes through with its payload; everything
   else that is not > 0 (including -0.0) becomes the constant +0.0. */
void oracle_relu_f32(const float *x, float *y, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    float v = x[i];
    int ugt = (v > 0.0f) || (v != v);
    y[i] = ugt ? v : 0.0f;
  }
}

void oracle_relu_16(const uint16_t *x, uint16_t *y, size_t n, int dtype) {
  for (size_t i = 0; i < n; ++i) {
    float v = load_as_f32(x, i, dtype);
    int ugt = (v > 0.0f) || (v != v);
    y[i] = ugt ? x[i] : (uint16_t)0;
  }
}

/* test/PlaidML/OpTest.Relu.mlir:29-35: select(x olt 0, 0, x) -- keeps -0.0 and NaN. */
void oracle_relu_olt_f32(const float *x, float *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = (x[i] < 0.0f) ? 0.0f : x[i];
}

/* benchmarks/silu/silu_gpu.mlir.in:8-18: negf, exp, addf 1, divf 1/., then a
   second generic multiplies sigmoid * x.  Five separately rounded f32 ops;
   exp is libm expf on the CPU path (linalg-to-cpu.pp:18-19). */
float oracle_silu_scalar_f32(float x) {
  float t = -x;
  float e = expf(t);
  float d = e + 1.0f;
  float s = 1.0f / d;
  return s * x;
}

void oracle_silu_f32(const float *x, float *y, size_t n) {
  for (size_t i = 0; i < n; ++i) y[i] = oracle_silu_scalar_f32(x[i]);
}

/* SiLU on 16-bit tensors: widen, the f32 chain above, one rounding (same policy;
   benchmarks/silu/silu.dtypes.in lists f16). */
void oracle_silu_16(const uint16_t *x, uint16_t *y, size_t n, int dtype) {
  for (size_t i = 0; i < n; ++i) {
    float in = dtype == ORACLE_F16 ? oracle_half_to_float(x[i]) : oracle_bfloat_to_float(x[i]);
    float out;
    oracle_silu_f32(&in, &out, 1);
    y[i] = dtype == ORACLE_F16 ? oracle_float_to_half(out) : oracle_float_to_bfloat(out);
  }
}

/* benchmarks/kLoopFusion/kLoopFusion.mlir.in:6-29: log, absf, addf, subf -- four
   separately rounded f32 ops; log is libm logf on the CPU path. */
void oracle_loop_fusion_f32(const float *a, const float *b, float *out, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    float t1 = logf(a[i]);
    float t2 = fabsf(b[i]);
    float t3 = t1 + t2;
    out[i] = t3 - a[i];
  }
}

/* benchmarks/kInputFusion/kInputFusion.mlir.in:8-39: log of the SECOND argument,
   absf of the first, addf, then out[j] = 0 + sum over rows i (ascending) of
   t[i][j] (maps (d1,d0) -> (d0), d1 the reduction). */
void oracle_input_fusion_f32(const float *a, const float *b, float *out, int64_t rows, int64_t cols) {
  for (int64_t j = 0; j < cols; ++j) {
    float acc = 0.0f;
    for (int64_t i = 0; i < rows; ++i) {
      float t1 = logf(b[i * cols + j]);
      float t2 = fabsf(a[i * cols + j]);
      float t3 = t1 + t2;
      acc = acc + t3;
    }
    out[j] = acc;
  }
}

/* test/Integration/Dialect/XeGPU/WG/flash_attention_fwd.mlir:332-421 (cpu_impl):
   per (batch, head), qk[i][j] = (sum_d q*k, f32, ascending d) * sm_scale; row max from
   -inf; exp2((qk - max) * log2e); sequential row sum; divide; P truncated to f16;
   out = f16(sum_k P[i][k] * v[k][j], f32, ascending k).  Q, K, V, out are
   [(ZH * n_ctx), d_head] f16; only the listed rows (global row indices) are
   computed, into out_rows[nrows][d_head]. */
void oracle_flash_attention_rows(const uint16_t *Q, const uint16_t *K, const uint16_t *V, uint16_t *out_rows,
                                 int64_t n_ctx, int64_t d_head, float sm_scale, const int64_t *rows,
                                 int64_t nrows) {
  const float log2e = 1.442695040888963f;
  float *qk = (float *)malloc((size_t)n_ctx * sizeof(float));
  for (int64_t ri = 0; ri < nrows; ++ri) {
    const int64_t row = rows[ri];
    const int64_t x_offset = (row / n_ctx) * n_ctx;
    for (int64_t j = 0; j < n_ctx; ++j) {
      float acc = 0.0f;
      for (int64_t k = 0; k < d_head; ++k) {
        float t = oracle_half_to_float(Q[row * d_head + k]) * oracle_half_to_float(K[(x_offset + j) * d_head + k]);
        acc = acc + t;
      }
      qk[j] = acc * sm_scale;
    }
    float mx = -INFINITY;
    for (int64_t j = 0; j < n_ctx; ++j) mx = (qk[j] > mx || mx != mx) ? qk[j] : mx; /* maximumf on non-NaN data */
    for (int64_t j = 0; j < n_ctx; ++j) {
      float t = qk[j] - mx;
      float t1 = t * log2e;
      qk[j] = exp2f(t1);
    }
    float sum = 0.0f;
    for (int64_t j = 0; j < n_ctx; ++j) sum = sum + qk[j];
    for (int64_t j = 0; j < n_ctx; ++j) qk[j] = qk[j] / sum;
    for (int64_t j = 0; j < d_head; ++j) {
      float pv = 0.0f;
      for (int64_t k = 0; k < n_ctx; ++k) {
        float p = oracle_half_to_float(oracle_float_to_half(qk[k]));
        float t = p * oracle_half_to_float(V[(x_offset + k) * d_head + j]);
        pv = t + pv;
      }
      out_rows[ri * d_head + j] = oracle_float_to_half(pv);
    }
  }
  free(qk);
}

void oracle_logf_n(const float *in, float *out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = logf(in[i]);
}

float oracle_expf_cr(float x) { return (float)exp((double)x); }

/* arith.maximumf, as the CPU loop of WG/arith_maximumf.mlir:122-129 applies it element by element:
   IEEE-754 maximum -- NaN if either operand is NaN (the first one, quieted, is what x86 code
   generation returns), +0 above -0. */
void oracle_maximum_f32(const float *a, const float *b, float *out, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    uint32_t ua, ub, r;
    memcpy(&ua, &a[i], 4);
    memcpy(&ub, &b[i], 4);
    if (a[i] != a[i]) r = ua | 0x00400000u;
    else if (b[i] != b[i]) r = ub | 0x00400000u;
    else if (a[i] == b[i]) r = (ua & 0x80000000u) ? ub : ua; /* equal values: -0 only if both are */
    else r = a[i] > b[i] ? ua : ub;
    memcpy(&out[i], &r, 4);
  }
}

void oracle_expf_n(const float *in, float *out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = expf(in[i]);
}

/* ======================================================================== */
/* Softmax                                                                    */
/* ======================================================================== */

/* arith.maxf / arith.maximumf: NaN if either operand is NaN. */
static inline float maximumf_(float a, float b) {
  if (a != a) return a;
  if (b != b) return b;
  return a > b ? a : b;
}

/* benchmarks/softmax/softmax_gpu.mlir.in:4-44.  Pass order of the reference:
   max (init -3.40282347E+38, :6) -> x - max -> exp -> sum (init 0, in + out)
   -> z / sum.  The dropped argmax side result (:8-20) is not computed. */
void oracle_softmax_f32(const float *x, float *y, int64_t rows, int64_t cols) {
  for (int64_t r = 0; r < rows; ++r) {
    const float *xr = x + r * cols;
    float *yr = y + r * cols;
    float m = -FLT_MAX;
    for (int64_t c = 0; c < cols; ++c) m = maximumf_(xr[c], m);
    for (int64_t c = 0; c < cols; ++c) yr[c] = xr[c] - m;
    for (int64_t c = 0; c < cols; ++c) yr[c] = expf(yr[c]);
    float s = 0.0f;
    for (int64_t c = 0; c < cols; ++c) s = yr[c] + s;
    for (int64_t c = 0; c < cols; ++c) yr[c] = yr[c] / s;
  }
}

/* WG/softmax_intra_sg_cross_lane.mlir:85-117 (the test's own CPU reference):
   max from -inf, exp(x - max) stored and summed in one pass, divide. */
void oracle_softmax_3pass_f32(const float *x, float *y, int64_t rows, int64_t cols) {
  for (int64_t r = 0; r < rows; ++r) {
    const float *xr = x + r * cols;
    float *yr = y + r * cols;
    float m = -INFINITY;
    for (int64_t c = 0; c < cols; ++c) m = maximumf_(m, xr[c]);
    float s = 0.0f;
    for (int64_t c = 0; c < cols; ++c) {
      float e = expf(xr[c] - m);
      yr[c] = e;
      s = s + e;
    }
    for (int64_t c = 0; c < cols; ++c) yr[c] = yr[c] / s;
  }
}

/* 16-bit input/output with f32 internals: truncf( softmax_f32( extf(x) ) ),
   the form the reference checks 16-bit variants against
   (test/Gen/PlaidML/OpTest.Softmax.mlir.in:1-5,47-50). */
void oracle_softmax_16(const uint16_t *x, uint16_t *y, int64_t rows, int64_t cols, int dtype) {
  float *xf = (float *)malloc((size_t)cols * sizeof(float));
  float *yf = (float *)malloc((size_t)cols * sizeof(float));
  for (int64_t r = 0; r < rows; ++r) {
    for (int64_t c = 0; c < cols; ++c) xf[c] = load_as_f32(x, (size_t)(r * cols + c), dtype);
    oracle_softmax_f32(xf, yf, 1, cols);
    for (int64_t c = 0; c < cols; ++c)
      y[r * cols + c] = dtype == ORACLE_F16 ? oracle_float_to_half(yf[c]) : oracle_float_to_bfloat(yf[c]);
  }
  free(xf);
  free(yf);
}

/* ======================================================================== */
/* Reductions                                                                 */
/* ======================================================================== */

/* out[i] = init + x[i,0] + x[i,1] + ... sequentially, left to right
   (vector.multi_reduction <add> with acc, WG/reduction_2D_1D_cross_sg_cross_lane.mlir:31-37;
    linalg form benchmarks/kInputFusion/kInputFusion.mlir.in:29-39). */
void oracle_rowsum_f32(const float *x, float *out, int64_t rows, int64_t cols, float init) {
  for (int64_t r = 0; r < rows; ++r) {
    float acc = init;
    const float *xr = x + r * cols;
    for (int64_t c = 0; c < cols; ++c) acc = acc + xr[c];
    out[r] = acc;
  }
}

/* WG/reduction_4D_3D_mean_intra_sg_intra_lane.mlir:115-127: the sequential sum from 0 over the last
   dimension, then one arith.divf by the dimension's length. */
void oracle_rowmean_f32(const float *x, float *out, int64_t rows, int64_t cols) {
  const float n = (float)cols;
  for (int64_t r = 0; r < rows; ++r) {
    float acc = 0.0f;
    const float *xr = x + r * cols;
    for (int64_t c = 0; c < cols; ++c) acc = acc + xr[c];
    out[r] = acc / n;
  }
}

/* benchmarks/reduce/reduce_gpu.mlir.in:4-21: in is [outer, inner...] and the
   OUTERMOST dimension is reduced: out[i] = init; for d3: out[i] = out[i] + in[d3, i]. */
void oracle_reduce_outer_f32(const float *x, float *out, int64_t outer, int64_t inner, float init) {
  for (int64_t i = 0; i < inner; ++i) {
    float acc = init;
    for (int64_t o = 0; o < outer; ++o) acc = acc + x[o * inner + i];
    out[i] = acc;
  }
}

/* The same reduction on 16-bit tensors: every element widened to f32 (exact), added in f32 in the
   same order, one rounding of the result (docs/Transforms/BF16ToGpu.md:17-26;
   benchmarks/reduce/reduce.dtypes.in lists f16 and bf16). */
void oracle_reduce_outer_16(const uint16_t *x, uint16_t *out, int64_t outer, int64_t inner, float init, int dtype) {
  for (int64_t i = 0; i < inner; ++i) {
    float acc = init;
    for (int64_t o = 0; o < outer; ++o) {
      uint16_t h = x[o * inner + i];
      acc = acc + (dtype == ORACLE_F16 ? oracle_half_to_float(h) : oracle_bfloat_to_float(h));
    }
    out[i] = dtype == ORACLE_F16 ? oracle_float_to_half(acc) : oracle_float_to_bfloat(acc);
  }
}

/* test/PlaidML/OpTest.Sum.mlir:18-26: both dims reduced into a 0-d tensor. */
float oracle_sum_all_f32(const float *x, int64_t n, float init) {
  float acc = init;
  for (int64_t i = 0; i < n; ++i) acc = acc + x[i];
  return acc;
}

/* ======================================================================== */
/* Transpose                                                                  */
/* ======================================================================== */

/* benchmarks/transpose/transpose2d_gpu.mlir.in:4-11: out[j,i] = in[i,j]; a pure
   move of elem_bytes per element, so NaN payloads and -0.0 survive. */
void oracle_transpose2d(const void *in, void *out, int64_t rows, int64_t cols, int elem_bytes) {
  if (elem_bytes == 4) {
    const uint32_t *src = (const uint32_t *)in;
    uint32_t *dst = (uint32_t *)out;
    for (int64_t i = 0; i < rows; ++i)
      for (int64_t j = 0; j < cols; ++j) dst[j * rows + i] = src[i * cols + j];
    return;
  }
  if (elem_bytes == 2) {
    const uint16_t *src = (const uint16_t *)in;
    uint16_t *dst = (uint16_t *)out;
    for (int64_t i = 0; i < rows; ++i)
      for (int64_t j = 0; j < cols; ++j) dst[j * rows + i] = src[i * cols + j];
    return;
  }
  const char *src = (const char *)in;
  char *dst = (char *)out;
  for (int64_t i = 0; i < rows; ++i)
    for (int64_t j = 0; j < cols; ++j)
      memcpy(dst + (size_t)(j * rows + i) * elem_bytes, src + (size_t)(i * cols + j) * elem_bytes,
             (size_t)elem_bytes);
}

/* benchmarks/transpose/transpose3d_gpu.mlir.in:4-11: full reversal (d2,d1,d0). */
void oracle_transpose3d(const void *in, void *out, int64_t d0, int64_t d1, int64_t d2, int elem_bytes) {
  const char *src = (const char *)in;
  char *dst = (char *)out;
  for (int64_t i = 0; i < d0; ++i)
    for (int64_t j = 0; j < d1; ++j)
      for (int64_t k = 0; k < d2; ++k)
        memcpy(dst + (size_t)((k * d1 + j) * d0 + i) * elem_bytes,
               src + (size_t)((i * d1 + j) * d2 + k) * elem_bytes, (size_t)elem_bytes);
}

/* ======================================================================== */
/* GEMM                                                                       */
/* ======================================================================== */

/* ImexRunnerUtils.cpp:283-317: widen A and B to f32 storage, then
   for i, for k, for j: C[i,j] += A[i,k] * B[k,j] with a rounded multiply and a
   rounded add (the reference is built without FMA contraction on x86-64). */
static void gemm_row(const float *a_row, const float *Bf, float *c_row, int64_t N, int64_t K) {
  for (int64_t k = 0; k < K; ++k) {
    float a = a_row[k];
    const float *b = Bf + k * N;
    for (int64_t j = 0; j < N; ++j) c_row[j] += a * b[j];
  }
}

static float *widen(const void *p, size_t n, int dtype) {
  float *f = (float *)malloc(n * sizeof(float));
  for (size_t i = 0; i < n; ++i) f[i] = load_as_f32(p, i, dtype);
  return f;
}

void oracle_gemm(const void *A, const void *B, float *C, int64_t M, int64_t N, int64_t K,
                 int ab_dtype, int out_round) {
  float *Af = widen(A, (size_t)(M * K), ab_dtype);
  float *Bf = widen(B, (size_t)(K * N), ab_dtype);
  for (int64_t i = 0; i < M; ++i) gemm_row(Af + i * K, Bf, C + i * N, N, K);
  /* ImexRunnerUtils.cpp:320-333: optional round trip of the result through the
     16-bit output type. */
  if (out_round == ORACLE_F16)
    for (int64_t i = 0; i < M * N; ++i) C[i] = oracle_half_to_float(oracle_float_to_half(C[i]));
  else if (out_round == ORACLE_BF16)
    for (int64_t i = 0; i < M * N; ++i) C[i] = oracle_bfloat_to_float(oracle_float_to_bfloat(C[i]));
  free(Af);
  free(Bf);
}

void oracle_gemm_rows(const void *A, const void *B, float *C_rows, const int64_t *rows, int64_t nrows,
                      int64_t N, int64_t K, int ab_dtype) {
  float *Bf = widen(B, (size_t)(K * N), ab_dtype);
  float *a_row = (float *)malloc((size_t)K * sizeof(float));
  for (int64_t r = 0; r < nrows; ++r) {
    for (int64_t k = 0; k < K; ++k) a_row[k] = load_as_f32(A, (size_t)(rows[r] * K + k), ab_dtype);
    gemm_row(a_row, Bf, C_rows + r * N, N, K);
  }
  free(a_row);
  free(Bf);
}

/* WG/gemm_4kx4kx4k_f16_f16_f32_bias.mlir:164-172: C_ref[i,j] = C_ref[i,j] + bias[j]. */
void oracle_bias_add_rows(float *C, const float *bias, int64_t M, int64_t N) {
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) C[i * N + j] = C[i * N + j] + bias[j];
}

/* MLP epilogue: f32 accumulator + bias[n] (bias.mlir:112) -> SiLU in the op
   order of silu_gpu.mlir.in:8-18 -> RNE to bf16. */
void oracle_bias_silu_bf16(const float *acc, const float *bias, uint16_t *out, int64_t M, int64_t N) {
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      float v = acc[i * N + j] + bias[j];
      out[i * N + j] = oracle_float_to_bfloat(oracle_silu_scalar_f32(v));
    }
}

/* ======================================================================== */
/* Checking helpers                                                           */
/* ======================================================================== */

/* ImexRunnerUtils.cpp:185-205: all-float arithmetic, atol 1e-4, rtol 1e-3,
   fails on |a - ref| > atol + rtol*|ref| (a NaN difference does not fail). */
int oracle_allclose_f32(const float *a, const float *ref, size_t n) {
  const float atol = 1e-04f;
  const float rtol = 1e-03f;
  for (size_t i = 0; i < n; ++i) {
    float lhs = a[i], rhs = ref[i];
    if (fabsf(lhs - rhs) > atol + rtol * fabsf(rhs)) return 0;
  }
  return 1;
}

/* ImexRunnerUtils.cpp:217-245: f64 deltas; relative error over max(|a|,|b|). */
void oracle_max_error_f32(const float *a, const float *b, size_t n, double *max_abs, double *max_rel) {
  double ma = 0.0, mr = 0.0;
  for (size_t i = 0; i < n; ++i) {
    double x = a[i], y = b[i];
    double d = fabs(x - y);
    double rel = d / fmax(fabs(x), fabs(y));
    if (d > ma) ma = d;
    if (rel > mr) mr = rel;
  }
  *max_abs = ma;
  *max_rel = mr;
}

/* ======================================================================== */
/* Profiler statistics (ExecutionEngineUtils.cpp)                              */
/* ======================================================================== */

static int cmp_float(const void *a, const void *b) {
  float x = *(const float *)a, y = *(const float *)b;
  return (x > y) - (x < y);
}
static float *sorted_copy(const float *v, size_t n) {
  float *s = (float *)malloc(n * sizeof(float));
  memcpy(s, v, n * sizeof(float));
  qsort(s, n, sizeof(float), cmp_float);
  return s;
}

float oracle_stat_min(const float *v, size_t n) { /* :18-25 */
  if (!n) return FLT_MAX;
  float m = v[0];
  for (size_t i = 1; i < n; ++i) if (v[i] < m) m = v[i];
  return m;
}
float oracle_stat_max(const float *v, size_t n) { /* :28-35; empty -> numeric_limits<float>::min() */
  if (!n) return FLT_MIN;
  float m = v[0];
  for (size_t i = 1; i < n; ++i) if (v[i] > m) m = v[i];
  return m;
}
float oracle_stat_avg(const float *v, size_t n) { /* :38-47: f32 running sum / n */
  if (!n) return 0.0f;
  float s = 0.0f;
  for (size_t i = 0; i < n; ++i) s += v[i];
  return s / (float)n;
}
float oracle_stat_median_textbook(const float *v, size_t n) {
  if (!n) return 0.0f;
  float *s = sorted_copy(v, n);
  float m = (n % 2) ? s[n / 2] : (s[n / 2] + s[n / 2 - 1]) / 2;
  free(s);
  return m;
}
/* :50-72 as written: the pivot index is n/2 + 1, one past the textbook one. */
float oracle_stat_median_reference(const float *v, size_t n) {
  if (n < 3) return 0.0f / 0.0f;
  float *s = sorted_copy(v, n);
  size_t idx = n / 2 + 1;
  float m = (n % 2) ? s[idx] : (s[idx] + s[idx - 1]) / 2;
  free(s);
  return m;
}
float oracle_stat_variance(const float *v, size_t n) { /* :92-104: population variance about the f32 mean */
  if (!n) return 0.0f;
  float mean = oracle_stat_avg(v, n);
  float s = 0.0f;
  for (size_t i = 0; i < n; ++i) s += (v[i] - mean) * (v[i] - mean);
  return s / (float)n;
}
float oracle_stat_stddev(const float *v, size_t n) { /* :75-89 */
  if (!n) return 0.0f;
  return sqrtf(oracle_stat_variance(v, n));
}
float oracle_stat_p95(const float *v, size_t n) { /* :107-117: element at floor(0.95 n) of the sorted run */
  if (!n) return 0.0f;
  size_t idx = (size_t)(0.95 * (double)n);
  if (idx >= n) idx = n - 1;
  float *s = sorted_copy(v, n);
  float r = s[idx];
  free(s);
  return r;
}
float oracle_stat_p5(const float *v, size_t n) { /* :120-130 */
  if (!n) return 0.0f;
  size_t idx = (size_t)(0.05 * (double)n);
  if (idx >= n) idx = n - 1;
  float *s = sorted_copy(v, n);
  float r = s[idx];
  free(s);
  return r;
}
float oracle_stat_middle_third_avg(const float *v, size_t n) { /* :134-150 */
  if (!n) return 0.0f;
  if (n < 3) return oracle_stat_median_textbook(v, n);
  float *s = sorted_copy(v, n);
  size_t start = n / 3, end = n - start;
  float sum = 0.0f;
  for (size_t i = start; i < end; ++i) sum += s[i];
  free(s);
  return sum / (float)(end - start);
}

/* ======================================================================== */
/* CPU-baseline timing legs                                                    */
/* Protocol of benchmarks/relu/relu_cpu.mlir.in:22-61: warm-up calls, then     */
/* `runs` calls each bracketed by a wall clock, the result buffer allocated    */
/* inside the timed call and freed outside it; returns the mean in ms.         */
/* ======================================================================== */

static double now_s(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}
static volatile float g_sink;

#define TIME_LOOP(ALLOC_BYTES, BODY)                                      \
  do {                                                                     \
    double total = 0.0;                                                    \
    for (int it = 0; it < warmup + runs; ++it) {                           \
      double t0 = now_s();                                                 \
      void *res = malloc(ALLOC_BYTES);                                     \
      BODY;                                                                \
      double t1 = now_s();                                                 \
      g_sink = ((volatile float *)res)[0];                                 \
      free(res);                                                           \
      if (it >= warmup) total += t1 - t0;                                  \
    }                                                                      \
    return runs ? 1e3 * total / runs : 0.0;                                \
  } while (0)

double oracle_time_relu_f32(const float *x, size_t n, int warmup, int runs) {
  TIME_LOOP(n * sizeof(float), oracle_relu_f32(x, (float *)res, n));
}
double oracle_time_silu_f32(const float *x, size_t n, int warmup, int runs) {
  TIME_LOOP(n * sizeof(float), oracle_silu_f32(x, (float *)res, n));
}
double oracle_time_softmax_f16(const uint16_t *x, int64_t rows, int64_t cols, int warmup, int runs) {
  TIME_LOOP((size_t)(rows * cols) * 2 + 4, oracle_softmax_16(x, (uint16_t *)res, rows, cols, ORACLE_F16));
}
double oracle_time_rowsum_f32(const float *x, int64_t rows, int64_t cols, int warmup, int runs) {
  TIME_LOOP((size_t)rows * sizeof(float), oracle_rowsum_f32(x, (float *)res, rows, cols, 0.0f));
}
double oracle_time_transpose2d(const void *x, int64_t rows, int64_t cols, int elem_bytes, int warmup, int runs) {
  TIME_LOOP((size_t)(rows * cols) * (size_t)elem_bytes + 4, oracle_transpose2d(x, res, rows, cols, elem_bytes));
}
/* One un-warmed call of the reference GEMM loop on the first nrows rows of C. */
double oracle_time_gemm_rows(const void *A, const void *B, int64_t nrows, int64_t N, int64_t K, int ab_dtype) {
  int64_t *rows = (int64_t *)malloc((size_t)nrows * sizeof(int64_t));
  for (int64_t i = 0; i < nrows; ++i) rows[i] = i;
  float *C = (float *)calloc((size_t)(nrows * N), sizeof(float));
  double t0 = now_s();
  oracle_gemm_rows(A, B, C, rows, nrows, N, K, ab_dtype);
  double t1 = now_s();
  g_sink = C[0];
  free(C);
  free(rows);
  return 1e3 * (t1 - t0);
}
/* The MLP layer on the first nrows rows: the GEMM loop, then bias + SiLU + rounding to bf16. */
double oracle_time_mlp_rows(const void *A, const void *B, const float *bias, int64_t nrows, int64_t N, int64_t K) {
  int64_t *rows = (int64_t *)malloc((size_t)nrows * sizeof(int64_t));
  for (int64_t i = 0; i < nrows; ++i) rows[i] = i;
  float *C = (float *)calloc((size_t)(nrows * N), sizeof(float));
  uint16_t *out = (uint16_t *)malloc((size_t)(nrows * N) * sizeof(uint16_t));
  double t0 = now_s();
  oracle_gemm_rows(A, B, C, rows, nrows, N, K, ORACLE_BF16);
  oracle_bias_silu_bf16(C, bias, out, nrows, N);
  double t1 = now_s();
  g_sink = (float)out[0];
  free(out);
  free(C);
  free(rows);
  return 1e3 * (t1 - t0);
}
