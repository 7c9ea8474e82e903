// Row-wise softmax over the last dimension.
//
// Reference: benchmarks/softmax/softmax_gpu.mlir.in:4-44 -- seven linalg ops
// (fill, max, sub, exp, fill, sum, div), each its own launch with full-size
// temporaries; single-kernel streaming form in
// test/Integration/Dialect/XeGPU/WG/softmax_intra_sg_cross_lane.mlir:118-205.
//
// Here: ONE kernel, input read once from HBM and output written once.
//  * rows of up to 128 lanes x 16 B (1024 16-bit / 512 f32 elements): a
//    wavefront owns a row and keeps it in registers; max and sum are wavefront-64
//    reductions on the VALU's cross-lane paths (DPP), no LDS.
//    f16: a wavefront walks rows w, w + W, ... with the next row's loads in
//    flight while it computes the current one, and the arithmetic is written for
//    the instruction count (packed f16 maximum, mixed-precision FMAs straight
//    from and into the f16 halves, one reciprocal per row): about 6 vector
//    instructions per element where the generic form below needs 14.
//    f32 / bf16: the generic form, a wavefront owns one row (two from 16384 rows
//    on, all loads issued before the first reduction), eight wavefronts per SIMD.
//  * rows of up to 4096 elements: a workgroup owns a row and stages it in LDS
//    as f32 (read once, three passes over LDS).
//  * longer rows: workgroup per row, the streaming form -- a running (max, sum)
//    pair rescaled as the maximum moves, then a second read of the row to
//    normalise (WG/softmax_intra_sg_cross_lane.mlir:135-175): two reads, one write.
// Internals are f32; 16-bit I/O follows the reference's policy for 16-bit types
// on the GPU: extend to f32, compute, truncate (docs/Transforms/BF16ToGpu.md:17-26).
//
// Arguments: (in, out, rows: i64, cols: i64).
// Launch: block (256,1,1); any grid >= 1 is correct (workgroups stride over the
// rows); the catalogue sizes it to one pass: ceil(rows/4) for register-resident
// rows (ceil(rows/8) from 16384 rows on; f16: min(ceil(rows/4), 2048) -- one
// wavefront per wavefront slot of the chip), else min(rows, 65535 * 16).

#include "device_common.h"

using namespace imexhip;

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kRegChunks = 2;          // 16-byte chunks per lane and row on the register path
constexpr int64_t kTwoRowsFrom = 16384; // rows from which a wavefront takes two: every wavefront slot of the chip is then filled
constexpr int kLdsCols = 4096;         // longest row staged in LDS

enum class Dt { F32, F16, BF16 };

template <Dt D> struct Elem;
template <> struct Elem<Dt::F32> {
  static constexpr int kBytes = 4;
  static constexpr int kPerVec = 4;
  static __device__ __forceinline__ void unpack(u32x4 v, float *f) {
    f[0] = u2f(v.x); f[1] = u2f(v.y); f[2] = u2f(v.z); f[3] = u2f(v.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float *f) {
    return u32x4{f2u(f[0]), f2u(f[1]), f2u(f[2]), f2u(f[3])};
  }
  static __device__ __forceinline__ float load(const void *p, int64_t i) { return static_cast<const float *>(p)[i]; }
  static __device__ __forceinline__ void store(void *p, int64_t i, float v) { static_cast<float *>(p)[i] = v; }
};
template <> struct Elem<Dt::F16> {
  static constexpr int kBytes = 2;
  static constexpr int kPerVec = 8;
  static __device__ __forceinline__ void unpack(u32x4 v, float *f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = half_bits_to_float(w[i] & 0xffffu);
      f[2 * i + 1] = half_bits_to_float(w[i] >> 16);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float *f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = float_to_half_bits(f[2 * i]) | (float_to_half_bits(f[2 * i + 1]) << 16);
    return u32x4{w[0], w[1], w[2], w[3]};
  }
  static __device__ __forceinline__ float load(const void *p, int64_t i) {
    return half_bits_to_float(static_cast<const uint16_t *>(p)[i]);
  }
  static __device__ __forceinline__ void store(void *p, int64_t i, float v) {
    static_cast<uint16_t *>(p)[i] = static_cast<uint16_t>(float_to_half_bits(v));
  }
};
template <> struct Elem<Dt::BF16> {
  static constexpr int kBytes = 2;
  static constexpr int kPerVec = 8;
  static __device__ __forceinline__ void unpack(u32x4 v, float *f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = bf16_bits_to_float(w[i] & 0xffffu);
      f[2 * i + 1] = bf16_bits_to_float(w[i] >> 16);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float *f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = float_to_bf16_bits(f[2 * i]) | (float_to_bf16_bits(f[2 * i + 1]) << 16);
    return u32x4{w[0], w[1], w[2], w[3]};
  }
  static __device__ __forceinline__ float load(const void *p, int64_t i) {
    return bf16_bits_to_float(static_cast<const uint16_t *>(p)[i]);
  }
  static __device__ __forceinline__ void store(void *p, int64_t i, float v) {
    static_cast<uint16_t *>(p)[i] = static_cast<uint16_t>(float_to_bf16_bits(v));
  }
};

// exp for the normalised row: the argument is <= 0, the result feeds a sum and
// a division whose outputs are compared at 1e-3, so the hardware exp2 is used.
__device__ __forceinline__ float fast_exp(float x) { return __expf(x); }

// The reference starts the running max at -3.40282347E+38, not -inf
// (softmax_gpu.mlir.in:6).
constexpr float kMaxInit = -3.40282347e+38f;

// ---- register path: a wavefront owns kRowsPerWave rows ---------------------------
template <Dt D, bool kStream, int kRowsPerWave>
__device__ __forceinline__ void softmax_rows_in_regs(const void *in, void *out, int64_t rows, int64_t cols) {
  using E = Elem<D>;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t vecsPerRow = cols / E::kPerVec;
  const int64_t rowBytes = cols * E::kBytes;
  const int64_t groups = (rows + kRowsPerWave - 1) / kRowsPerWave;
  for (int64_t g = int64_t(blockIdx.x) * kWaves + wave; g < groups; g += int64_t(gridDim.x) * kWaves) {
    float x[kRowsPerWave][kRegChunks][E::kPerVec];
    u32x4 raw[kRowsPerWave][kRegChunks];
    // all loads of both rows first
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
      const int64_t row = g * kRowsPerWave + r;
      const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(in) + row * rowBytes);
#pragma unroll
      for (int c = 0; c < kRegChunks; ++c) {
        const int64_t v = int64_t(c) * kWave + lane;
        if (row < rows && v < vecsPerRow)
          raw[r][c] = load128<kStream>(src + v);
      }
    }
#pragma unroll
    for (int r = 0; r < kRowsPerWave; ++r) {
      const int64_t row = g * kRowsPerWave + r;
      if (row >= rows)
        continue; // uniform across the wavefront
      float m = kMaxInit;
#pragma unroll
      for (int c = 0; c < kRegChunks; ++c) {
        const bool live = int64_t(c) * kWave + lane < vecsPerRow;
        if (live)
          E::unpack(raw[r][c], x[r][c]);
#pragma unroll
        for (int i = 0; i < E::kPerVec; ++i) {
          x[r][c][i] = live ? x[r][c][i] : kMaxInit;
          m = fmaxf(m, x[r][c][i]);
        }
      }
      m = wave_max(m);
      float s = 0.0f;
#pragma unroll
      for (int c = 0; c < kRegChunks; ++c) {
        const bool live = int64_t(c) * kWave + lane < vecsPerRow;
#pragma unroll
        for (int i = 0; i < E::kPerVec; ++i) {
          x[r][c][i] = live ? fast_exp(x[r][c][i] - m) : 0.0f;
          s += x[r][c][i];
        }
      }
      s = wave_sum(s);
      // one IEEE division per row, then multiplies (differs from z / s by at
      // most an f32 rounding, far inside the 1e-3 bar)
      const float inv = 1.0f / s;
      u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(out) + row * rowBytes);
#pragma unroll
      for (int c = 0; c < kRegChunks; ++c) {
        const int64_t v = int64_t(c) * kWave + lane;
        if (v < vecsPerRow) {
#pragma unroll
          for (int i = 0; i < E::kPerVec; ++i)
            x[r][c][i] = x[r][c][i] * inv;
          store128<kStream>(E::pack(x[r][c]), dst + v);
        }
      }
    }
  }
}

// ---- f16 rows in registers: the benchmark's path, written for the instruction count ----------
// At [16384,1024] every SIMD has 16384 elements to get through while 64 MiB stream past: the
// vector instructions per element, not the memory system, decide the run time.  Per element:
//   maximum       v_pk_max_f16 on the packed input words (exact in f16)                   1/2
//   exponent      one v_fma_mix_f32 straight from the f16 half: x*log2(e) - m*log2(e)      1
//   exponential   v_exp_f32 (quarter rate)                                                1
//   row sum       v_add_f32                                                               1
//   normalise     v_fma_mixlo/hi_f16: e * (1/sum), rounded to f16 into its half           1
// and no conversion instruction on either side.  m*log2(e) is rounded once per row; the error
// of that rounding multiplies every exponential of the row by the same factor and leaves the
// quotients alone.  f16 only: |m| <= 65504 keeps m*log2(e) finite (a bf16 or f32 maximum near
// 3e38 would not), and a row of nothing but -inf still comes out NaN (fma(-inf, c, +inf)), as
// the reference's 0/0 does.  Outputs are >= +0, so folding the final multiplication into the
// rounding instruction cannot lose a sign.
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
constexpr float kLog2e = 1.44269504088896340736f;

// The instruction itself: the builtin maximum puts a canonicalising v_pk_max_f16 x, x in front of
// every operand that comes from memory.  A NaN is passed over or (a signalling one) returned quiet;
// the row comes out all-NaN either way, through the sum.
__device__ __forceinline__ f16x2 pk_max_f16(f16x2 a, f16x2 b) {
  f16x2 d;
  asm("v_pk_max_f16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
  return d;
}

// One row of up to 1024 columns held by a wavefront as two 16-byte vectors per lane.
struct F16Row {
  u32x4 raw[kRegChunks];

  // kFull: the row is exactly 1024 columns.  Otherwise lanes whose vector lies past the end of the
  // row load the row's first vector instead (no lane is switched off, so the compiler can count the
  // loads in flight) and are given -inf afterwards, which the maximum and the sum pass over.
  template <bool kFull> __device__ __forceinline__ void load(const char *rowBase, int lane, int vecsPerRow) {
#pragma unroll
    for (int c = 0; c < kRegChunks; ++c) {
      const int v = c * kWave + lane;
      const int vc = kFull || v < vecsPerRow ? v : 0;
      raw[c] = load128<true>(reinterpret_cast<const u32x4 *>(rowBase) + vc);
    }
  }

  // kSite: a different number at every call site.  It goes into the code as a comment, which keeps
  // the compiler from merging the ends of two call sites into one block: the merged block waited for
  // every memory operation of every path into it, stores of the row before included.
  template <bool kFull, int kSite>
  __device__ __forceinline__ void softmax_and_store(char *rowBase, int lane, int vecsPerRow) {
    constexpr uint32_t kMinusInfPair = 0xfc00fc00u;
    f16x2 h[kRegChunks * 4];
#pragma unroll
    for (int c = 0; c < kRegChunks; ++c) {
      const bool live = kFull || c * kWave + lane < vecsPerRow;
      // (through named words: a bit cast applied directly to a vector component reads component 0)
      const uint32_t w0 = live ? raw[c].x : kMinusInfPair, w1 = live ? raw[c].y : kMinusInfPair,
                     w2 = live ? raw[c].z : kMinusInfPair, w3 = live ? raw[c].w : kMinusInfPair;
      h[4 * c + 0] = __builtin_bit_cast(f16x2, w0);
      h[4 * c + 1] = __builtin_bit_cast(f16x2, w1);
      h[4 * c + 2] = __builtin_bit_cast(f16x2, w2);
      h[4 * c + 3] = __builtin_bit_cast(f16x2, w3);
    }
    f16x2 m2 = pk_max_f16(pk_max_f16(pk_max_f16(h[0], h[1]), pk_max_f16(h[2], h[3])),
                          pk_max_f16(pk_max_f16(h[4], h[5]), pk_max_f16(h[6], h[7])));
    static_assert(kRegChunks == 2, "the maximum above is written out for eight words");
    // lanes past the end of a short row hold -inf; the reference's maximum starts at kMaxInit
    const float m = fmaxf(wave_max(fmaxf(static_cast<float>(m2.x), static_cast<float>(m2.y))), kMaxInit);
    const float negMl2 = -(m * kLog2e);
    float e[kRegChunks * 8];
#pragma unroll
    for (int i = 0; i < kRegChunks * 4; ++i) {
      e[2 * i] = __builtin_amdgcn_exp2f(__builtin_fmaf(static_cast<float>(h[i].x), kLog2e, negMl2));
      e[2 * i + 1] = __builtin_amdgcn_exp2f(__builtin_fmaf(static_cast<float>(h[i].y), kLog2e, negMl2));
    }
    float s0 = e[0], s1 = e[1];
#pragma unroll
    for (int i = 1; i < kRegChunks * 4; ++i) {
      s0 += e[2 * i];
      s1 += e[2 * i + 1];
    }
    const float s = wave_sum(s0 + s1);
    // one reciprocal per row (the hardware's estimate and a Newton step: within an ulp of 1 / s),
    // then multiplies; s = 0, inf or NaN all give a NaN row, like the reference's division
    float inv = __builtin_amdgcn_rcpf(s);
    inv = __builtin_fmaf(__builtin_fmaf(-s, inv, 1.0f), inv, inv);
#pragma unroll
    for (int c = 0; c < kRegChunks; ++c) {
      const int v = c * kWave + lane;
      uint32_t w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const f16x2 p = {static_cast<_Float16>(__builtin_fmaf(e[8 * c + 2 * i], inv, 0.0f)),
                         static_cast<_Float16>(__builtin_fmaf(e[8 * c + 2 * i + 1], inv, 0.0f))};
        w[i] = __builtin_bit_cast(uint32_t, p);
      }
      asm volatile("; softmax row, call site %0, vector %1" ::"n"(kSite), "n"(c));
      if (kFull || v < vecsPerRow)
        store128<true>(u32x4{w[0], w[1], w[2], w[3]}, reinterpret_cast<u32x4 *>(rowBase) + v);
    }
    asm volatile("; softmax row done, call site %0" ::"n"(kSite));
  }
};

// The walk: wavefront w of W takes rows w, w + W, w + 2W, ... and always has its next row's loads
// in flight while it works on the current one -- reads, vector work and writes of different rows
// overlap inside a wavefront as well as between wavefronts.  The loads are unconditional
// straight-line code in a branch of their own ("there is a next row" is uniform), so the wait in
// front of a row's arithmetic is for that row's two loads only and leaves the next row's in flight.
// Any grid is correct; the catalogue's grid gives every wavefront slot of the chip one wavefront.
template <bool kFull>
__device__ __forceinline__ void softmax_f16_rows_in_regs(const void *in, void *out, int64_t rows, int64_t cols) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t stride = int64_t(gridDim.x) * kWaves;
  const int vecsPerRow = static_cast<int>(cols / 8);
  const int64_t rowBytes = cols * 2;
  const char *src = static_cast<const char *>(in);
  char *dst = static_cast<char *>(out);
  // the wavefront's number as a scalar, so that row addresses are formed on the scalar unit
  int64_t row = int64_t(blockIdx.x) * kWaves + __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  if (row >= rows || vecsPerRow == 0)
    return;
  F16Row a, b;
  a.load<kFull>(src + row * rowBytes, lane, vecsPerRow);
  if (row + stride >= rows) {
    a.softmax_and_store<kFull, 1>(dst + row * rowBytes, lane, vecsPerRow);
    return;
  }
  // The first row is taken outside the loop so that the loop is entered, the first time and every
  // later time, with the same memory operations in flight (a row's loads, then the row before's two
  // stores): the wait counts inside are then exact and never wait for a store.
  b.load<kFull>(src + (row + stride) * rowBytes, lane, vecsPerRow);
  __builtin_amdgcn_sched_barrier(0); // the loads stay in front of the wait for the current row
  a.softmax_and_store<kFull, 2>(dst + row * rowBytes, lane, vecsPerRow);
  row += stride;
  for (;;) {
    // b holds `row`
    if (row + stride < rows) {
      a.load<kFull>(src + (row + stride) * rowBytes, lane, vecsPerRow);
      __builtin_amdgcn_sched_barrier(0);
      b.softmax_and_store<kFull, 3>(dst + row * rowBytes, lane, vecsPerRow);
    } else {
      b.softmax_and_store<kFull, 4>(dst + row * rowBytes, lane, vecsPerRow);
      return;
    }
    row += stride;
    // a holds `row`
    if (row + stride < rows) {
      b.load<kFull>(src + (row + stride) * rowBytes, lane, vecsPerRow);
      __builtin_amdgcn_sched_barrier(0);
      a.softmax_and_store<kFull, 5>(dst + row * rowBytes, lane, vecsPerRow);
    } else {
      a.softmax_and_store<kFull, 6>(dst + row * rowBytes, lane, vecsPerRow);
      return;
    }
    row += stride;
  }
}

// ---- workgroup reductions -------------------------------------------------------------
__device__ __forceinline__ float block_reduce(float v, bool isMax, float *scratch) {
  v = isMax ? wave_max(v) : wave_sum(v);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  __syncthreads(); // scratch may still be read from a previous reduction
  if (lane == 0)
    scratch[wave] = v;
  __syncthreads();
  float r = scratch[0];
#pragma unroll
  for (int w = 1; w < kWaves; ++w)
    r = isMax ? fmaxf(r, scratch[w]) : r + scratch[w];
  return r;
}

// ---- LDS path: a workgroup owns a row, staged once in LDS as f32 ------------------------
template <Dt D>
__device__ __forceinline__ void softmax_row_in_lds(const void *in, void *out, int64_t row, int64_t cols,
                                                   float *rowBuf, float *scratch, bool vec) {
  using E = Elem<D>;
  const int64_t base = row * cols;
  float m = kMaxInit;
  // Vector path: element i of 16-byte vector v lives at rowBuf[i * vecs + v], so
  // neighbouring lanes touch neighbouring LDS words (no bank conflicts).
  const int64_t vecs = cols / E::kPerVec;
  if (vec) {
    const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(in) + base * E::kBytes);
    for (int64_t v = threadIdx.x; v < vecs; v += kThreads) {
      float f[E::kPerVec];
      E::unpack(src[v], f);
#pragma unroll
      for (int i = 0; i < E::kPerVec; ++i) {
        rowBuf[i * vecs + v] = f[i];
        m = fmaxf(m, f[i]);
      }
    }
  } else {
    for (int64_t c = threadIdx.x; c < cols; c += kThreads) {
      const float f = E::load(in, base + c);
      rowBuf[c] = f;
      m = fmaxf(m, f);
    }
  }
  m = block_reduce(m, true, scratch); // its barriers also publish rowBuf
  float s = 0.0f;
  // each thread revisits exactly the elements it wrote: no barrier needed until the sum
  if (vec) {
    for (int64_t v = threadIdx.x; v < vecs; v += kThreads)
#pragma unroll
      for (int i = 0; i < E::kPerVec; ++i) {
        const float e = fast_exp(rowBuf[i * vecs + v] - m);
        rowBuf[i * vecs + v] = e;
        s += e;
      }
  } else {
    for (int64_t c = threadIdx.x; c < cols; c += kThreads) {
      const float e = fast_exp(rowBuf[c] - m);
      rowBuf[c] = e;
      s += e;
    }
  }
  s = block_reduce(s, false, scratch);
  // normalised like the other two paths: one IEEE reciprocal per row, then multiplies (an f32 rounding away
  // from e / s at most, the same on every path, so a row's last bit does not depend on its length class)
  const float inv = 1.0f / s;
  if (vec) {
    u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(out) + base * E::kBytes);
    for (int64_t v = threadIdx.x; v < vecs; v += kThreads) {
      float f[E::kPerVec];
#pragma unroll
      for (int i = 0; i < E::kPerVec; ++i)
        f[i] = rowBuf[i * vecs + v] * inv;
      dst[v] = E::pack(f);
    }
  } else {
    for (int64_t c = threadIdx.x; c < cols; c += kThreads)
      E::store(out, base + c, rowBuf[c] * inv);
  }
  __syncthreads(); // rowBuf is reused by the next row
}

// ---- any length: workgroup per row, the input read twice -----------------------------------
// The streaming form of test/Integration/Dialect/XeGPU/WG/softmax_intra_sg_cross_lane.mlir:135-175:
// one pass carries a running maximum m and a running sum s of exp(x - m), rescaling s by
// exp(m_old - m_new) whenever the maximum moves; a second pass over the input normalises.  Here a
// lane moves its maximum once per 16-byte vector (one rescale per vector, not per element), and the
// lanes' (m, s) pairs are merged the same way: S = sum_i s_i exp(m_i - M), M = max_i m_i.
struct RunningSoftmax {
  float m = kMaxInit, s = 0.0f;
  template <int N> __device__ __forceinline__ void add(const float (&x)[N]) {
    float mx = m;
#pragma unroll
    for (int i = 0; i < N; ++i)
      mx = fmaxf(mx, x[i]);
    float t = s * fast_exp(m - mx); // m == mx: exp(0) = 1; first vector: s = 0
#pragma unroll
    for (int i = 0; i < N; ++i)
      t += fast_exp(x[i] - mx); // a NaN element, which fmaxf passes over, makes the sum NaN here
    m = mx;
    s = t;
  }
};

template <Dt D>
__device__ __forceinline__ void softmax_row_streamed(const void *in, void *out, int64_t row, int64_t cols,
                                                     float *scratch, bool vec) {
  using E = Elem<D>;
  const int64_t base = row * cols;
  const int64_t vecs = cols / E::kPerVec;
  const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(in) + base * E::kBytes);
  RunningSoftmax run;
  if (vec) {
    // two vectors in flight per lane
    int64_t v = threadIdx.x;
    for (; v + kThreads < vecs; v += 2 * kThreads) {
      const u32x4 r0 = src[v], r1 = src[v + kThreads];
      float f0[E::kPerVec], f1[E::kPerVec];
      E::unpack(r0, f0);
      E::unpack(r1, f1);
      run.add(f0);
      run.add(f1);
    }
    if (v < vecs) {
      float f[E::kPerVec];
      E::unpack(src[v], f);
      run.add(f);
    }
  } else {
    for (int64_t c = threadIdx.x; c < cols; c += kThreads) {
      const float f[1] = {E::load(in, base + c)};
      run.add(f);
    }
  }
  // merge the 256 running pairs: the row maximum, then every lane's sum brought to it
  const float m = block_reduce(run.m, true, scratch);
  const float sum = block_reduce(run.s * fast_exp(run.m - m), false, scratch);
  // one IEEE division per row, then multiplies (an f32 rounding away from z / s at most); a sum of
  // zero (a row of -inf) gives 0 * inf = NaN like the 0 / 0 of the reference's division
  const float inv = 1.0f / sum;
  if (vec) {
    u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(out) + base * E::kBytes);
    for (int64_t v = threadIdx.x; v < vecs; v += kThreads) {
      float f[E::kPerVec];
      E::unpack(src[v], f);
#pragma unroll
      for (int i = 0; i < E::kPerVec; ++i)
        f[i] = fast_exp(f[i] - m) * inv;
      dst[v] = E::pack(f);
    }
  } else {
    for (int64_t c = threadIdx.x; c < cols; c += kThreads)
      E::store(out, base + c, fast_exp(E::load(in, base + c) - m) * inv);
  }
}

template <Dt D>
__device__ __forceinline__ void softmax_kernel(const void *in, void *out, int64_t rows, int64_t cols) {
  using E = Elem<D>;
  __shared__ float scratch[kWaves];
  __shared__ __attribute__((aligned(16))) float rowBuf[kLdsCols];
  const bool aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 &&
                       (cols % E::kPerVec) == 0;
  if (aligned && cols <= int64_t(kRegChunks) * kWave * E::kPerVec) {
    // non-temporal accesses: measured faster hot and cold
    if constexpr (D == Dt::F16) {
      if (cols == int64_t(kRegChunks) * kWave * 8)
        softmax_f16_rows_in_regs<true>(in, out, rows, cols);
      else
        softmax_f16_rows_in_regs<false>(in, out, rows, cols);
    } else if (rows >= kTwoRowsFrom)
      softmax_rows_in_regs<D, true, 2>(in, out, rows, cols);
    else
      softmax_rows_in_regs<D, true, 1>(in, out, rows, cols);
  } else if (cols <= kLdsCols) {
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x)
      softmax_row_in_lds<D>(in, out, row, cols, rowBuf, scratch, aligned);
  } else {
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x)
      softmax_row_streamed<D>(in, out, row, cols, scratch, aligned);
  }
}

} // namespace

// 8 wavefronts per SIMD (64 registers per lane) so two rows per wavefront still
// leave room for full occupancy.
#define IMEX_SOFTMAX_BOUNDS __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(8, 8)))

extern "C" __global__ IMEX_SOFTMAX_BOUNDS void imex_softmax_f32(const float *in, float *out, int64_t rows,
                                                                int64_t cols) {
  softmax_kernel<Dt::F32>(in, out, rows, cols);
}
extern "C" __global__ IMEX_SOFTMAX_BOUNDS void imex_softmax_f16(const uint16_t *in, uint16_t *out, int64_t rows,
                                                                int64_t cols) {
  softmax_kernel<Dt::F16>(in, out, rows, cols);
}
extern "C" __global__ IMEX_SOFTMAX_BOUNDS void imex_softmax_bf16(const uint16_t *in, uint16_t *out, int64_t rows,
                                                                 int64_t cols) {
  softmax_kernel<Dt::BF16>(in, out, rows, cols);
}
