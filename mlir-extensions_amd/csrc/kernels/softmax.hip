// Row-wise softmax over the last dimension.
//
// Reference: benchmarks/softmax/softmax_gpu.mlir.in:4-44 -- seven linalg ops
// (fill, max, sub, exp, fill, sum, div), each its own launch with full-size
// temporaries; single-kernel streaming form in
// test/Integration/Dialect/XeGPU/WG/softmax_intra_sg_cross_lane.mlir:118-205.
//
// Here: ONE kernel, input read once and output written once.  A wavefront owns
// a row and keeps it in registers (128-bit loads, 8 x 16-bit or 4 x f32 per
// load), max and sum are wavefront-64 butterfly reductions, internals are f32.
// Rows too long for registers, or whose length breaks 16-byte alignment, go
// through a workgroup-per-row path that re-reads the row from cache.
//
// 16-bit I/O follows the reference's policy for 16-bit types on the GPU:
// extend to f32, compute, truncate (docs/Transforms/BF16ToGpu.md:17-26).
//
// Arguments: (in, out, rows: i64, cols: i64).
// Launch: block (256,1,1); grid (ceil(rows / 4), 1, 1)  [4 wavefronts = 4 rows].

#include "device_common.h"

using namespace imexhip;

namespace {

constexpr int kThreads = 256;
constexpr int kRowsPerBlock = kThreads / kWave;
// Up to kMaxChunks 16-byte chunks per lane live in registers.
constexpr int kMaxChunks = 8;

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

// ---- wavefront-per-row, row resident in registers ---------------------------
template <Dt D, int kChunks>
__device__ __forceinline__ void softmax_row_in_regs(const void *in, void *out, int64_t row, int64_t cols) {
  using E = Elem<D>;
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t vecsPerRow = cols / E::kPerVec; // cols is a multiple of kPerVec here
  const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(in) + row * cols * E::kBytes);
  u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(out) + row * cols * E::kBytes);

  float x[kChunks][E::kPerVec];
  float m = kMaxInit;
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    const int64_t v = int64_t(c) * kWave + lane;
    if (v < vecsPerRow) {
      E::unpack(__builtin_nontemporal_load(src + v), x[c]);
#pragma unroll
      for (int i = 0; i < E::kPerVec; ++i)
        m = fmaxf(m, x[c][i]);
    } else {
#pragma unroll
      for (int i = 0; i < E::kPerVec; ++i)
        x[c][i] = kMaxInit;
    }
  }
  m = wave_max(m);

  float s = 0.0f;
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    const bool live = int64_t(c) * kWave + lane < vecsPerRow;
#pragma unroll
    for (int i = 0; i < E::kPerVec; ++i) {
      x[c][i] = live ? fast_exp(x[c][i] - m) : 0.0f;
      s += x[c][i];
    }
  }
  s = wave_sum(s);

#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    const int64_t v = int64_t(c) * kWave + lane;
    if (v < vecsPerRow) {
#pragma unroll
      for (int i = 0; i < E::kPerVec; ++i)
        x[c][i] = x[c][i] / s;
      __builtin_nontemporal_store(E::pack(x[c]), dst + v);
    }
  }
}

// ---- workgroup-per-row, any length and alignment ------------------------------
__device__ __forceinline__ float block_reduce(float v, bool isMax, float *scratch) {
  v = isMax ? wave_max(v) : wave_sum(v);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  __syncthreads(); // scratch may still be read from a previous reduction
  if (lane == 0)
    scratch[wave] = v;
  __syncthreads();
  float r = scratch[0];
#pragma unroll
  for (int w = 1; w < kRowsPerBlock; ++w)
    r = isMax ? fmaxf(r, scratch[w]) : r + scratch[w];
  return r;
}

template <Dt D>
__device__ __forceinline__ void softmax_row_streamed(const void *in, void *out, int64_t row, int64_t cols,
                                                     float *scratch) {
  using E = Elem<D>;
  const int64_t base = row * cols;
  float m = kMaxInit;
  for (int64_t c = threadIdx.x; c < cols; c += kThreads)
    m = fmaxf(m, E::load(in, base + c));
  m = block_reduce(m, true, scratch);
  float s = 0.0f;
  for (int64_t c = threadIdx.x; c < cols; c += kThreads)
    s += fast_exp(E::load(in, base + c) - m);
  s = block_reduce(s, false, scratch);
  for (int64_t c = threadIdx.x; c < cols; c += kThreads)
    E::store(out, base + c, fast_exp(E::load(in, base + c) - m) / s);
}

template <Dt D>
__device__ __forceinline__ void softmax_kernel(const void *in, void *out, int64_t rows, int64_t cols) {
  using E = Elem<D>;
  __shared__ float scratch[kRowsPerBlock];
  const bool aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 &&
                       (cols % E::kPerVec) == 0;
  const int64_t chunks = (cols / E::kPerVec + kWave - 1) / kWave;
  const int64_t row0 = int64_t(blockIdx.x) * kRowsPerBlock;
  if (aligned && chunks <= kMaxChunks) {
    const int64_t row = row0 + threadIdx.x / kWave;
    if (row >= rows)
      return;
    if (chunks <= 1)
      softmax_row_in_regs<D, 1>(in, out, row, cols);
    else if (chunks <= 2)
      softmax_row_in_regs<D, 2>(in, out, row, cols);
    else if (chunks <= 4)
      softmax_row_in_regs<D, 4>(in, out, row, cols);
    else
      softmax_row_in_regs<D, kMaxChunks>(in, out, row, cols);
  } else {
    // Uniform per workgroup: every thread walks the same rows, so the barriers
    // inside block_reduce are reached by all of them.
    for (int r = 0; r < kRowsPerBlock; ++r) {
      const int64_t row = row0 + r;
      if (row >= rows)
        break;
      softmax_row_streamed<D>(in, out, row, cols, scratch);
    }
  }
}

} // namespace

extern "C" __global__ __launch_bounds__(kThreads) void imex_softmax_f32(const float *in, float *out,
                                                                       int64_t rows, int64_t cols) {
  softmax_kernel<Dt::F32>(in, out, rows, cols);
}
extern "C" __global__ __launch_bounds__(kThreads) void imex_softmax_f16(const uint16_t *in, uint16_t *out,
                                                                       int64_t rows, int64_t cols) {
  softmax_kernel<Dt::F16>(in, out, rows, cols);
}
extern "C" __global__ __launch_bounds__(kThreads) void imex_softmax_bf16(const uint16_t *in, uint16_t *out,
                                                                        int64_t rows, int64_t cols) {
  softmax_kernel<Dt::BF16>(in, out, rows, cols);
}
