// Sum reductions, f32.
//
//  * imex_rowsum_f32: out[r] = init + sum_c in[r, c]  (row-sum / last-dim form:
//    test/Integration/Dialect/XeGPU/WG/reduction_2D_1D_cross_sg_cross_lane.mlir:31-37,
//    benchmarks/kInputFusion/kInputFusion.mlir.in:29-39).
//    The reference's linalg path runs the whole sum in one work-item
//    (test/SPIRV/OpTest.Sum_FLOAT32.mlir:39); here a workgroup (or a wavefront,
//    for short rows) owns a row, streams it once with 128-bit loads, and
//    combines partial sums with wavefront-64 butterflies and one LDS hop.
//  * imex_reduce_outer_f32 / _f16 / _bf16: out[i] = init + sum_o in[o, i], the OUTERMOST
//    dimension reduced (benchmarks/reduce/reduce_gpu.mlir.in:4-21).  Each lane
//    owns groups of four adjacent outputs and adds the `outer` slices in order,
//    which is the reference's summation order, so this one is bit-exact.
//
//  * imex_rowmean_f32: out[r] = (0 + sum_c in[r, c]) / cols, the same reduction with the
//    division the reference applies afterwards
//    (WG/reduction_4D_3D_mean_intra_sg_intra_lane.mlir:51-52, 1x24x1024x64 -> 1x24x1024x1).
//
// Arguments: rowsum (in, out, rows: i64, cols: i64, init: f32); rowmean (in, out, rows: i64, cols: i64);
//            reduce_outer (in, out, outer: i64, inner: i64, init: f32).
// Launch: block (256,1,1);
//   rowsum: cols > 2048 -> grid (rows,1,1) [workgroup per row],
//           else grid (ceil(rows/4),1,1)  [wavefront per row];
//   reduce_outer: grid (ceil(inner / (1024 v)), 1, 1), v = 8, 4, 2 or 1: the largest that leaves
//           512 workgroups (any other grid works too, the workgroups stride).

#include "device_common.h"

using namespace imexhip;

namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / kWave;
constexpr int64_t kWavePerRowMaxCols = 2048;

template <bool kStream> __device__ __forceinline__ f32x4 loadf4(const f32x4 *p) {
  if constexpr (kStream)
    return __builtin_nontemporal_load(p);
  else
    return *p;
}

// Partial sum of one row over the lanes [tid, tid+stride, ...).
template <bool kStream>
__device__ __forceinline__ float row_partial(const float *__restrict__ row, int64_t cols, int tid, int stride) {
  float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if ((reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    const int64_t vecs = cols / 4;
    const f32x4 *src = reinterpret_cast<const f32x4 *>(row);
    int64_t v = tid;
    // four independent 16-byte loads in flight per lane
    for (; v + 3 * int64_t(stride) < vecs; v += 4 * int64_t(stride)) {
      f32x4 a = loadf4<kStream>(src + v);
      f32x4 b = loadf4<kStream>(src + v + stride);
      f32x4 c = loadf4<kStream>(src + v + 2 * int64_t(stride));
      f32x4 d = loadf4<kStream>(src + v + 3 * int64_t(stride));
      acc[0] += (a.x + a.y) + (a.z + a.w);
      acc[1] += (b.x + b.y) + (b.z + b.w);
      acc[2] += (c.x + c.y) + (c.z + c.w);
      acc[3] += (d.x + d.y) + (d.z + d.w);
    }
    for (; v < vecs; v += stride) {
      f32x4 a = loadf4<kStream>(src + v);
      acc[0] += (a.x + a.y) + (a.z + a.w);
    }
    for (int64_t c = vecs * 4 + tid; c < cols; c += stride)
      acc[1] += row[c];
  } else {
    for (int64_t c = tid; c < cols; c += stride)
      acc[0] += row[c];
  }
  return (acc[0] + acc[1]) + (acc[2] + acc[3]);
}

} // namespace

// kMean: the sum (from `init`) divided by the row length, the post-op of
// WG/reduction_4D_3D_mean_intra_sg_intra_lane.mlir:51-52.
template <bool kMean>
__device__ __forceinline__ void row_reduce(const float *in, float *out, int64_t rows, int64_t cols, float init) {
  const float divisor = static_cast<float>(cols);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  // the input is read exactly once: stream it past the caches (non-temporal)
  constexpr bool stream = true;
  // workgroups (wavefronts) stride over the rows, so any grid covers all of them
  if (cols > kWavePerRowMaxCols) {
    __shared__ float partial[kWavesPerBlock];
    for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
      const float p = stream ? row_partial<true>(in + row * cols, cols, threadIdx.x, kThreads)
                             : row_partial<false>(in + row * cols, cols, threadIdx.x, kThreads);
      float s = wave_sum(p);
      if (lane == 0)
        partial[wave] = s;
      __syncthreads();
      if (threadIdx.x == 0)
        out[row] = kMean ? (init + ((partial[0] + partial[1]) + (partial[2] + partial[3]))) / divisor
                         : init + ((partial[0] + partial[1]) + (partial[2] + partial[3]));
      __syncthreads(); // `partial` is reused by the next row
    }
  } else {
    for (int64_t row = int64_t(blockIdx.x) * kWavesPerBlock + wave; row < rows;
         row += int64_t(gridDim.x) * kWavesPerBlock) {
      const float p = stream ? row_partial<true>(in + row * cols, cols, lane, kWave)
                             : row_partial<false>(in + row * cols, cols, lane, kWave);
      float s = wave_sum(p);
      if (lane == 0)
        out[row] = kMean ? (init + s) / divisor : init + s;
    }
  }
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_rowsum_f32(const float *in, float *out, int64_t rows,
                                                                      int64_t cols, float init) {
  row_reduce<false>(in, out, rows, cols, init);
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_rowmean_f32(const float *in, float *out, int64_t rows,
                                                                       int64_t cols) {
  row_reduce<true>(in, out, rows, cols, 0.0f);
}

// Outer-dimension sum: lane owns kVecs vectors of four adjacent outputs, 4 KiB apart, so a
// workgroup reads kVecs * 4 KiB contiguous bytes of every slice.  With `outer` slices a power-of-two
// number of bytes apart, all of a lane's loads fall into the same DRAM channel; wide contiguous
// spans per workgroup are what keeps the channels streaming (measured on 32 x 4 Mi: 111 us with
// 4 KiB spans, 83 us with 32 KiB).  Four slices' loads are kept in flight (a register ring), adds
// kept in slice order.  Workgroups stride over the blocks of outputs, so any grid covers everything.
template <io::Dt D, int kVecs>
__device__ __forceinline__ void reduce_outer_vec(const void *__restrict__ in, void *__restrict__ out, int64_t outer,
                                                 int64_t inner, float init) {
  using E = io::Elem<D>;
  constexpr int kPer = E::kPerVec;                             // outputs per 16-byte vector: 4 or 8
  constexpr int64_t kSpan = int64_t(kThreads) * kPer * kVecs;  // outputs per workgroup and pass
  const u32x4 *src = static_cast<const u32x4 *>(in);
  const int64_t strideVecs = inner / kPer;
  for (int64_t base = int64_t(blockIdx.x) * kSpan; base < inner; base += int64_t(gridDim.x) * kSpan) {
    const int64_t i0 = base + threadIdx.x * kPer;
    float acc[kVecs][kPer];
#pragma unroll
    for (int v = 0; v < kVecs; ++v)
#pragma unroll
      for (int e = 0; e < kPer; ++e)
        acc[v][e] = init;
    auto add = [&](int v, u32x4 raw) {
      float f[kPer];
      E::unpack(raw, f);
#pragma unroll
      for (int e = 0; e < kPer; ++e)
        acc[v][e] = acc[v][e] + f[e];
    };
    // Lanes past the end of the last block read the last vector instead (and store nothing): the loads
    // are unconditional, so the wait for one slice leaves the loads of the next three in flight.
    int64_t at[kVecs];
#pragma unroll
    for (int v = 0; v < kVecs; ++v) {
      const int64_t i = i0 + v * (kThreads * kPer);
      at[v] = (i < inner ? i : inner - kPer) / kPer;
    }
    // A ring of four slices: slice o is added, in slice order, and its registers are at once reloaded with
    // slice o + 4, so three to four slices' loads are in flight all the time.
    constexpr int kRing = 4;
    int64_t o = 0;
    if (outer >= kRing) {
      u32x4 t[kRing][kVecs];
#pragma unroll
      for (int u = 0; u < kRing; ++u)
#pragma unroll
        for (int v = 0; v < kVecs; ++v)
          t[u][v] = __builtin_nontemporal_load(src + at[v] + u * strideVecs);
      for (; o + 2 * kRing <= outer; o += kRing) {
#pragma unroll
        for (int u = 0; u < kRing; ++u) {
#pragma unroll
          for (int v = 0; v < kVecs; ++v)
            add(v, t[u][v]);
#pragma unroll
          for (int v = 0; v < kVecs; ++v)
            t[u][v] = __builtin_nontemporal_load(src + at[v] + (o + kRing + u) * strideVecs);
        }
      }
#pragma unroll
      for (int u = 0; u < kRing; ++u)
#pragma unroll
        for (int v = 0; v < kVecs; ++v)
          add(v, t[u][v]);
      o += kRing;
    }
    for (; o < outer; ++o)
#pragma unroll
      for (int v = 0; v < kVecs; ++v)
        add(v, __builtin_nontemporal_load(src + at[v] + o * strideVecs));
#pragma unroll
    for (int v = 0; v < kVecs; ++v) {
      const int64_t i = i0 + v * (kThreads * kPer);
      if (i < inner)
        static_cast<u32x4 *>(out)[i / kPer] = E::pack(acc[v]);
    }
  }
}

// 16-bit inputs widen to f32, are added in f32 in slice order and rounded once at the end (the
// reference's policy for 16-bit element types on the GPU, docs/Transforms/BF16ToGpu.md:17-26;
// benchmarks/reduce/reduce.dtypes.in lists f32, f16, bf16).
template <io::Dt D>
__device__ __forceinline__ void reduce_outer(const void *in, void *out, int64_t outer, int64_t inner, float init) {
  using E = io::Elem<D>;
  const bool vec = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 &&
                   (inner % E::kPerVec) == 0;
  if (vec) {
    // the widest span that still leaves 512 workgroups (two per CU): 32, 16, 8 or 4 KiB per slice
    const int64_t perVec = int64_t(kThreads) * E::kPerVec;
    if (inner >= 512 * 8 * perVec)
      reduce_outer_vec<D, 8>(in, out, outer, inner, init);
    else if (inner >= 512 * 4 * perVec)
      reduce_outer_vec<D, 4>(in, out, outer, inner, init);
    else if (inner >= 512 * 2 * perVec)
      reduce_outer_vec<D, 2>(in, out, outer, inner, init);
    else
      reduce_outer_vec<D, 1>(in, out, outer, inner, init);
  } else {
    for (int64_t i = int64_t(blockIdx.x) * kThreads + threadIdx.x; i < inner; i += int64_t(gridDim.x) * kThreads) {
      float acc = init;
      for (int64_t o = 0; o < outer; ++o)
        acc = acc + E::get(in, o * inner + i);
      E::put(out, i, acc);
    }
  }
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_reduce_outer_f32(const float *in, float *out,
                                                                            int64_t outer, int64_t inner,
                                                                            float init) {
  reduce_outer<io::Dt::F32>(in, out, outer, inner, init);
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_reduce_outer_f16(const uint16_t *in, uint16_t *out,
                                                                            int64_t outer, int64_t inner,
                                                                            float init) {
  reduce_outer<io::Dt::F16>(in, out, outer, inner, init);
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_reduce_outer_bf16(const uint16_t *in, uint16_t *out,
                                                                             int64_t outer, int64_t inner,
                                                                             float init) {
  reduce_outer<io::Dt::BF16>(in, out, outer, inner, init);
}
