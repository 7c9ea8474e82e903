// Element-wise kernels: ReLU and SiLU (f32 / f16 / bf16), exp and maximum (f32).
//
// Reference op bodies: benchmarks/relu/relu_gpu.mlir.in:3-13 (cmpf ugt + select)
// and benchmarks/silu/silu_gpu.mlir.in:3-19 (negf, exp, addf, divf, then mulf in
// a second pass over a full-size temporary).  Here each is ONE streaming pass:
// 128-bit loads and stores, four of them in flight per lane, HBM-bound.
//
// Kernel arguments follow the IMEX launch convention: one raw base pointer per
// memref, scalars (index = i64) by value.
//
// Launch: block (256,1,1); grid (ceil(n / kElemsPerBlock), 1, 1).

#include "device_common.h"

using namespace imexhip;

namespace {

constexpr int kThreads = 256;

// ---------------------------------------------------------------------------
// Generic streaming driver: Op works on one 16-byte vector (u32x4) and on one
// scalar element (for ragged tails and unaligned bases).
// ---------------------------------------------------------------------------
template <typename Op, int kElemBytes, bool kStream, int kVecsPerThread = 4>
__device__ __forceinline__ void stream_map_impl(const void *__restrict__ in, void *__restrict__ out, int64_t n,
                                                Op op) {
  constexpr int kElemsPerVec = 16 / kElemBytes;
  constexpr int64_t kElemsPerBlock = int64_t(kThreads) * kVecsPerThread * kElemsPerVec;
  const bool aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  // workgroups stride over the blocks, so a grid smaller than ceil(n / kElemsPerBlock) still covers n
  for (int64_t base = int64_t(blockIdx.x) * kElemsPerBlock; base < n; base += int64_t(gridDim.x) * kElemsPerBlock) {
    if (aligned && base + kElemsPerBlock <= n) {
      const u32x4 *src = reinterpret_cast<const u32x4 *>(static_cast<const char *>(in) + base * kElemBytes);
      u32x4 *dst = reinterpret_cast<u32x4 *>(static_cast<char *>(out) + base * kElemBytes);
      u32x4 v[kVecsPerThread];
#pragma unroll
      for (int j = 0; j < kVecsPerThread; ++j)
        v[j] = load128<kStream>(src + j * kThreads + threadIdx.x);
#pragma unroll
      for (int j = 0; j < kVecsPerThread; ++j)
        store128<kStream>(op.vec(v[j]), dst + j * kThreads + threadIdx.x);
    } else {
      for (int64_t i = base + threadIdx.x; i < base + kElemsPerBlock && i < n; i += kThreads)
        op.scalar(in, out, i);
    }
  }
}

// Non-temporal accesses throughout: measured on MI355X they match ordinary
// loads/stores when the tensors are cache-resident and are ~45% faster when
// they are not (no write-back of evicted lines on the critical path).
template <typename Op, int kElemBytes>
__device__ __forceinline__ void stream_map(const void *in, void *out, int64_t n, Op op) {
  stream_map_impl<Op, kElemBytes, true>(in, out, n, op);
}

// Two inputs, one output, all of one shape: Op::one(a, b) on 32-bit elements.
template <typename Op>
__device__ __forceinline__ void stream_map2_b32(const uint32_t *__restrict__ a, const uint32_t *__restrict__ b,
                                                uint32_t *__restrict__ out, int64_t n, Op op) {
  constexpr int kVecsPerThread = 4;
  constexpr int64_t kElemsPerBlock = int64_t(kThreads) * kVecsPerThread * 4;
  const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
                         reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  for (int64_t base = int64_t(blockIdx.x) * kElemsPerBlock; base < n; base += int64_t(gridDim.x) * kElemsPerBlock) {
    if (aligned && base + kElemsPerBlock <= n) {
      const u32x4 *pa = reinterpret_cast<const u32x4 *>(a + base), *pb = reinterpret_cast<const u32x4 *>(b + base);
      u32x4 *po = reinterpret_cast<u32x4 *>(out + base);
      u32x4 va[kVecsPerThread], vb[kVecsPerThread];
#pragma unroll
      for (int j = 0; j < kVecsPerThread; ++j) {
        va[j] = load128<true>(pa + j * kThreads + threadIdx.x);
        vb[j] = load128<true>(pb + j * kThreads + threadIdx.x);
      }
#pragma unroll
      for (int j = 0; j < kVecsPerThread; ++j)
        store128<true>(u32x4{op.one(va[j].x, vb[j].x), op.one(va[j].y, vb[j].y), op.one(va[j].z, vb[j].z),
                             op.one(va[j].w, vb[j].w)},
                       po + j * kThreads + threadIdx.x);
    } else {
      for (int64_t i = base + threadIdx.x; i < base + kElemsPerBlock && i < n; i += kThreads)
        out[i] = op.one(a[i], b[i]);
    }
  }
}

// ---------------------------------------------------------------------------
// arith.maximumf (test/Integration/Dialect/XeGPU/WG/arith_maximumf.mlir:61): the larger operand,
// +0 above -0, and NaN if either operand is NaN (the first NaN operand, quieted).  On the bit
// patterns: a float's order is its sign-magnitude integer order.
// ---------------------------------------------------------------------------
struct MaximumF32 {
  static __device__ __forceinline__ int32_t key(uint32_t u) { // monotone in the float's value, -0 below +0
    return static_cast<int32_t>(u ^ ((static_cast<int32_t>(u) >> 31) & 0x7fffffff));
  }
  __device__ __forceinline__ uint32_t one(uint32_t a, uint32_t b) const {
    const bool nanA = (a & 0x7fffffffu) > 0x7f800000u, nanB = (b & 0x7fffffffu) > 0x7f800000u;
    const uint32_t larger = key(a) >= key(b) ? a : b;
    return nanA ? (a | 0x00400000u) : (nanB ? (b | 0x00400000u) : larger);
  }
};

// ---------------------------------------------------------------------------
// ReLU.  "ugt" = unordered or greater than: x if x > 0 or x is NaN (payload
// kept), else the constant +0.0 (so -0.0 -> +0.0).  Done on the bit patterns,
// which makes the result independent of the FP mode registers.
// ---------------------------------------------------------------------------
struct ReluF32 {
  static __device__ __forceinline__ uint32_t one(uint32_t u) {
    const bool keep = (static_cast<int32_t>(u) > 0) || (u > 0xff800000u);
    return keep ? u : 0u;
  }
  __device__ __forceinline__ u32x4 vec(u32x4 v) const {
    return u32x4{one(v.x), one(v.y), one(v.z), one(v.w)};
  }
  __device__ __forceinline__ void scalar(const void *in, void *out, int64_t i) const {
    static_cast<uint32_t *>(out)[i] = one(static_cast<const uint32_t *>(in)[i]);
  }
};

// 16-bit variants; kNanAbove = magnitude bits of +Inf (0x7c00 f16, 0x7f80 bf16).
template <uint32_t kNanAbove> struct Relu16 {
  static __device__ __forceinline__ uint32_t one(uint32_t h) {
    const uint32_t mag = h & 0x7fffu;
    const bool positive = (h & 0x8000u) == 0 && mag != 0;
    const bool nan = mag > kNanAbove;
    return (positive || nan) ? h : 0u;
  }
  static __device__ __forceinline__ uint32_t pair(uint32_t w) { return one(w & 0xffffu) | (one(w >> 16) << 16); }
  __device__ __forceinline__ u32x4 vec(u32x4 v) const {
    return u32x4{pair(v.x), pair(v.y), pair(v.z), pair(v.w)};
  }
  __device__ __forceinline__ void scalar(const void *in, void *out, int64_t i) const {
    static_cast<uint16_t *>(out)[i] = static_cast<uint16_t>(one(static_cast<const uint16_t *>(in)[i]));
  }
};

// ---------------------------------------------------------------------------
// SiLU, f32, bit-compatible with the reference's CPU lowering: five separately
// rounded f32 operations  t = -x; e = exp(t); d = e + 1; s = 1 / d; y = s * x
// where exp is libm's expf (benchmarks/pipelines/linalg-to-cpu.pp:18-19).
//
// expf_libm restates the algorithm glibc's expf uses (Arm Optimized Routines
// exp2f/expf: reduce x*32/ln2 = k + r, 2^(k/32) from a 32-entry table, cubic in
// r, everything in f64, one final rounding to f32).  Every f64 operation here
// is an IEEE one, so the result equals the host's for every input.
// ---------------------------------------------------------------------------
__device__ const uint64_t kExp2Table[32] = {
    0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,
    0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,
    0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,
    0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,
    0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,
    0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,
    0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,
    0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull};

// The arithmetic of expf for an x libm sends down its main path (|x| < 88, finite).
__device__ __forceinline__ float expf_libm_core(float x, const uint64_t *table) {
  constexpr double kInvLn2N = 0x1.71547652b82fep+0 * 32;
  constexpr double kShift = 0x1.8p+52;
  constexpr double kC0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32;
  constexpr double kC1 = 0x1.ebfce50fac4f3p-3 / 32 / 32;
  constexpr double kC2 = 0x1.62e42ff0c52d6p-1 / 32;
  const double xd = static_cast<double>(x);
  const double z = kInvLn2N * xd;
  double kd = z + kShift;
  const uint64_t ki = __builtin_bit_cast(uint64_t, kd);
  kd -= kShift;
  const double r = z - kd;
  uint64_t t = table[ki & 31u];
  t += ki << (52 - 5);
  const double s = __builtin_bit_cast(double, t);
  const double p = kC0 * r + kC1;
  const double r2 = r * r;
  double y = kC2 * r + 1.0;
  y = p * r2 + y;
  y = y * s;
  return static_cast<float>(y);
}

__device__ __forceinline__ float expf_libm(float x, const uint64_t *table) {
  const float result = expf_libm_core(x, table);
  // |x| >= 88, infinities and NaN: libm branches to these cases before the arithmetic above; here
  // they are selects after it (whatever the arithmetic made of such an x is discarded), which
  // keeps the instruction stream straight -- a taken branch per element costs more than the math.
  const uint32_t ux = f2u(x);
  const uint32_t abstop = (ux >> 20) & 0x7ffu;
  const float big = x > 0x1.62e42ep6f ? __builtin_inff() : (x < -0x1.9fe368p6f ? 0.0f : result);
  const float special = abstop >= 0x7f8u ? (ux == 0xff800000u ? 0.0f : x + x) : big;
  return abstop >= 0x42bu ? special : result;
}

// 1 / d for 1 <= d < 2^100, correctly rounded: the instruction sequence the compiler expands an f32
// division into (reciprocal estimate, two refinements, a final correction), minus the operand scaling
// and the special-case fix-up, neither of which does anything for a denominator in that range.
__device__ __forceinline__ float reciprocal_of_moderate(float d) {
  const float r = __builtin_amdgcn_rcpf(d);
  const float e0 = __builtin_fmaf(-d, r, 1.0f);
  const float r1 = __builtin_fmaf(e0, r, r);
  const float res = __builtin_fmaf(-d, r1, 1.0f);
  const float q1 = __builtin_fmaf(res, r1, r1);
  const float res2 = __builtin_fmaf(-d, q1, 1.0f);
  return __builtin_fmaf(res2, r1, q1);
}

struct SiluF32 {
  const uint64_t *table;
  __device__ __forceinline__ float one(float x) const {
    const float t = -x;
    const float e = expf_libm(t, table);
    const float d = e + 1.0f;
    const float s = 1.0f / d; // correctly rounded IEEE division
    return s * x;
  }
  // |x| < 64: exp(-x) is an ordinary number and so is 1 + exp(-x) < 2^93 -- the same five operations
  // with no special case anywhere, so that the elements of a vector are independent straight-line
  // chains the scheduler can interleave (the general form above costs a masked region per element).
  static __device__ __forceinline__ bool moderate(float x) { return ((f2u(x) >> 20) & 0x7ffu) < 0x428u; }
  __device__ __forceinline__ float one_moderate(float x) const {
    const float e = expf_libm_core(-x, table);
    const float d = e + 1.0f;
    return reciprocal_of_moderate(d) * x;
  }
  __device__ __forceinline__ u32x4 vec(u32x4 v) const {
    const float x0 = u2f(v.x), x1 = u2f(v.y), x2 = u2f(v.z), x3 = u2f(v.w);
    const bool all = moderate(x0) && moderate(x1) && moderate(x2) && moderate(x3);
    if (__builtin_amdgcn_ballot_w64(!all) == 0) // uniform over the wavefront: no lane holds anything unusual
      return u32x4{f2u(one_moderate(x0)), f2u(one_moderate(x1)), f2u(one_moderate(x2)), f2u(one_moderate(x3))};
    return u32x4{f2u(one(x0)), f2u(one(x1)), f2u(one(x2)), f2u(one(x3))};
  }
  __device__ __forceinline__ void scalar(const void *in, void *out, int64_t i) const {
    static_cast<float *>(out)[i] = one(static_cast<const float *>(in)[i]);
  }
};

// math.exp on f32 (test/Integration/Dialect/XeGPU/WG/math_exp.mlir:57): libm's expf, as the CPU
// lowering the reference checks against calls it.  |x| < 64 in every lane: the arithmetic alone.
struct ExpF32 {
  const uint64_t *table;
  __device__ __forceinline__ u32x4 vec(u32x4 v) const {
    const float x0 = u2f(v.x), x1 = u2f(v.y), x2 = u2f(v.z), x3 = u2f(v.w);
    const bool all = SiluF32::moderate(x0) && SiluF32::moderate(x1) && SiluF32::moderate(x2) && SiluF32::moderate(x3);
    if (__builtin_amdgcn_ballot_w64(!all) == 0)
      return u32x4{f2u(expf_libm_core(x0, table)), f2u(expf_libm_core(x1, table)), f2u(expf_libm_core(x2, table)),
                   f2u(expf_libm_core(x3, table))};
    return u32x4{f2u(expf_libm(x0, table)), f2u(expf_libm(x1, table)), f2u(expf_libm(x2, table)),
                 f2u(expf_libm(x3, table))};
  }
  __device__ __forceinline__ void scalar(const void *in, void *out, int64_t i) const {
    static_cast<float *>(out)[i] = expf_libm(static_cast<const float *>(in)[i], table);
  }
};

// 16-bit SiLU: widen to f32, the same five f32 operations, one rounding back to the 16-bit type
// (the policy the reference applies to 16-bit element types on the GPU,
// docs/Transforms/BF16ToGpu.md:17-26; benchmarks/silu/silu.dtypes.in lists f16).
//
// A 16-bit type has 65536 inputs, so what the f32 chain must deliver is the right 16-bit result for each
// of them, not a correctly rounded f32 value in between -- and that can be checked for every input.  The
// vector path therefore evaluates x * rcp(1 + exp2(-x * log2(e))) with the hardware's exponential and
// reciprocal estimates (an ulp or two of f32 each, fixed functions of their input on this part):
//   f16:  the same bits as the libm-exact chain for every one of the 65536 input patterns, NaN and
//         infinities included, so there is no other case;
//   bf16: with one Newton step on the reciprocal the same bits for every |x| < 64; beyond that
//         (exp(-x) near the f32 overflow threshold gives denormal results) the exact chain runs, chosen
//         once per wavefront and vector like the f32 kernel's general form.
// A GPU test compares every input pattern of both types with the CPU restatement, so a part or a compiler
// whose estimates differ cannot go unnoticed.  The exact chain (twelve f64 operations per element) is about
// 45 vector operations per element where four bytes of traffic leave time for about 24; this form is 8
// ordinary and 2 quarter-rate ones, and the kernel is memory-bound like ReLU.
template <io::Dt D> struct Silu16 {
  using E = io::Elem<D>;
  SiluF32 f32;
  static __device__ __forceinline__ float estimate(float x) {
    constexpr float kMinusLog2e = -1.44269504088896340736f;
    const float e = __builtin_amdgcn_exp2f(x * kMinusLog2e);
    const float d = 1.0f + e;
    float r = __builtin_amdgcn_rcpf(d);
    if constexpr (D == io::Dt::BF16)
      r = __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
    return x * r;
  }
  __device__ __forceinline__ u32x4 vec(u32x4 v) const {
    float f[E::kPerVec];
    E::unpack(v, f);
    if constexpr (D == io::Dt::F16) {
#pragma unroll
      for (int i = 0; i < E::kPerVec; ++i)
        f[i] = estimate(f[i]);
    } else {
      bool all = true;
#pragma unroll
      for (int i = 0; i < E::kPerVec; ++i)
        all = all && SiluF32::moderate(f[i]);
      if (__builtin_amdgcn_ballot_w64(!all) == 0) {
#pragma unroll
        for (int i = 0; i < E::kPerVec; ++i)
          f[i] = estimate(f[i]);
      } else {
#pragma unroll
        for (int i = 0; i < E::kPerVec; ++i)
          f[i] = f32.one(f[i]);
      }
    }
    return E::pack(f);
  }
  __device__ __forceinline__ void scalar(const void *in, void *out, int64_t i) const {
    E::put(out, i, f32.one(E::get(in, i)));
  }
};

// SiLU / exp launch body: the 32-entry table staged in LDS (the index is data-dependent, and LDS serves
// 64 different addresses per access where a constant load would not); below 4 Mi elements a lane's
// exponentials and divisions are the critical path, so one vector per lane and pass instead of four.
template <typename Op, int kElemBytes, typename Make>
__device__ __forceinline__ void silu_launch(const void *in, void *out, int64_t n, Make make) {
  __shared__ uint64_t table[32];
  if (threadIdx.x < 32)
    table[threadIdx.x] = kExp2Table[threadIdx.x];
  __syncthreads();
  if (n < (int64_t(1) << 22))
    stream_map_impl<Op, kElemBytes, true, 1>(in, out, n, make(table));
  else
    stream_map<Op, kElemBytes>(in, out, n, make(table));
}

} // namespace

extern "C" __global__ __launch_bounds__(kThreads) void imex_relu_f32(const float *in, float *out, int64_t n) {
  stream_map<ReluF32, 4>(in, out, n, ReluF32{});
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_relu_f16(const uint16_t *in, uint16_t *out,
                                                                    int64_t n) {
  stream_map<Relu16<0x7c00u>, 2>(in, out, n, Relu16<0x7c00u>{});
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_relu_bf16(const uint16_t *in, uint16_t *out,
                                                                     int64_t n) {
  stream_map<Relu16<0x7f80u>, 2>(in, out, n, Relu16<0x7f80u>{});
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_silu_f32(const float *in, float *out, int64_t n) {
  silu_launch<SiluF32, 4>(in, out, n, [](const uint64_t *table) { return SiluF32{table}; });
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_exp_f32(const float *in, float *out, int64_t n) {
  silu_launch<ExpF32, 4>(in, out, n, [](const uint64_t *table) { return ExpF32{table}; });
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_maximum_f32(const uint32_t *a, const uint32_t *b,
                                                                       uint32_t *out, int64_t n) {
  stream_map2_b32(a, b, out, n, MaximumF32{});
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_silu_f16(const uint16_t *in, uint16_t *out,
                                                                    int64_t n) {
  silu_launch<Silu16<io::Dt::F16>, 2>(in, out, n, [](const uint64_t *table) { return Silu16<io::Dt::F16>{SiluF32{table}}; });
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_silu_bf16(const uint16_t *in, uint16_t *out,
                                                                     int64_t n) {
  silu_launch<Silu16<io::Dt::BF16>, 2>(in, out, n, [](const uint64_t *table) { return Silu16<io::Dt::BF16>{SiluF32{table}}; });
}
