// Shared device helpers for the gfx950 kernels: 128-bit vector types, bit
// casts, wavefront-64 reductions and 16-bit float conversions.
#ifndef IMEX_HIP_DEVICE_COMMON_H
#define IMEX_HIP_DEVICE_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace imexhip {

constexpr int kWave = 64;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }

// f16 / bf16 bits -> f32 (exact) and f32 -> 16-bit with round-to-nearest-even.
__device__ __forceinline__ float half_bits_to_float(uint32_t h16) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h16)));
}
__device__ __forceinline__ uint32_t float_to_half_bits(float f) {
  // The empty asm keeps the conversion a conversion.  Left to itself the compiler folds a
  // multiplication that feeds it into v_fma_mixlo_f16 a, b, 0 -- and (-0) + (+0) is +0, so a
  // product that is exactly -0.0 (SiLU of a large negative input: 0 * x) would lose its sign.
  asm volatile("" : "+v"(f));
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}
__device__ __forceinline__ float bf16_bits_to_float(uint32_t b16) { return u2f(b16 << 16); }
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u)
    return (u & 0x80000000u) ? 0xffc0u : 0x7fc0u;
  u += ((u >> 16) & 1u) + 0x7fffu;
  return u >> 16;
}

// Cache policy helpers.  MI355X has 256 MiB of Infinity Cache behind the L2s.
// Every kernel here touches each byte once, so the streaming kernels and the
// transposes use non-temporal accesses: measured on tensors that are not already
// cache-resident (buffers rotated through 2 GiB, or after a cache flush), that is
// the faster policy everywhere.  Ordinary accesses only win when one and the same
// buffer pair, small enough for the Infinity Cache, is processed again and again.
template <bool kStream> __device__ __forceinline__ u32x4 load128(const u32x4 *p) {
  if constexpr (kStream)
    return __builtin_nontemporal_load(p);
  else
    return *p;
}
template <bool kStream> __device__ __forceinline__ void store128(u32x4 v, u32x4 *p) {
  if constexpr (kStream)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}

// Reductions across the 64 lanes of a wavefront, every lane active, on the VALU's own
// cross-lane paths (DPP): four steps inside each row of 16 lanes (quad swaps, half-row and row
// mirrors: afterwards every lane holds its row's result), two row broadcasts (rows 1 and 3 take
// lane 15 of the row before, rows 2 and 3 take lane 31; the row mask leaves the other rows as they
// are), and lane 63 read out as a wavefront-uniform value.  Seven instructions and no LDS round
// trip; the xor-shuffle form costs six dependent ds_bpermute.  Written as instructions: from the
// builtins the compiler made a copy, a canonicalising maximum and the maximum itself out of every
// step.  A DPP operand must not be read for two wait states after a VALU wrote it, hence the
// s_nop before each step (the compiler cannot see hazards inside an asm block); the trailing one
// covers whatever reads the result next.
#define IMEX_DPP_REDUCE(op)                                                                                   \
  "s_nop 1\n\t" op " %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"                            \
  "s_nop 1\n\t" op " %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"                            \
  "s_nop 1\n\t" op " %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"                                \
  "s_nop 1\n\t" op " %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"                                     \
  "s_nop 1\n\t" op " %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"                                   \
  "s_nop 1\n\t" op " %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"                                   \
  "s_nop 1"
__device__ __forceinline__ float wave_sum(float v) {
  asm volatile(IMEX_DPP_REDUCE("v_add_f32_dpp") : "+v"(v));
  return u2f(__builtin_amdgcn_readlane(f2u(v), 63));
}
// NaN operands are passed over (v_max_f32 returns the other operand), like fmaxf.
__device__ __forceinline__ float wave_max(float v) {
  asm volatile(IMEX_DPP_REDUCE("v_max_f32_dpp") : "+v"(v));
  return u2f(__builtin_amdgcn_readlane(f2u(v), 63));
}
#undef IMEX_DPP_REDUCE

// Element traits for kernels that exist in f32, f16 and bf16 forms: scalar get / put through
// f32, and a 16-byte vector (u32x4) unpacked to / packed from kPerVec f32 values.  16-bit values
// widen exactly and narrow with round-to-nearest-even.  (In a namespace of their own: kernels with
// different needs keep local traits.)
namespace io {
enum class Dt { F32, F16, BF16 };
template <Dt D> struct Elem;
template <> struct Elem<Dt::F32> {
  static constexpr int kBytes = 4, kPerVec = 4;
  static __device__ __forceinline__ float get(const void *p, int64_t i) { return static_cast<const float *>(p)[i]; }
  static __device__ __forceinline__ void put(void *p, int64_t i, float v) { static_cast<float *>(p)[i] = v; }
  static __device__ __forceinline__ void unpack(u32x4 v, float *f) {
    f[0] = u2f(v.x); f[1] = u2f(v.y); f[2] = u2f(v.z); f[3] = u2f(v.w);
  }
  static __device__ __forceinline__ u32x4 pack(const float *f) { return u32x4{f2u(f[0]), f2u(f[1]), f2u(f[2]), f2u(f[3])}; }
};
template <bool kBf> struct Elem16 {
  static constexpr int kBytes = 2, kPerVec = 8;
  static __device__ __forceinline__ float widen(uint32_t h) { return kBf ? bf16_bits_to_float(h) : half_bits_to_float(h); }
  static __device__ __forceinline__ uint32_t narrow(float f) { return kBf ? float_to_bf16_bits(f) : float_to_half_bits(f); }
  static __device__ __forceinline__ float get(const void *p, int64_t i) { return widen(static_cast<const uint16_t *>(p)[i]); }
  static __device__ __forceinline__ void put(void *p, int64_t i, float v) {
    static_cast<uint16_t *>(p)[i] = static_cast<uint16_t>(narrow(v));
  }
  static __device__ __forceinline__ void unpack(u32x4 v, float *f) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = widen(w[i] & 0xffffu);
      f[2 * i + 1] = widen(w[i] >> 16);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float *f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = narrow(f[2 * i]) | (narrow(f[2 * i + 1]) << 16);
    return u32x4{w[0], w[1], w[2], w[3]};
  }
};
template <> struct Elem<Dt::F16> : Elem16<false> {};
template <> struct Elem<Dt::BF16> : Elem16<true> {};
} // namespace io

} // namespace imexhip
#endif
