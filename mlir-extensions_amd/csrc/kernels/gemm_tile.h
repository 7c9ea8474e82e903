// The tile code of the MFMA GEMM for gfx950 (entry points: gemm.hip; timing probes: probe.hip):
// C[M,N] = A[M,K] . B[K,N], A and B f16 or bf16
// (row-major), f32 accumulate; also with A stored [K,M] or B stored [N,K].
//
// Reference kernels (workgroup-level XeGPU, the role XeTile's
// load_tile / prefetch_tile / tile_mma played):
//   test/Integration/Dialect/XeGPU/WG/gemm_4kx4kx4k_f16_f16_f32.mlir:47-91
//     256x256 workgroup tile, K-step 32, three-deep prefetch, C += A.B;
//   test/Integration/Dialect/XeGPU/WG/gemm_4kx4kx4k_f16_f16_f32_bias.mlir:77-116
//     bias[n] broadcast over rows and added after the K loop;
//   benchmarks/silu/silu_gpu.mlir.in:3-19 for the activation fused below;
//   test/Integration/Dialect/XeGPU/WG/gemm_4kx4kx4k_transpose_{a,b}.mlir for the
//     operand storage orders (the same kernel with the other operand loader).
//
// Blocking on MI355X:
//   workgroup tile 256 x 256, 512 threads = 8 wavefronts in a 2 x 4 grid (two per
//   SIMD), each owning 128 x 64 = 8 x 4 MFMA 16x16x32 blocks (128 accumulator
//   registers).  16x16x32 rather than 32x32x16: the two read the same LDS bytes per
//   FLOP, but on random operands the part sustains about 9 % more with the former
//   (the shader clock under MFMA load follows the operand values);
//   K advances 32 at a time; each operand has a ring of four 16 KiB LDS stages,
//   except that A [M,K] with K % 64 == 0 is copied as slabs of 64 k (128-byte rows:
//   one L2 request per cache line where 32-k slabs make 64-byte requests) into a
//   ring of three 32 KiB stages, half a slab with each of the two steps it covers
//   (160 KiB of LDS in all).  A and B tiles go from global memory STRAIGHT into
//   LDS (buffer_load ... lds, 16 bytes per lane, no register staging) three steps
//   ahead of the step that multiplies them; a step waits (vmcnt) only for the
//   oldest tile in flight, then meets the other wavefronts at the step's single
//   barrier;
//   the LDS images are swizzled -- A [256 rows][32 k] by 16-byte group, B
//   [32 k][256 n] by 32-byte pair -- and because a direct copy fixes each lane's
//   LDS position, the swizzle is applied to the lane's GLOBAL address instead;
//   A fragments are 128-bit LDS reads; B is row-major [K,N] while the MFMA wants
//   eight consecutive k per lane, so B fragments use the LDS transpose read
//   (ds_read_b64_tr_b16) -- no permutes, no transposed copy of B anywhere;
//   a K-step is multiplied in two halves of 16 MFMAs (the wavefront's upper, then
//   lower four row blocks, each by all four column blocks); fragments are
//   double-buffered in registers: the LDS reads the next half needs are placed by
//   hand between the MFMAs of this one (sched_barrier fences keep the order), and
//   the step's barrier sits between the halves so that sixteen MFMAs are always
//   queued behind it;
//   f32 results: the accumulator blocks of two neighbouring column blocks swap
//   16-lane rows (v_permlane16_swap) so that every store instruction writes whole
//   128-byte lines; 16-bit results: the product is taken transposed, which leaves
//   four consecutive columns in a lane's registers -- one 8-byte store;
//   workgroup ids are remapped so that the 32 workgroups resident on one XCD
//   (ids congruent mod 8) cover a compact 4 x 8 block of tiles and share A and
//   B panels in that XCD's L2.
//
// M and N need not divide the tile: edge tiles copy the last row / column that exists
// in place of the missing ones and store only what is inside C.  What the MFMA path
// does need is 16-byte aligned rows in memory (K % 8 == 0; N % 8 == 0
// where B is [K,N], M % 8 == 0 where A is [K,M]; a K that does not fill the last 32-wide step is
// padded with zeros on the way into LDS); other shapes take the vector-ALU path of the
// same kernels (128 x 128 tiles, gemm_blocked), which adds in ascending k like the
// reference's CPU loop (lib/ExecutionEngine/ImexRunnerUtils.cpp:308-317).
//
// Launch: block (512,1,1); grid (tiles,1,1) with tiles = ceil(M/256)*ceil(N/256) on
// the MFMA path, else (ceil(M/128)*ceil(N/128),1,1); workgroups stride, so any grid is correct.  The fixed-shape 4096^3 entry
// points take the reference's own launch: blocks (16,16,1), threads (512,1,1).

#ifndef IMEX_HIP_GEMM_TILE_H
#define IMEX_HIP_GEMM_TILE_H

#include "device_common.h"

namespace imexhip_gemm {
using namespace imexhip;

// Timing probes (bench-only code object, never the operators): parts of the tile code switched off
// to price them.  Results are then meaningless; the instruction stream that remains is the operator's.
enum : int {
  kProbeNoLoopCopies = 1, // no global -> LDS copies inside the K loop (the prologue fills all four ring stages once)
  kProbeNoEpilogue = 2,   // accumulators kept alive but not stored
  kProbeCopiesOnly = 4,   // no LDS fragment reads and no MFMAs: the copy pipeline and its barriers alone
  kProbeNoCopyA = 8,      // A's slabs are not copied
  kProbeNoCopyB = 16,     // B's slabs are not copied
};

// Wavefront grid inside the 256 x 256 workgroup tile: 2 x 4, each wavefront 128 x 64.
constexpr int kWavesM = 2, kWavesN = 4;
constexpr int kWaves = kWavesM * kWavesN;
constexpr int kThreads = 64 * kWaves;
constexpr int BM = 256, BN = 256;
constexpr int RK = 32;                              // K per step (one ring stage)
constexpr int WM = BM / kWavesM, WN = BN / kWavesN; // wavefront tile
constexpr int FI = WM / 16, FJ = WN / 16;           // MFMA 16x16 tiles per wavefront: 8 x 4
constexpr int kStages = 4;                          // LDS ring: 4 x 32 KiB of the 160 KiB
constexpr int kImageBytes = 256 * RK * 2;           // one operand's 256 x 32 slab: 16 KiB
constexpr int kDmaPerWave = kImageBytes / 1024 / kWaves; // 1 KiB global->LDS copies per wavefront, operand and step
constexpr int kDist = kStages - 1;                  // tiles in flight ahead of the one being multiplied
constexpr int kRingBytes = kStages * kImageBytes;   // one operand's ring of four slabs: 64 KiB; B's ring first, then A's
constexpr int kWideStages = 3;                      // A as 64-k-wide slabs (2 x 16 KiB each): a ring of three
constexpr int kWideBytes = 2 * kImageBytes;
constexpr int kLdsBytes = kRingBytes + kWideStages * kWideBytes; // 160 KiB: all of a CU's LDS
constexpr int kGroupM = 4;                          // tile rows per L2-sharing group

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4u __attribute__((ext_vector_type(4), aligned(4)));   // 4 floats at any float address
typedef uint16_t u16x4u __attribute__((ext_vector_type(4), aligned(2))); // 4 halves at any half address
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4 LdsI16x4; // operand type of the LDS transpose read
typedef __attribute__((address_space(3))) char LdsChar;

struct F16 {
  using Frag = f16x8;
  static __device__ __forceinline__ f32x4 mfma(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float widen(uint16_t h) { return half_bits_to_float(h); }
};
struct BF16 {
  using Frag = bf16x8;
  static __device__ __forceinline__ f32x4 mfma(Frag a, Frag b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float widen(uint16_t h) { return bf16_bits_to_float(h); }
};

// Keeps the compiler's scheduler from moving anything across this point.
#define IMEX_FENCE() __builtin_amdgcn_sched_barrier(0)

// ---- epilogues ------------------------------------------------------------------
// operator() takes one element of the accumulator.  kColumnsInRegisters picks how the tiled
// path holds the accumulator: true = four consecutive columns of one row in a lane's four
// registers, handed to vec4() (16-bit outputs: one 8-byte store per lane); false = one column
// per lane, rows in the registers, stored element by element after the lane-row swap that
// lines 32 consecutive columns up across lanes (32-bit outputs: whole 128-byte lines).
struct StoreF32 {       // C = acc
  static constexpr bool kColumnsInRegisters = false;
  float *C;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    C[m * N + n] = acc; // ordinary store: C stays in the last-level cache for whoever reads it next
  }
};
// Epilogues that read C first also offer the two halves separately -- fetch() the old value, put() the new one
// computed from it -- so that the tiled path can issue a whole batch of reads before the first dependent store
// (element by element, every read would wait for the store before it: C may alias itself).
struct AccumulateF32 {  // C = C + acc   (the reference kernel loads C as its initial accumulator)
  static constexpr bool kColumnsInRegisters = false;
  static constexpr bool kReadsC = true;
  float *C;
  __device__ __forceinline__ float fetch(int64_t m, int64_t n, int64_t N) const { return C[m * N + n]; }
  __device__ __forceinline__ void put(int64_t m, int64_t n, int64_t N, float acc, float old) const {
    C[m * N + n] = old + acc;
  }
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    put(m, n, N, acc, fetch(m, n, N));
  }
};
struct BiasAccumulateF32 { // C = bias[n] + (C + acc)  (bias.mlir:88-94,112-113)
  static constexpr bool kColumnsInRegisters = false;
  static constexpr bool kReadsC = true;
  float *C;
  const float *bias;
  __device__ __forceinline__ float fetch(int64_t m, int64_t n, int64_t N) const { return C[m * N + n]; }
  __device__ __forceinline__ void put(int64_t m, int64_t n, int64_t N, float acc, float old) const {
    C[m * N + n] = bias[n] + (old + acc);
  }
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    put(m, n, N, acc, fetch(m, n, N));
  }
};
// f32 results stored 16 bytes per lane from the transposed accumulator (row lane % 16, four consecutive
// columns): before the stores the upper half-rows (lanes 8-15 of every 16) of column block j trade places
// with the lower half-rows of block j + 1, after which a lane of block j's registers holds row lane % 8 of
// block j + (lane % 16) / 8 -- a store instruction then covers eight rows by 128 bytes, whole lines, with a
// quarter of the store instructions of the element-per-lane form.
struct StoreF32Lines {
  static constexpr bool kColumnsInRegisters = true;
  static constexpr bool kHalfRowExchange = true;
  float *C;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const { C[m * N + n] = acc; }
  __device__ __forceinline__ void vec4(int64_t m, int64_t n, int64_t N, f32x4 acc) const {
    *reinterpret_cast<f32x4 *>(C + m * N + n) = acc;
  }
};
template <typename Epi, typename = void> struct ExchangesHalfRows { static constexpr bool value = false; };
template <typename Epi> struct ExchangesHalfRows<Epi, decltype(void(Epi::kHalfRowExchange))> {
  static constexpr bool value = Epi::kHalfRowExchange;
};
template <typename Epi, typename = void> struct ReadsC { static constexpr bool value = false; };
template <typename Epi> struct ReadsC<Epi, decltype(void(Epi::kReadsC))> { static constexpr bool value = Epi::kReadsC; };
// v / (1 + exp(-v)) with the hardware's exponential and reciprocal estimates (about an ulp each):
// the result is rounded to bf16, 2^-9 relative, straight afterwards.
__device__ __forceinline__ float silu_fast(float v) { return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v)); }

// f32 -> bf16 by the hardware's conversion (round to nearest even; pairs become one v_cvt_pk_bf16_f32).
// Numbers convert as float_to_bf16_bits does; a NaN keeps its leading payload bits instead of becoming
// the canonical one.
__device__ __forceinline__ uint16_t bf16_bits_hw(float f) { return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f)); }

struct BiasSiluBF16 {   // out = bf16( silu( acc + bias[n] ) )
  static constexpr bool kColumnsInRegisters = true;
  uint16_t *out;
  const float *bias;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    const float v = acc + bias[n];
    const float y = silu_fast(v);
    out[m * N + n] = bf16_bits_hw(y);
  }
  __device__ __forceinline__ void vec4(int64_t m, int64_t n, int64_t N, f32x4 acc) const {
    const f32x4 b = *reinterpret_cast<const f32x4u *>(bias + n);
    u16x4u o;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float v = acc[r] + b[r];
      const float y = silu_fast(v);
      o[r] = bf16_bits_hw(y);
    }
    *reinterpret_cast<u16x4u *>(out + m * N + n) = o;
  }
};
struct StoreF16 {       // C(f16) = acc   (WG/gemm_4kx4kx4k_f16_f16_f16.mlir)
  static constexpr bool kColumnsInRegisters = true;
  uint16_t *C;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    C[m * N + n] = static_cast<uint16_t>(float_to_half_bits(acc));
  }
  __device__ __forceinline__ void vec4(int64_t m, int64_t n, int64_t N, f32x4 acc) const {
    u16x4u o;
#pragma unroll
    for (int r = 0; r < 4; ++r)
      o[r] = static_cast<uint16_t>(float_to_half_bits(acc[r]));
    *reinterpret_cast<u16x4u *>(C + m * N + n) = o;
  }
};

// ---- any-shape path: 128 x 128 tiles on the vector ALUs -----------------------------------
// For operands the MFMA path cannot take (rows that are not 16-byte aligned in memory).  Every output is
// the reference's CPU loop (lib/ExecutionEngine/ImexRunnerUtils.cpp:308-317): acc = 0, then for ascending
// k a rounded multiply and a rounded add (this file is built with contraction off), so the result is the
// oracle's bit for bit; the tiling only shares the operand loads.  512 lanes hold 8 x 4 outputs each; A
// and B go through LDS sixteen k at a time, widened to f32, zero beyond M, N and K (a zero product leaves
// the sum as it is: the sum starts at +0.0 and never becomes -0.0).
// kAT: A is stored [K,M] (A[k*M+m]) instead of [M,K]; kBT: B is stored [N,K] (B[n*K+k]) instead of [K,N].
template <typename T, bool kAT, bool kBT, typename Epi>
__device__ __forceinline__ void gemm_blocked(const uint16_t *A, const uint16_t *B, int64_t M, int64_t N, int64_t K,
                                             Epi epi, char *ldsBytes) {
  constexpr int TM = 128, TN = 128, TK = 16, kPitch = TM + 4; // the pad keeps a k-fastest fill off one bank
  float(*As)[kPitch] = reinterpret_cast<float(*)[kPitch]>(ldsBytes);
  float(*Bs)[kPitch] = reinterpret_cast<float(*)[kPitch]>(ldsBytes + TK * kPitch * sizeof(float));
  const int tid = threadIdx.x, tx = tid & 31, ty = tid >> 5; // columns 4 tx .., rows 8 ty ..
  const int64_t tilesN = (N + TN - 1) / TN, tiles = ((M + TM - 1) / TM) * tilesN;
  const int64_t workgroups = int64_t(gridDim.x) * gridDim.y;
  for (int64_t id = int64_t(blockIdx.y) * gridDim.x + blockIdx.x; id < tiles; id += workgroups) {
    const int64_t m0 = (id / tilesN) * TM, n0 = (id % tilesN) * TN;
    float acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = 0.0f;
    for (int64_t k0 = 0; k0 < K; k0 += TK) {
      __syncthreads(); // the previous k block has been read
#pragma unroll
      for (int u = 0; u < TM * TK / kThreads; ++u) {
        const int e = u * kThreads + tid;
        // the index that is contiguous in memory varies fastest over the lanes
        const int am = kAT ? e % TM : e / TK, ak = kAT ? e / TM : e % TK;
        const int64_t m = m0 + am, k = k0 + ak;
        As[ak][am] = m < M && k < K ? T::widen(kAT ? A[k * M + m] : A[m * K + k]) : 0.0f;
        const int bn = kBT ? e / TK : e % TN, bk = kBT ? e % TK : e / TN;
        const int64_t n = n0 + bn, kb = k0 + bk;
        Bs[bk][bn] = n < N && kb < K ? T::widen(kBT ? B[n * K + kb] : B[kb * N + n]) : 0.0f;
      }
      __syncthreads();
#pragma unroll
      for (int k = 0; k < TK; ++k) {
        float a[8], b[4];
#pragma unroll
        for (int i = 0; i < 8; ++i)
          a[i] = As[k][ty * 8 + i];
#pragma unroll
        for (int j = 0; j < 4; ++j)
          b[j] = Bs[k][tx * 4 + j];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float p = a[i] * b[j];
            acc[i][j] = acc[i][j] + p; // rounded multiply, rounded add
          }
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t m = m0 + ty * 8 + i, n = n0 + tx * 4 + j;
        if (m < M && n < N)
          epi(m, n, N, acc[i][j]);
      }
  }
}

// ---- tiled MFMA path ----------------------------------------------------------------
// Buffer resource for raw buffer loads: base pointer, byte range, and the gfx9
// "32-bit data format" word; out-of-range lanes read zeros.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, int64_t bytes) {
  const int range = bytes > 0x7fffffff ? 0x7fffffff : int(bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, range, 0x00020000);
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}

// One MFMA operand of a workgroup tile: a 256 x 32 (rows x k) slab per step.  Both
// A (rows = m) and B (rows = n) want, per lane, row = lane % 16 of a 16-row
// fragment and the 8 consecutive k starting at (lane / 16) * 8.
//
// KContig: the slab is k-contiguous in memory (A as [M,K], B as [N,K]).  LDS image
//   [256 rows][32 k], 64-byte rows; 16-byte group c of row r is stored at group
//   c ^ h((r >> 2) & 3), h = {0, 2, 3, 1}.  A fragment is one ds_read_b128 (lane: row
//   lane % 16, group lane / 16); the LDS serves such a read 16 lanes at a time, and the
//   lanes that go together are not neighbours (0-3 with 12-15, 20-23 and 24-27; 4-7 with
//   8-11, 16-19 and 28-31; likewise in the upper half) -- h is chosen so that each of
//   those sets touches every bank once.  One 1 KiB copy = 16 rows.
// KStrided: the slab's rows are strided in memory (B as [K,N], A as [K,M]).  LDS
//   image [32 k][256 rows], 512-byte rows; 32-byte pair p of k-row r at pair
//   p ^ g(r), g(r) = (r & 3) | ((r >> 3 & 1) << 2).  One copy = 2 k-rows.  A
//   fragment is two LDS transpose reads (ds_read_b64_tr_b16): within each group of
//   16 lanes, lane t supplies the address of 4 consecutive rows at k-row t/4 and
//   receives 4 consecutive k of row t.
// A direct global->LDS copy puts lane l's 16 bytes at base + 16 l, so the swizzle
// is applied to the lane's GLOBAL address instead.
__device__ __forceinline__ int kcontig_swizzle(int row) { return (0x78 >> (((row >> 2) & 3) * 2)) & 3; }

// kTail: K is not a multiple of the 32-wide step; the copies of the last step then use a second set of
// offsets in which every 16-byte piece that lies at k >= K is sent out of the buffer's range -- such a
// lane fetches nothing and its 16 bytes of LDS are written with zeros, so the step multiplies zeros
// there.  (An offset beyond the range, not a skipped lane: the LDS image must not keep stale values.)
constexpr int kOutOfRange = 0x7ffffff0;

template <typename T, bool kStrided, int kFrags, bool kTail> struct Operand {
  __amdgpu_buffer_rsrc_t rsrc;
  int voff[kDmaPerWave];         // per-lane byte offset of each copy at step 0
  int voffTail[kTail ? kDmaPerWave : 1]; // the same for the last, partial step
  int step;                      // bytes per K-step in memory
  int dstWave;                   // LDS byte offset of this wavefront's copies inside the image
  int rd[kStrided ? kFrags : 1]; // per-lane LDS read bases: KStrided one per fragment, KContig one (fragments 1 KiB apart)

  // ptr: the operand's matrix; ld: its leading dimension; first: first row (m0 or n0)
  // of the slab; w0: the wavefront's first row inside the slab; extent: rows * cols.
  // A slab that sticks out of the matrix (last tile row / column of a ragged shape): the
  // lanes that would copy rows past the end copy the last row that exists instead, so no
  // address ever leaves the matrix; those rows only feed outputs that are never stored.
  // kRem: the k the last step still holds (8 .. 32; 32 unless kTail)
  __device__ __forceinline__ void setup(const uint16_t *ptr, int64_t ld, int64_t first, int w0, int64_t extent,
                                        int wave, int lane, int kRem) {
    if constexpr (!kStrided) {
      const int64_t rows = extent / ld - first; // rows of the matrix from `first` on, >= 1
      const int last = rows < 256 ? int(rows) - 1 : 255;
      rsrc = make_rsrc(ptr + first * ld, int64_t(last + 1) * ld * 2);
#pragma unroll
      for (int q = 0; q < kDmaPerWave; ++q) {
        const int row = wave * (256 / kWaves) + q * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ kcontig_swizzle(row);
        voff[q] = int((int64_t(min(row, last)) * ld + chunk * 8) * 2);
        if constexpr (kTail)
          voffTail[q] = chunk * 8 < kRem ? voff[q] : kOutOfRange;
      }
      step = RK * 2;
      dstWave = wave * (256 / kWaves) * (RK * 2);
      const int fragRow = lane & 15, kGroup = lane >> 4;
      rd[0] = (w0 + fragRow) * (RK * 2) + ((kGroup ^ kcontig_swizzle(fragRow)) << 4);
    } else {
      rsrc = make_rsrc(ptr + first, (extent - first) * 2);
#pragma unroll
      for (int q = 0; q < kDmaPerWave; ++q) {
        const int row = wave * (RK / kWaves) + q * 2 + (lane >> 5);
        const int g = (row & 3) | (((row >> 3) & 1) << 2);
        const int chunk = (((((lane & 31) >> 1) ^ g)) << 1) | (lane & 1);
        const int64_t col = min(int64_t(chunk * 8), ld - 8 - first); // ld % 8 == 0: the last 16 bytes of the k-row
        voff[q] = int((int64_t(row) * ld + col) * 2);
        if constexpr (kTail)
          voffTail[q] = row < kRem ? voff[q] : kOutOfRange;
      }
      step = int(RK * ld * 2);
      dstWave = wave * (RK / kWaves) * 512;
      const int t = lane & 15, kGroup = lane >> 4;
      const int g = (t >> 2) | ((kGroup & 1) << 2); // g(k-row) for k-row = kGroup*8 + h*4 + t/4
      const int pair0 = w0 / 16;                    // 32-byte pair holding fragment 0's rows
#pragma unroll
      for (int f = 0; f < kFrags; ++f)
        rd[f] = (kGroup * 8 + (t >> 2)) * 512 + (((pair0 + f) ^ g) * 32) + (t & 3) * 8;
    }
  }
  // the wavefront's copies of K-step kt into the image at LDS byte offset `image`; partial: kt is the
  // last step of a K that does not fill it (uniform over the wavefront)
  __device__ __forceinline__ void dma(LdsChar *lds, int image, int kt, bool partial) const {
#pragma unroll
    for (int q = 0; q < kDmaPerWave; ++q) {
      int v = voff[q];
      if constexpr (kTail)
        v = partial ? voffTail[q] : v;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, lds + image + dstWave + q * 1024, 16, v, kt * step, 0, 0);
    }
  }
  // fragment f (rows w0 + 16 f ..., all 32 k) of the image at `image`
  __device__ __forceinline__ typename T::Frag read(const char *lds, int image, int f) const {
    if constexpr (!kStrided) {
      return *reinterpret_cast<const typename T::Frag *>(lds + image + rd[0] + f * 16 * (RK * 2));
    } else {
      const char *p = lds + image + rd[f];
      const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsI16x4 *)(p));           // k +0..3
      const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsI16x4 *)(p + 4 * 512)); // k +4..7
      return __builtin_bit_cast(typename T::Frag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
  }
};

// A k-contiguous operand ([M,K] A) as 64-k-wide slabs: a row of the slab is 128 bytes, one whole L2 line
// and ONE request to the L2 (the 32-k slab's 64-byte rows go out as twice as many half-line requests --
// measured: A-only copies 33 us against 26 us for B's 512-byte rows, same bytes).  A slab serves two
// K-steps and is copied over two steps -- the first 16 of a wavefront's 32 rows at the even step, the
// rest at the odd one, so every step issues two A and two B copies per wavefront like the 32-k form --
// into a ring of three.  LDS image [256 rows][64 k]; 16-byte group c of row r at c ^ ((r >> 1) & 7), which
// keeps the fragment reads (row lane % 16, group 4 p + lane / 16 in the step of parity p) off each
// other's banks for the lanes the LDS serves together.  One 1 KiB copy = 8 rows.
template <typename T, int kFrags> struct OperandWide {
  static constexpr int kCopies = kWideBytes / 1024 / kWaves; // 4
  __amdgpu_buffer_rsrc_t rsrc;
  int voff[kCopies];
  int dstWave;
  int rd; // parity 0; parity 1 is 64 bytes (four groups) further, i.e. rd ^ 64

  __device__ __forceinline__ void setup(const uint16_t *ptr, int64_t ld, int64_t first, int w0, int64_t extent,
                                        int wave, int lane) {
    const int64_t rows = extent / ld - first;
    const int last = rows < 256 ? int(rows) - 1 : 255;
    rsrc = make_rsrc(ptr + first * ld, int64_t(last + 1) * ld * 2);
#pragma unroll
    for (int q = 0; q < kCopies; ++q) {
      const int row = wave * (256 / kWaves) + q * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ ((row >> 1) & 7);
      voff[q] = int((int64_t(min(row, last)) * ld + chunk * 8) * 2);
    }
    dstWave = wave * (256 / kWaves) * (2 * RK * 2);
    const int fragRow = lane & 15, kGroup = lane >> 4;
    rd = (w0 + fragRow) * (2 * RK * 2) + ((kGroup ^ ((fragRow >> 1) & 7)) << 4);
  }
  // one half (the first or the last 16 of the wavefront's 32 rows) of the wavefront's copies of slab kt2
  // (K-steps 2 kt2 and 2 kt2 + 1)
  __device__ __forceinline__ void dma(LdsChar *lds, int image, int kt2, int half) const {
#pragma unroll
    for (int q = half * (kCopies / 2); q < (half + 1) * (kCopies / 2); ++q)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, lds + image + dstWave + q * 1024, 16, voff[q], kt2 * (2 * RK * 2), 0, 0);
  }
  __device__ __forceinline__ typename T::Frag read(const char *lds, int image, int f, int parity) const {
    return *reinterpret_cast<const typename T::Frag *>(lds + image + (rd ^ (parity * 64)) + f * 16 * (2 * RK * 2));
  }
};

// kAT / kBT as in gemm_blocked.  A is KContig unless transposed; B is KContig only
// when transposed.  kWideA: A's slabs are 64 k wide (A [M,K] and K a multiple of 64 only).
// Tile number -> tile origin, XCD-aware: workgroup ids congruent mod 8 share an XCD, and the tiles they
// take cover a compact band kGroupM tiles high, so the XCD's L2 serves few A and B panels at a time.
struct TileOrigin {
  int64_t m0, n0;
};
__device__ __forceinline__ TileOrigin tile_origin(int id, int tilesM, int tilesN) {
  const int tiles = tilesM * tilesN;
  int pid = id;
  if (tiles % 8 == 0)
    pid = (pid % 8) * (tiles / 8) + pid / 8;
  const int group = kGroupM * tilesN;
  const int firstM = (pid / group) * kGroupM;
  const int groupRows = min(tilesM - firstM, kGroupM);
  const int tileM = firstM + (pid % group) % groupRows;
  const int tileN = (pid % group) / groupRows;
  return TileOrigin{int64_t(tileM) * BM, int64_t(tileN) * BN};
}

// The K loop of one 256 x 256 tile of C at (m0, n0) over K-steps [ktBegin, ktEnd) (32 k each; with wide A
// slabs both even), ADDED onto acc.  acc[i][j] is the 16 x 16 block at rows 16 i, columns 16 j of the
// wavefront's 128 x 64 part; Epi::kColumnsInRegisters says which way round it is held (see the epilogue).
template <typename T, bool kAT, bool kBT, typename Epi, int kProbe = 0, bool kTail = false, bool kWideA = false>
__device__ __forceinline__ void gemm_tile_mainloop(f32x4 (&acc)[FI][FJ], const uint16_t *__restrict__ A,
                                                   const uint16_t *__restrict__ B, int64_t M, int64_t N, int64_t K,
                                                   char *lds, int64_t m0, int64_t n0, int ktBegin, int ktEnd) {
  static_assert(FI == 8 && FJ == 4 && kWaves == 8, "written for 8 wavefronts of 8 x 4 MFMA tiles");
  static_assert(!kWideA || (!kAT && !kTail), "wide A slabs: A is [M,K] and K a multiple of 64");
  LdsChar *lds_base = (LdsChar *)lds;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / kWavesN, wn = wave % kWavesN;

  const int waveU = __builtin_amdgcn_readfirstlane(wave);
  const int kTiles = ktEnd - ktBegin;           // steps of this call; step t below is K-step ktBegin + t
  const int lastTile = kTiles - 1;
  const int lastOfK = int((K + RK - 1) / RK) - 1; // the last K-step of the whole product
  const int kRem = int(K - int64_t(lastOfK) * RK); // k in that step: 32, or 8 / 16 / 24 with kTail
  Operand<T, kAT, FI, kTail> opA;
  OperandWide<T, FI> opAW;
  Operand<T, !kBT, FJ, kTail> opB;
  if constexpr (kWideA)
    opAW.setup(A, K, m0, wm * WM, M * K, waveU, lane);
  else
    opA.setup(A, kAT ? M : K, m0, wm * WM, M * K, waveU, lane, kRem);
  opB.setup(B, kBT ? K : N, n0, wn * WN, K * N, waveU, lane, kRem);
  // LDS: B's ring of four 16 KiB slabs at 0, then A's -- four 16 KiB slabs, or three 64-k-wide ones of 32 KiB.
  // Offsets below are wave-uniform byte offsets of a slab.
  constexpr int kRingA = kRingBytes;
  const int lastWide = kTiles / 2 - 1; // (kWideA: kTiles is even)
  auto dma_a = [&](int kt, int off, int half = 0) { // narrow: step kt of this call; wide: one half of its 64-k slab kt
    if constexpr (!(kProbe & kProbeNoCopyA)) {
      if constexpr (kWideA)
        opAW.dma(lds_base, off, ktBegin / 2 + kt, half);
      else
        opA.dma(lds_base, off, ktBegin + kt, kTail && ktBegin + kt == lastOfK);
    }
  };
  auto dma_b = [&](int kt, int off) {
    if constexpr (!(kProbe & kProbeNoCopyB))
      opB.dma(lds_base, off, ktBegin + kt, kTail && ktBegin + kt == lastOfK);
  };

  // A step multiplies the wavefront's upper four row fragments (half 0), then the lower four
  // (half 1), each by all four B fragments.  af[h] holds half h's A fragments; bf[p] the B
  // fragments of a step of parity p.
  typename T::Frag af[2][FI / 2], bf[2][FJ];
  // off: the slab's byte offset; parity: which half of a wide slab (the K-step's parity)
  auto read_a = [&](int off, int h, int ii, int parity) {
    if constexpr (kProbe & kProbeCopiesOnly)
      asm volatile("" : "+v"(af[h][ii]));
    else if constexpr (kWideA)
      af[h][ii] = opAW.read(lds, off, h * (FI / 2) + ii, parity);
    else
      af[h][ii] = opA.read(lds, off, h * (FI / 2) + ii);
  };
  auto read_b = [&](int off, int p, int j) {
    if constexpr (kProbe & kProbeCopiesOnly)
      asm volatile("" : "+v"(bf[p][j]));
    else
      bf[p][j] = opB.read(lds, off, j);
  };
  auto mm = [&](int h, int p, int ii, int j) {
    if constexpr (kProbe & kProbeCopiesOnly)
      asm volatile("" ::"v"(af[h][ii]), "v"(bf[p][j]));
    else if constexpr (Epi::kColumnsInRegisters)
      acc[h * (FI / 2) + ii][j] = T::mfma(bf[p][j], af[h][ii], acc[h * (FI / 2) + ii][j]);
    else
      acc[h * (FI / 2) + ii][j] = T::mfma(af[h][ii], bf[p][j], acc[h * (FI / 2) + ii][j]);
  };
  // half 0 of a step of parity p: 16 MFMAs, and between them the reads of this step's lower
  // A fragments (the fences keep the compiler from regrouping them).  The MFMAs go column
  // block by column block, up and down the row blocks in turn, so that one operand at most
  // changes from one MFMA to the next (fewer operand bits switching: about 1 % on random data).
  auto half0 = [&](int p, int aCur) {
#pragma unroll
    for (int j = 0; j < FJ; ++j) {
#pragma unroll
      for (int s = 0; s < FI / 2; ++s) {
        mm(0, p, (j & 1) ? FI / 2 - 1 - s : s, j);
        if (s == 0) read_a(aCur, 1, j, p);
        IMEX_FENCE();
      }
    }
  };
  // half 1: 16 MFMAs, and between them the reads of the NEXT step's upper A fragments and
  // of its B fragments (into the other parity's registers)
  auto half1 = [&](int p, int aNxt, int bNxt) {
#pragma unroll
    for (int j = 0; j < FJ; ++j) {
#pragma unroll
      for (int s = 0; s < FI / 2; ++s) {
        mm(1, p, (j & 1) ? FI / 2 - 1 - s : s, j);
        if (s == 0) read_a(aNxt, 0, j, p ^ 1);
        if (s == 2) read_b(bNxt, p ^ 1, j);
        IMEX_FENCE();
      }
    }
  };

  // prologue: tiles 0 .. kDist-1 in flight, tile 0 landed, its first fragments in registers.
  // Wide A: slabs 0 and 1 (K-steps 0-3) and B's tiles 0-2, issued in the order A0 B0 | A1 (first half) B1 |
  // A1 (second half) B2 -- the loop's own pattern of two A and two B copies per step -- so that the
  // same count of copies may stay in flight here and at every step's wait: two steps' worth, eight per wavefront.
  constexpr int kInFlight = (kDist - 1) * 2 * kDmaPerWave;
  static_assert(!kWideA || OperandWide<T, FI>::kCopies / 2 == kDmaPerWave, "a wide slab's half is one step's A copies");
  if constexpr (kProbe & kProbeNoLoopCopies) { // every stage filled once, with real operand values
#pragma unroll
    for (int t = 0; t < kStages; ++t) {
      dma_b(min(t, lastTile), t * kImageBytes);
      if constexpr (!kWideA)
        dma_a(min(t, lastTile), kRingA + t * kImageBytes);
    }
    if constexpr (kWideA)
#pragma unroll
      for (int d = 0; d < kWideStages; ++d) {
        dma_a(min(d, lastWide), kRingA + d * kWideBytes, 0);
        dma_a(min(d, lastWide), kRingA + d * kWideBytes, 1);
      }
    wait_vmcnt<0>();
  } else if constexpr (kWideA) {
    dma_a(0, kRingA, 0);
    dma_a(0, kRingA, 1);
    dma_b(0, 0);
    dma_a(min(1, lastWide), kRingA + kWideBytes, 0);
    dma_b(min(1, lastTile), kImageBytes);
    dma_a(min(1, lastWide), kRingA + kWideBytes, 1);
    dma_b(min(2, lastTile), 2 * kImageBytes);
    if constexpr (kProbe & (kProbeNoCopyA | kProbeNoCopyB))
      wait_vmcnt<(kDist - 1) * kDmaPerWave>();
    else
      wait_vmcnt<kInFlight>();
  } else {
#pragma unroll
    for (int t = 0; t < kDist; ++t) {
      dma_a(min(t, lastTile), kRingA + t * kImageBytes);
      dma_b(min(t, lastTile), t * kImageBytes);
    }
    wait_vmcnt<kInFlight>();
  }
  __builtin_amdgcn_s_barrier();
  IMEX_FENCE();
#pragma unroll
  for (int ii = 0; ii < FI / 2; ++ii) read_a(kRingA, 0, ii, 0);
#pragma unroll
  for (int j = 0; j < FJ; ++j) read_b(0, 0, j);
  IMEX_FENCE();

  // slab offsets: B's of tile t, t+1 and the one tile t+kDist goes to (= tile t-1's); A's likewise, or,
  // wide: the slab of K-steps t and t+1 (t even), the next one, and the one the copies of steps t and
  // t+1 go to (the slab two ahead = the one that K-steps t-2 and t-1 were read from)
  int bCur = 0, bNxt = kImageBytes, bDma = kDist * kImageBytes;
  int aCur = kRingA, aNxt = kRingA + (kWideA ? kWideBytes : kImageBytes);
  int aDma = kRingA + (kWideA ? 2 * kWideBytes : kDist * kImageBytes);
  auto next_b = [](int off) { return off + kImageBytes == kRingBytes ? 0 : off + kImageBytes; };
  auto next_a = [](int off) {
    constexpr int kSlab = kWideA ? kWideBytes : kImageBytes, kEnd = kRingA + (kWideA ? kWideStages * kWideBytes : kRingBytes);
    return off + kSlab == kEnd ? kRingA : off + kSlab;
  };
  auto step = [&](int p, int t) {
    // The slabs of tile t-1 are free: every wavefront passed the previous step's
    // barrier after its last reads of them.  Past the end of K the copies re-fetch the
    // last tile into a slab nobody reads, so every step is the same code.
    if constexpr (!(kProbe & kProbeNoLoopCopies)) {
      if constexpr (kWideA) {
        dma_a(min(t / 2 + 2, lastWide), aDma, p);
      } else {
        dma_a(min(t + kDist, lastTile), aDma);
      }
      dma_b(min(t + kDist, lastTile), bDma);
    }
    IMEX_FENCE();
    half0(p, aCur);                                 // rows 0-63 of tile t; reads its rows 64-127
    if constexpr (kProbe & (kProbeNoCopyA | kProbeNoCopyB))
      wait_vmcnt<(kDist - 1) * kDmaPerWave>();      // (probe with one operand's copies only)
    else
      wait_vmcnt<kInFlight>();                      // tile t+1 has landed (this wavefront's part) ...
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();                   // ... and everyone else's; all reads of tile t are done
    IMEX_FENCE();
    // rows 64-127 of tile t; reads tile t+1's rows 0-63 and B (wide A: tile t+1 is the other half of
    // the same slab after an even step, the first half of the next slab after an odd one)
    half1(p, kWideA && p == 0 ? aCur : aNxt, bNxt);
    bCur = bNxt;
    bNxt = next_b(bNxt);
    bDma = next_b(bDma);
    if (!kWideA || p == 1) {
      aCur = aNxt;
      aNxt = next_a(aNxt);
      aDma = next_a(aDma);
    }
  };
  int t = 0;
  for (; t + 1 < kTiles; t += 2) { // two steps per trip, so that the B registers' parity is a literal
    step(0, t);
    step(1, t + 1);
  }
  if (t < kTiles)
    step(0, t);
  wait_vmcnt<0>();
}

// The epilogue of a tile: what `epi` does with every element of acc that lies inside C.
template <typename Epi, int kProbe = 0>
__device__ __forceinline__ void gemm_tile_epilogue(f32x4 (&acc)[FI][FJ], int64_t M, int64_t N, Epi epi, int64_t m0,
                                                   int64_t n0) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int wm = wave / kWavesN, wn = wave % kWavesN;
  if constexpr (kProbe & (kProbeNoEpilogue | kProbeCopiesOnly)) {
#pragma unroll
    for (int i = 0; i < FI; ++i)
#pragma unroll
      for (int j = 0; j < FJ; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          asm volatile("" ::"v"(acc[i][j][r]));
    return;
  }
  // -- epilogue.  kColumnsInRegisters: lane holds, for block (i,j), row lane%16 and columns
  //    (lane/16)*4 + 0..3; otherwise column lane%16 and rows (lane/16)*4 + 0..3.
  const bool interior = m0 + BM <= M && n0 + BN <= N; // uniform over the workgroup: nothing to mask
  if constexpr (Epi::kColumnsInRegisters) {
    const int64_t mBase = m0 + wm * WM + (lane & 15), nBase = n0 + wn * WN + (lane >> 4) * 4;
    if constexpr (ExchangesHalfRows<Epi>::value) {
      if (interior && N % 4 == 0) {
        asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory"); // the last MFMA results are in their registers
        const int64_t mRow = m0 + wm * WM + (lane & 7), nCol = n0 + wn * WN + ((lane >> 3) & 1) * 16 + (lane >> 4) * 4;
#pragma unroll
        for (int i = 0; i < FI; ++i)
#pragma unroll
          for (int j = 0; j < FJ; j += 2) {
            // X = block j, Y = block j + 1.  T = X rotated by eight lanes within each row of 16; X's
            // lanes 8-15 take Y's lanes 0-7; Y's lanes 0-7 take what X's lanes 8-15 held.  Four
            // registers at a time, so that no DPP source was written by the three instructions before it.
            f32x4 &X = acc[i][j], &Y = acc[i][j + 1];
            float t0, t1, t2, t3;
            asm volatile("v_mov_b32_dpp %8, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                         "v_mov_b32_dpp %9, %1 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                         "v_mov_b32_dpp %10, %2 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                         "v_mov_b32_dpp %11, %3 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
                         "v_mov_b32_dpp %0, %4 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                         "v_mov_b32_dpp %1, %5 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                         "v_mov_b32_dpp %2, %6 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                         "v_mov_b32_dpp %3, %7 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                         "v_mov_b32_dpp %4, %8 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x3\n\t"
                         "v_mov_b32_dpp %5, %9 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x3\n\t"
                         "v_mov_b32_dpp %6, %10 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x3\n\t"
                         "v_mov_b32_dpp %7, %11 quad_perm:[0,1,2,3] row_mask:0xf bank_mask:0x3\n\t"
                         "s_nop 1"
                         : "+v"(X[0]), "+v"(X[1]), "+v"(X[2]), "+v"(X[3]), "+v"(Y[0]), "+v"(Y[1]), "+v"(Y[2]),
                           "+v"(Y[3]), "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3));
            epi.vec4(mRow + i * 16, nCol + j * 16, N, X);
            epi.vec4(mRow + i * 16 + 8, nCol + j * 16, N, Y);
          }
        return;
      }
    }
    if (interior) {
#pragma unroll
      for (int i = 0; i < FI; ++i)
#pragma unroll
        for (int j = 0; j < FJ; ++j)
          epi.vec4(mBase + i * 16, nBase + j * 16, N, acc[i][j]);
    } else {
#pragma unroll
      for (int i = 0; i < FI; ++i)
#pragma unroll
        for (int j = 0; j < FJ; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int64_t m = mBase + i * 16, n = nBase + j * 16 + r;
            if (m < M && n < N)
              epi(m, n, N, acc[i][j][r]);
          }
    }
  } else {
    // Blocks j and j+1 sit side by side in C.  Swapping the odd 16-lane rows of one with the
    // even rows of the other leaves lanes 0-31 of a register with 32 consecutive columns of
    // one row of C and lanes 32-63 with the row 8 below: whole 128-byte lines per store.
    const int64_t mBase = m0 + wm * WM + (lane >> 5) * 8, nBase = n0 + wn * WN + (lane & 31);
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory"); // the last MFMA results are in their registers
#pragma unroll
    for (int i = 0; i < FI; ++i)
#pragma unroll
      for (int j = 0; j < FJ; j += 2)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // (written as an instruction: the compiler's own handling of the corresponding builtin
          // lost track of the second result here; the waits on either side stand in for the
          // hazard padding the compiler would add)
          asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1"
                       : "+v"(acc[i][j][r]), "+v"(acc[i][j + 1][r])); // -> rows r, r+8 | rows r+4, r+12
        }
    if constexpr (ReadsC<Epi>::value) {
      if (interior) {
        // the old values of row block i + 1 are requested before row block i is combined and stored
        float old[2][FJ * 4];
        auto fetch_block = [&](int i, float(&into)[FJ * 4]) {
#pragma unroll
          for (int j = 0; j < FJ; j += 2)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              into[j * 4 + r] = epi.fetch(mBase + i * 16 + r, nBase + j * 16, N);
              into[j * 4 + 4 + r] = epi.fetch(mBase + i * 16 + r + 4, nBase + j * 16, N);
            }
        };
        fetch_block(0, old[0]);
#pragma unroll
        for (int i = 0; i < FI; ++i) {
          if (i + 1 < FI)
            fetch_block(i + 1, old[(i + 1) & 1]);
#pragma unroll
          for (int j = 0; j < FJ; j += 2)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              epi.put(mBase + i * 16 + r, nBase + j * 16, N, acc[i][j][r], old[i & 1][j * 4 + r]);
              epi.put(mBase + i * 16 + r + 4, nBase + j * 16, N, acc[i][j + 1][r], old[i & 1][j * 4 + 4 + r]);
            }
        }
        return;
      }
    }
    if (interior) {
#pragma unroll
      for (int i = 0; i < FI; ++i)
#pragma unroll
        for (int j = 0; j < FJ; j += 2)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            epi(mBase + i * 16 + r, nBase + j * 16, N, acc[i][j][r]);
            epi(mBase + i * 16 + r + 4, nBase + j * 16, N, acc[i][j + 1][r]);
          }
    } else {
#pragma unroll
      for (int i = 0; i < FI; ++i)
#pragma unroll
        for (int j = 0; j < FJ; j += 2)
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int64_t m = mBase + i * 16 + r + 4 * h, n = nBase + j * 16;
              if (m < M && n < N)
                epi(m, n, N, acc[i][j + h][r]);
            }
    }
  }
}

__device__ __forceinline__ void zero_accumulators(f32x4 (&acc)[FI][FJ]) {
#pragma unroll
  for (int i = 0; i < FI; ++i)
#pragma unroll
    for (int j = 0; j < FJ; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        acc[i][j][r] = 0.0f;
}

// One 256 x 256 tile of C: tile number `id` of a tilesM x tilesN grid, all of K.
template <typename T, bool kAT, bool kBT, typename Epi, int kProbe = 0, bool kTail = false, bool kWideA = false>
__device__ __forceinline__ void gemm_tile(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B, int64_t M,
                                          int64_t N, int64_t K, Epi epi, char *lds, int tilesM, int tilesN, int id) {
  const TileOrigin o = tile_origin(id, tilesM, tilesN);
  f32x4 acc[FI][FJ];
  zero_accumulators(acc);
  gemm_tile_mainloop<T, kAT, kBT, Epi, kProbe, kTail, kWideA>(acc, A, B, M, N, K, lds, o.m0, o.n0, 0,
                                                              int((K + RK - 1) / RK));
  gemm_tile_epilogue<Epi, kProbe>(acc, M, N, epi, o.m0, o.n0);
}

// Workgroups stride over the tiles: a launch with fewer workgroups than tiles still covers C, one
// with more leaves the surplus nothing to do.
template <typename T, bool kAT, bool kBT, typename Epi, int kProbe = 0, bool kTail = false, bool kWideA = false>
__device__ __forceinline__ void gemm_tiled(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                                           int64_t M, int64_t N, int64_t K, Epi epi, char *lds) {
  const int tilesM = int((M + BM - 1) / BM), tilesN = int((N + BN - 1) / BN);
  const int tiles = tilesM * tilesN, workgroups = gridDim.x * gridDim.y;
  for (int id = blockIdx.y * gridDim.x + blockIdx.x; id < tiles; id += workgroups) {
    gemm_tile<T, kAT, kBT, Epi, kProbe, kTail, kWideA>(A, B, M, N, K, epi, lds, tilesM, tilesN, id);
    if (id + workgroups < tiles)
      __syncthreads(); // the ring is reused by this workgroup's next tile
  }
}

// ---- stream-K: a tile count that does not fill the chip a whole number of times ------------------------
// W workgroups (one per CU: the launch must not exceed the CUs, so that all of them are resident) take
// floor(tiles / W) * W tiles whole, as above.  The K loops of the R tiles that are left -- R * K / 64
// slabs of 64 k -- are then dealt out evenly, W consecutive ranges of slabs over the tiles laid end to end,
// so every CU is busy for R / W of a tile's time instead of R of them for all of it.  A range touches at
// most two tiles.  The part of a range that ends with its tile's last slab FINISHES that tile: it keeps its
// sums in registers, adds what the earlier parts of the tile produced and runs the epilogue.  Any other part
// is a PRODUCER: it writes its 256 x 256 partial sums (f32, 256 KiB) to the workgroup's own slot of the
// workspace and then publishes flags[workgroup] = epoch.  A workgroup runs its producer part first and its
// finisher part second, so a finisher only ever waits for parts that were started before it started its
// own; the wait is bounded, and a finisher that runs out of patience computes the missing slabs itself --
// the result is the same and the kernel always ends.
//
// workspace: 4096 bytes of flags (one 32-bit word per workgroup, at most 1024 workgroups), then W slots
// of 256 KiB.  epoch: any value that differs from the one of the previous launch that used the same
// workspace (the flags are never cleared; a stale flag cannot equal a new epoch).  Launches that share a
// workspace must not overlap.  The sums of a tile are added in a different order than in the one-workgroup
// form (partials, then the finisher's own), so results agree to rounding, not bit for bit.
constexpr int kStreamKMaxWorkgroups = 1024;
constexpr int64_t kStreamKFlagBytes = 4096, kStreamKSlotFloats = int64_t(BM) * BN;
constexpr int kStreamKDefaultSpins = 1 << 20; // x ~1 us of sleep each: about a second

// A slot holds the 32 blocks of every lane, block by block: 512 lanes x 16 bytes = 8 KiB per block, so every
// store and load instruction moves whole lines.  Addresses are (uniform block base, pinned to scalar
// registers by the empty asm) + (the lane's 32-bit byte offset); left alone, the compiler forms all 32
// addresses as 64-bit vector values ahead of the K loop and spills them.
__device__ __forceinline__ char *partial_block(const float *slot, int block) {
  char *base = reinterpret_cast<char *>(const_cast<float *>(slot)) + block * (kThreads * 16);
  asm volatile("" : "+s"(base));
  return base;
}
__device__ __forceinline__ void store_partial(const f32x4 (&acc)[FI][FJ], float *slot) {
  const uint32_t lane16 = threadIdx.x * 16u;
#pragma unroll
  for (int i = 0; i < FI; ++i)
#pragma unroll
    for (int j = 0; j < FJ; ++j)
      *reinterpret_cast<f32x4 *>(partial_block(slot, i * FJ + j) + lane16) = acc[i][j];
}
__device__ __forceinline__ void add_partial(f32x4 (&acc)[FI][FJ], const float *slot) {
  const uint32_t lane16 = threadIdx.x * 16u;
#pragma unroll
  for (int i = 0; i < FI; ++i) { // a row of blocks at a time: four loads in flight, four registers of staging
    f32x4 v[FJ];
#pragma unroll
    for (int j = 0; j < FJ; ++j)
      v[j] = *reinterpret_cast<const f32x4 *>(partial_block(slot, i * FJ + j) + lane16);
#pragma unroll
    for (int j = 0; j < FJ; ++j)
      acc[i][j] += v[j];
  }
}

template <typename T, typename Epi>
__device__ __forceinline__ void gemm_streamk(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B, int64_t M,
                                             int64_t N, int64_t K, Epi epi, char *lds, void *workspace, int64_t epoch,
                                             int64_t spinLimit) {
  const int tilesM = int((M + BM - 1) / BM), tilesN = int((N + BN - 1) / BN);
  const int tiles = tilesM * tilesN, W = gridDim.x * gridDim.y, w = blockIdx.y * gridDim.x + blockIdx.x;
  const int kSteps = int(K / RK), full = tiles / W * W;
  for (int id = w; id < full; id += W) {
    gemm_tile<T, false, false, Epi, 0, false, true>(A, B, M, N, K, epi, lds, tilesM, tilesN, id);
    __syncthreads(); // the ring is reused
  }
  const int R = tiles - full;
  if (R == 0)
    return;
  uint32_t *flags = static_cast<uint32_t *>(workspace);
  float *slots = reinterpret_cast<float *>(static_cast<char *>(workspace) + kStreamKFlagBytes);
  const int64_t perTile = kSteps / 2, U = int64_t(R) * perTile; // slabs of 64 k
  auto range_begin = [&](int q) { return int64_t(q) * U / W; };
  const int64_t begin = range_begin(w), end = range_begin(w + 1);
  if (begin == end)
    return;
  const int tFirst = int(begin / perTile), tLast = int((end - 1) / perTile);
  const uint32_t stamp = static_cast<uint32_t>(epoch);
  // The range's parts: the one in tile tLast when the range crosses into it (slabs from 0: a producer, unless
  // the range happens to end with the tile), then the one in tile tFirst.  One loop around one K loop: a
  // finisher that has waited in vain goes round once more for the slabs nobody brought.
  const int parts = tLast != tFirst ? 2 : 1;
  int *verdict = reinterpret_cast<int *>(lds);
  f32x4 acc[FI][FJ];
  for (int part = 0; part < parts; ++part) {
    const int tile = part == parts - 1 ? tFirst : tLast;
    const int64_t tileStart = int64_t(tile) * perTile;
    const int64_t u0 = max(begin, tileStart) - tileStart, u1 = min(end, tileStart + perTile) - tileStart;
    const TileOrigin o = tile_origin(full + tile, tilesM, tilesN);
    const bool producer = u1 < perTile;
    zero_accumulators(acc);
    int64_t from = u0, to = u1;
    for (bool again = true; again;) {
      gemm_tile_mainloop<T, false, false, Epi, 0, false, true>(acc, A, B, M, N, K, lds, o.m0, o.n0, int(2 * from),
                                                                int(2 * to));
      __syncthreads(); // every wavefront has read its last fragments: the ring is free again
      again = false;
      if (producer) {
        // Partial sums travel between workgroups on different XCDs, whose L2 caches do not see each other's
        // lines: the producer's L2 is written back before the flag goes up (the release below, once per
        // workgroup, after the barrier has collected every wavefront's stores), and the finisher drops what
        // its caches hold once it has seen the flags (the acquire fence, once, outside the polling loop).
        // Device-scope accesses alone (the sc1 bit on the slot's loads and stores, no write-back, no
        // invalidate) were measured and gave stale partials on ordinary device allocations.
        store_partial(acc, slots + int64_t(w) * kStreamKSlotFloats);
        __syncthreads();
        if (threadIdx.x == 0)
          __hip_atomic_store(flags + w, stamp, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
      } else if (from > 0) {
        // the workgroups that hold slabs [0, u0) of this tile: from the one whose range contains the tile's
        // first slab up to w - 1 (those with an empty range hold nothing and publish nothing)
        int first = w;
        while (first > 0 && range_begin(first) > tileStart)
          --first;
        if (threadIdx.x == 0) {
          const int64_t limit = spinLimit > 0 ? spinLimit : kStreamKDefaultSpins;
          int arrived = 1;
          for (int q = first; q < w && arrived; ++q) {
            if (range_begin(q) == range_begin(q + 1))
              continue;
            int64_t spins = 0;
            while (__hip_atomic_load(flags + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != stamp) {
              if (++spins > limit) {
                arrived = 0;
                break;
              }
              __builtin_amdgcn_s_sleep(32);
            }
          }
          if (arrived)
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
          *verdict = arrived;
        }
        __syncthreads();
        const int arrived = *verdict;
        __syncthreads(); // the word is read before the ring is written again
        if (arrived) {
          for (int q = first; q < w; ++q)
            if (range_begin(q) != range_begin(q + 1))
              add_partial(acc, slots + int64_t(q) * kStreamKSlotFloats);
        } else { // nobody came: the missing slabs, computed here, on top of what is in the registers
          to = from;
          from = 0;
          again = true;
        }
      }
    }
    if (!producer)
      gemm_tile_epilogue<Epi>(acc, M, N, epi, o.m0, o.n0);
  }
}

// Whether gemm_streamk can take the problem: the wide-A MFMA path (see gemm_entry), a workspace, and few
// enough workgroups for the flag words.
__device__ __forceinline__ bool streamk_applies(const void *A, const void *B, int64_t M, int64_t N, int64_t K,
                                                const void *workspace) {
  constexpr int64_t kMaxBytes = int64_t(1) << 31, kMaxRow = int64_t(1) << 22;
  return workspace != nullptr && M > 0 && N > 0 && K > 0 && K % (2 * RK) == 0 && N % 8 == 0 && K < kMaxRow &&
         K * N * 2 < kMaxBytes && ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 &&
         (reinterpret_cast<uintptr_t>(workspace) & 15) == 0 && int(gridDim.x * gridDim.y) <= kStreamKMaxWorkgroups;
}

// kWideOk: take A as 64-k-wide slabs where the shape allows (A [M,K], K a multiple of 64)
template <typename T, bool kAT, bool kBT, int kProbe = 0, bool kWideOk = true, typename Epi>
__device__ __forceinline__ void gemm_dispatch(const uint16_t *A, const uint16_t *B, int64_t M, int64_t N, int64_t K,
                                              Epi epi, char *lds) {
  // The MFMA path wants 16-byte aligned rows in memory: K % 8 == 0 (rows of A [M,K], of B [N,K]), and a
  // row of B [K,N] (or of A [K,M] when transposed) is N (M) elements long, so those must be multiples
  // of 8 as well.  K need not fill the last 32-wide step: its copies fetch zeros beyond K.  M and N need not divide the tile: edge tiles multiply padding and store what exists.
  // An operand whose rows are strided in memory is addressed with 32-bit byte offsets from one
  // buffer descriptor, so it has to stay below 2 GiB; a k-contiguous one below 4 Mi elements per row.
  constexpr int64_t kMaxBytes = int64_t(1) << 31, kMaxRow = int64_t(1) << 22;
  const bool fitsA = kAT ? K * M * 2 < kMaxBytes : K < kMaxRow;
  const bool fitsB = kBT ? K < kMaxRow : K * N * 2 < kMaxBytes;
  const bool tileable = M > 0 && N > 0 && K > 0 && K % 8 == 0 && (kBT || N % 8 == 0) && (!kAT || M % 8 == 0) &&
                        fitsA && fitsB &&
                        ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0;
  if (!kAT && kWideOk && tileable && K % (2 * RK) == 0)
    gemm_tiled<T, kAT, kBT, Epi, kProbe, false, !kAT && kWideOk>(A, B, M, N, K, epi, lds);
  else if (tileable && K % RK == 0)
    gemm_tiled<T, kAT, kBT, Epi, kProbe, false>(A, B, M, N, K, epi, lds);
  else if (tileable)
    gemm_tiled<T, kAT, kBT, Epi, kProbe, true>(A, B, M, N, K, epi, lds);
  else
    gemm_blocked<T, kAT, kBT, Epi>(A, B, M, N, K, epi, lds);
}

template <typename T, bool kAT, bool kBT, int kProbe = 0, bool kWideOk = true, typename Epi>
__device__ __forceinline__ void gemm_entry(const uint16_t *A, const uint16_t *B, int64_t M, int64_t N, int64_t K,
                                           Epi epi) {
  // B's four slabs (64 KiB) and A's four (64 KiB), or A's three 64-k-wide ones (96 KiB): all 160 KiB of the CU's LDS.
  __shared__ __attribute__((aligned(16))) char lds[kLdsBytes];
  gemm_dispatch<T, kAT, kBT, kProbe, kWideOk>(A, B, M, N, K, epi, lds);
}

// Entry with a workspace: stream-K where it applies, otherwise exactly gemm_entry.
template <typename T, typename Epi>
__device__ __forceinline__ void gemm_entry_streamk(const uint16_t *A, const uint16_t *B, int64_t M, int64_t N,
                                                   int64_t K, Epi epi, void *workspace, int64_t epoch,
                                                   int64_t spinLimit) {
  __shared__ __attribute__((aligned(16))) char lds[kLdsBytes];
  if (streamk_applies(A, B, M, N, K, workspace))
    gemm_streamk<T, Epi>(A, B, M, N, K, epi, lds, workspace, epoch, spinLimit);
  else
    gemm_dispatch<T, false, false>(A, B, M, N, K, epi, lds);
}

} // namespace imexhip_gemm

#endif
