//===- probe.hip - measurement kernels (bench-only code object) --------------===//
//
// Not operators and not in the catalogue (no counterpart in the reference):
//  * imex_mfma_lds_ceiling_f16: what the MFMA pipe sustains on given operand values;
//  * imex_gemm_probe_*: the tiled GEMM's own tile code (gemm_tile.h) with one part switched
//    off -- the K loop's global -> LDS copies, the epilogue, both, or everything but the
//    copies -- to price each part on the benchmark's operands.  Their results are meaningless.
//
// imex_mfma_lds_ceiling_f16: the
// inner product loop of the tiled GEMM with everything but the matrix pipe and
// its LDS operand reads taken away -- no global loads, no barriers in the loop,
// no epilogue beyond one store per lane.
//
// Why it exists: on MI355X the shader clock under MFMA load depends on the
// operand VALUES (switching activity in the multiplier arrays).  With f16
// operands drawn uniformly from (-1, 1) the part settles well below the clock
// its 2.5 PFLOP/s peak is quoted at; with all-zero operands it does not.  This
// kernel measures that ceiling directly, on the same kind of data the GEMM
// benchmark uses, so the GEMM's rate can be held against what the silicon
// sustains on that data as well as against the published peak.
//
//   imex_mfma_lds_ceiling_f16(out: f32*, outCount: i64, iters: i64, mode: i64)
//
// Each workgroup (512 lanes = 8 wavefronts, two per SIMD, like the GEMM) fills
// 64 KiB of LDS with hashed f16 pairs and then runs `iters` steps of the GEMM's K-step: 8 A fragments + 4 B fragments
// read from LDS with ds_read_b128 at a position that moves every step, 32 MFMA
// 16x16x32 on them (a 128 x 64 x 32 product per wavefront).  FLOP per launch =
// gridX * 8 * iters * 32 * 2*16*16*32.  One f32 per lane is stored at the end
// (guarded by outCount) so the work is observable.
//
// mode 0: values uniform in (-1, 1) rounded to f16, the distribution of the GEMM
//         benchmark's operands (half of them have the exponent of 0.5, a quarter
//         the one below, ...);
// mode 1: zeros;
// mode 2: random sign and mantissa with every exponent below 1.0 equally likely --
//         more bits switching per operand than mode 0, and a lower sustained rate.
// mode + 4: the same operand values read from LDS once and then kept in registers, no LDS
//         read inside the loop: what the matrix pipe sustains on these values by itself, which
//         says how much of the distance to the published peak is the multiplier arrays and how
//         much is the LDS traffic that feeds them.
//
// The MFMA shape matters for this ceiling: on the same random operands a loop of
// 32x32x16 instructions with the same LDS bytes per FLOP sustained about 9 % less
// (and about 7 % more on zeros, where instruction issue is the limit instead).
//
//===----------------------------------------------------------------------===//

#include "device_common.h"
#include "gemm_tile.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;
constexpr int kLdsBytes = 65536;
constexpr int kSlots = kLdsBytes / 16; // 16-byte operand slots
constexpr int kFragsA = 8, kFragsB = 4;

} // namespace

extern "C" __global__ __launch_bounds__(kThreads) void imex_mfma_lds_ceiling_f16(float *out, int64_t outCount,
                                                                                  int64_t iters, int64_t mode) {
  __shared__ __attribute__((aligned(16))) uint32_t lds[kLdsBytes / 4];
  for (int i = threadIdx.x; i < kLdsBytes / 4; i += kThreads) {
    uint32_t x = (static_cast<uint32_t>(i) + blockIdx.x * 7919u) * 2654435761u;
    x ^= x >> 15;
    x *= 2246822519u;
    x ^= x >> 13;
    uint32_t lo, hi;
    if ((mode & 3) == 2) { // random sign and mantissa, exponent field 0..14, i.e. |v| < 1
      lo = (x & 0x83ffu) | (((x >> 10) % 15u) << 10);
      hi = ((x >> 16) & 0x83ffu) | (((x >> 26) % 15u) << 10);
    } else {         // h / 32768 - 1 for each 16-bit half h: uniform in [-1, 1), exact in f32, one rounding to f16
      lo = imexhip::float_to_half_bits(static_cast<float>(x & 0xffffu) * (1.0f / 32768.0f) - 1.0f);
      hi = imexhip::float_to_half_bits(static_cast<float>(x >> 16) * (1.0f / 32768.0f) - 1.0f);
    }
    lds[i] = (mode & 3) == 1 ? 0u : (lo | (hi << 16));
  }
  __syncthreads();

  f32x4 acc[kFragsA * kFragsB];
  for (int i = 0; i < kFragsA * kFragsB; ++i)
    for (int r = 0; r < 4; ++r)
      acc[i][r] = 0.0f;

  const f16x8 *slots = reinterpret_cast<const f16x8 *>(lds);
  const int lane = threadIdx.x;
  if (mode & 4) {
    // the same operand values, read from LDS once and then held in registers: the matrix pipe alone
    f16x8 a[kFragsA], b[kFragsB];
#pragma unroll
    for (int i = 0; i < kFragsA; ++i)
      a[i] = slots[(lane + i * 256) & (kSlots - 1)];
#pragma unroll
    for (int j = 0; j < kFragsB; ++j)
      b[j] = slots[(lane + 2048 + j * 256) & (kSlots - 1)];
    for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < kFragsA; ++i)
        asm volatile("" : "+v"(a[i])); // opaque to the compiler: nothing about the loop body is loop-invariant
#pragma unroll
      for (int i = 0; i < kFragsA; ++i)
#pragma unroll
        for (int j = 0; j < kFragsB; ++j)
          acc[i * kFragsB + j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], b[j], acc[i * kFragsB + j], 0, 0, 0);
    }
  } else {
    for (int64_t it = 0; it < iters; ++it) {
      const int off = static_cast<int>(it & 63) * 64;
      f16x8 a[kFragsA], b[kFragsB];
#pragma unroll
      for (int i = 0; i < kFragsA; ++i)
        a[i] = slots[(lane + off + i * 256) & (kSlots - 1)];
#pragma unroll
      for (int j = 0; j < kFragsB; ++j)
        b[j] = slots[(lane + off + 2048 + j * 256) & (kSlots - 1)];
#pragma unroll
      for (int i = 0; i < kFragsA; ++i)
#pragma unroll
        for (int j = 0; j < kFragsB; ++j)
          acc[i * kFragsB + j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], b[j], acc[i * kFragsB + j], 0, 0, 0);
    }
  }

  float s = 0.0f;
  for (int i = 0; i < kFragsA * kFragsB; ++i)
    for (int r = 0; r < 4; ++r)
      s += acc[i][r];
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx < outCount)
    out[idx] = s;
}

// ---- the GEMM's tile code with parts switched off (arguments and launch as imex_gemm_f16_f16_f32) ----
#define IMEX_GEMM_PROBE(name, switches, wideA)                                                                        \
  extern "C" __global__ __launch_bounds__(imexhip_gemm::kThreads) void name(                                          \
      const uint16_t *A, const uint16_t *B, float *C, int64_t M, int64_t N, int64_t K) {                              \
    imexhip_gemm::gemm_entry<imexhip_gemm::F16, false, false, (switches), wideA>(A, B, M, N, K,                       \
                                                                                  imexhip_gemm::StoreF32{C});          \
  }
IMEX_GEMM_PROBE(imex_gemm_probe_no_loop_copies, imexhip_gemm::kProbeNoLoopCopies, true)
IMEX_GEMM_PROBE(imex_gemm_probe_no_epilogue, imexhip_gemm::kProbeNoEpilogue, true)
IMEX_GEMM_PROBE(imex_gemm_probe_multiply_only, imexhip_gemm::kProbeNoLoopCopies | imexhip_gemm::kProbeNoEpilogue, true)
IMEX_GEMM_PROBE(imex_gemm_probe_copies_only, imexhip_gemm::kProbeCopiesOnly, true)
IMEX_GEMM_PROBE(imex_gemm_probe_copies_only_a, imexhip_gemm::kProbeCopiesOnly | imexhip_gemm::kProbeNoCopyB, true)
IMEX_GEMM_PROBE(imex_gemm_probe_copies_only_b, imexhip_gemm::kProbeCopiesOnly | imexhip_gemm::kProbeNoCopyA, true)
// the same with A copied as 32-k slabs (64-byte rows: two L2 requests per 128-byte line), the form
// shapes with K % 64 != 0 take; the whole kernel (real results) and the copy pipeline alone
IMEX_GEMM_PROBE(imex_gemm_probe_narrow_a, 0, false)
IMEX_GEMM_PROBE(imex_gemm_probe_narrow_a_copies_only, imexhip_gemm::kProbeCopiesOnly, false)
IMEX_GEMM_PROBE(imex_gemm_probe_narrow_a_copies_only_a, imexhip_gemm::kProbeCopiesOnly | imexhip_gemm::kProbeNoCopyB, false)

// f32 epilogue variants (real results), measured against the operator's element-per-lane stores after a
// 16-lane-row swap: the same stores non-temporal; 16-byte stores after a half-row exchange (StoreF32Lines)
struct StoreF32NonTemporal {
  static constexpr bool kColumnsInRegisters = false;
  float *C;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    __builtin_nontemporal_store(acc, C + m * N + n);
  }
};
extern "C" __global__ __launch_bounds__(imexhip_gemm::kThreads) void imex_gemm_probe_store_nontemporal(
    const uint16_t *A, const uint16_t *B, float *C, int64_t M, int64_t N, int64_t K) {
  imexhip_gemm::gemm_entry<imexhip_gemm::F16, false, false>(A, B, M, N, K, StoreF32NonTemporal{C});
}
extern "C" __global__ __launch_bounds__(imexhip_gemm::kThreads) void imex_gemm_probe_store_lines(
    const uint16_t *A, const uint16_t *B, float *C, int64_t M, int64_t N, int64_t K) {
  imexhip_gemm::gemm_entry<imexhip_gemm::F16, false, false>(A, B, M, N, K, imexhip_gemm::StoreF32Lines{C});
}

// The MLP epilogue with its 8-byte stores marked non-temporal: does keeping the 90 MB output stream out of the
// last-level cache leave more of it to the operand panels, which every round of tiles fetches again?
struct BiasSiluBF16NonTemporal {
  static constexpr bool kColumnsInRegisters = true;
  uint16_t *out;
  const float *bias;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    imexhip_gemm::BiasSiluBF16{out, bias}(m, n, N, acc);
  }
  __device__ __forceinline__ void vec4(int64_t m, int64_t n, int64_t N, imexhip::f32x4 acc) const {
    const imexhip::f32x4 b = *reinterpret_cast<const imexhip_gemm::f32x4u *>(bias + n);
    imexhip::u32x2 o;
    uint16_t h[4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
      h[r] = imexhip_gemm::bf16_bits_hw(imexhip_gemm::silu_fast(acc[r] + b[r]));
    o.x = h[0] | (uint32_t(h[1]) << 16);
    o.y = h[2] | (uint32_t(h[3]) << 16);
    __builtin_nontemporal_store(o, reinterpret_cast<imexhip::u32x2 *>(out + m * N + n));
  }
};
extern "C" __global__ __launch_bounds__(imexhip_gemm::kThreads) void imex_gemm_probe_mlp_store_nontemporal(
    const uint16_t *A, const uint16_t *B, const float *bias, uint16_t *out, int64_t M, int64_t N, int64_t K) {
  imexhip_gemm::gemm_entry<imexhip_gemm::BF16, false, false>(A, B, M, N, K, BiasSiluBF16NonTemporal{out, bias});
}

// ---- tile copy: the 16-bit transpose's memory traffic without the transposition -------------------
// imex_probe_tile_copy_b16(in, out, rows, cols, mode): the matrix is walked in 256 x 256 tiles of 16-bit
// elements in the transpose's own order (diagonal by diagonal, one 256-lane workgroup per tile, workgroups
// striding), a tile is read as 512-byte row segments (32 lanes x 16 bytes, eight rows per pass, all 32
// loads of a lane issued before its first store, non-temporal) and written back unchanged
//   mode 0: to its own position (a copy),
//   mode 1: to the transposed tile position (tile (ty, tx) lands at (tx, ty); rows == cols): the reads and
//           writes of imex_transpose2d_b16 on the same matrix, row segment for row segment, with no LDS
//           stage and no repacking in between,
//   mode 2: read only (the tile is folded into a value that is practically never stored),
//   mode 3: write only (a pattern instead of input),
//   mode + 4: the eight rows a pass of the workgroup touches lie 32 rows apart instead of side by side.
// What it is for: at a row pitch of 16 KiB (8192 16-bit columns) against 32 KiB, this bounds from above
// what any tile-wise transpose of that matrix can reach.  rows and cols must be multiples of 256.
extern "C" __global__ __launch_bounds__(256) void imex_probe_tile_copy_b16(const uint16_t *in, uint16_t *out,
                                                                          int64_t rows, int64_t cols, int64_t mode) {
  using imexhip::u32x4;
  const int64_t tilesX = cols / 256, tilesY = rows / 256, total = tilesX * tilesY;
  const int seg = threadIdx.x % 32, rb = threadIdx.x / 32;
  const bool transposed = (mode & 3) == 1, readOnly = (mode & 3) == 2, writeOnly = (mode & 3) == 3;
  // mode + 4: a pass takes eight rows 32 apart (rows rb * 32 + p) instead of eight adjacent ones (8 p + rb)
  const int rowStep = (mode & 4) ? 1 : 8, row0 = (mode & 4) ? rb * 32 : rb;
  u32x4 sink = {0, 0, 0, 0};
  for (int64_t t = blockIdx.x; t < total; t += gridDim.x) {
    const int64_t ty = t % tilesY, tx = (ty + t / tilesY) % tilesX;
    const int64_t dy = transposed ? tx : ty, dx = transposed ? ty : tx;
    const uint16_t *src = in + (ty * 256 + row0) * cols + tx * 256 + seg * 8;
    uint16_t *dst = out + (dy * 256 + row0) * cols + dx * 256 + seg * 8;
    u32x4 x[32];
    if (!writeOnly) {
#pragma unroll
      for (int p = 0; p < 32; ++p)
        x[p] = imexhip::load128<true>(reinterpret_cast<const u32x4 *>(src + int64_t(p) * rowStep * cols));
    } else {
#pragma unroll
      for (int p = 0; p < 32; ++p)
        x[p] = u32x4{uint32_t(p), uint32_t(t), threadIdx.x, 0};
    }
    if (!readOnly) {
#pragma unroll
      for (int p = 0; p < 32; ++p)
        imexhip::store128<true>(x[p], reinterpret_cast<u32x4 *>(dst + int64_t(p) * rowStep * cols));
    } else {
#pragma unroll
      for (int p = 0; p < 32; ++p)
        sink ^= x[p];
    }
  }
  if (readOnly && (sink.x ^ sink.y ^ sink.z ^ sink.w) == 0x9e3779b9u) // keeps the loads alive; practically never taken
    out[threadIdx.x] = 1;
}

// ---- tile traffic: the memory traffic of a tile-wise 16-bit transpose for any tile shape ----------------
// imex_probe_tile_traffic_b16_<R>x<C>(in, out, rows, cols): R x C tiles (rows x columns of 16-bit elements)
// are read as row segments of 2 C bytes and the transposed tile position (C rows of R elements) is written
// as row segments of 2 R bytes, in the transpose's tile order.  The 16-byte pieces a lane reads are the ones
// it writes, so the contents end up permuted inside each tile (this is a traffic probe, not a transpose):
// every address a real transpose with that tile shape would touch is touched once, with the same segment
// lengths on both sides, and nothing else happens in between.  rows % R == 0, cols % C == 0, rows == cols.
template <int R, int C, int kLanes>
__device__ __forceinline__ void tile_traffic_b16(const uint16_t *in, uint16_t *out, int64_t rows, int64_t cols) {
  using imexhip::u32x4;
  constexpr int kPieces = R * C / 8 / kLanes; // 16-byte pieces per lane
  static_assert(kPieces >= 1 && kPieces <= 64, "a lane holds its share of the tile in registers");
  const int64_t tilesX = cols / C, tilesY = rows / R, total = tilesX * tilesY;
  for (int64_t t = blockIdx.x; t < total; t += gridDim.x) {
    const int64_t ty = t % tilesY, tx = (ty + t / tilesY) % tilesX;
    u32x4 x[kPieces];
#pragma unroll
    for (int p = 0; p < kPieces; ++p) {
      const int i = p * kLanes + threadIdx.x;
      x[p] = imexhip::load128<true>(
          reinterpret_cast<const u32x4 *>(in + (ty * R + i / (C / 8)) * cols + tx * C + (i % (C / 8)) * 8));
    }
#pragma unroll
    for (int p = 0; p < kPieces; ++p) {
      const int i = p * kLanes + threadIdx.x;
      imexhip::store128<true>(x[p],
                              reinterpret_cast<u32x4 *>(out + (tx * C + i / (R / 8)) * rows + ty * R + (i % (R / 8)) * 8));
    }
  }
}
#define IMEX_TILE_TRAFFIC(R, C, lanes)                                                                          \
  extern "C" __global__ __launch_bounds__(lanes) void imex_probe_tile_traffic_b16_##R##x##C(                     \
      const uint16_t *in, uint16_t *out, int64_t rows, int64_t cols) {                                          \
    tile_traffic_b16<R, C, lanes>(in, out, rows, cols);                                                         \
  }
IMEX_TILE_TRAFFIC(256, 256, 256)
IMEX_TILE_TRAFFIC(128, 128, 256)
IMEX_TILE_TRAFFIC(512, 128, 256)
IMEX_TILE_TRAFFIC(128, 512, 256)
IMEX_TILE_TRAFFIC(512, 256, 512)
IMEX_TILE_TRAFFIC(256, 512, 512)
IMEX_TILE_TRAFFIC(1024, 128, 512)
IMEX_TILE_TRAFFIC(512, 512, 1024)

// ---- LDS service: which lanes an LDS access serves together, and the bank period ---------------------------
// imex_probe_lds_pair(out, kind, lane, bytes_apart): one wavefront; lanes 0 and `lane` alone access LDS 64 times,
// lane 0 at offset 0 and the other at offset bytes_apart, with the access kind 0 .. 5 = 128-bit read, 128-bit
// write, 64-bit read, 64-bit write, 32-bit read, 32-bit write.  Two lanes that are served in one pass and whose
// addresses fall into the same bank cost a bank-conflict cycle per access (SQ_LDS_BANK_CONFLICT of the dispatch:
// 64 or 0); lanes served in different passes never do.  Launch: grid 1, block 64.
extern "C" __global__ __launch_bounds__(64) void imex_probe_lds_pair(uint32_t *out, int64_t kind, int64_t lane,
                                                                    int64_t bytes_apart) {
  using imexhip::u32x2;
  using imexhip::u32x4;
  __shared__ __attribute__((aligned(16))) uint32_t words[1024];
  for (int k = threadIdx.x; k < 1024; k += 64)
    words[k] = k;
  __syncthreads();
  uint32_t acc = 0;
  const int me = threadIdx.x;
  if (me == 0 || me == lane) {
    volatile uint32_t *at = words + (me == 0 ? 0 : (bytes_apart / 4) % 1020);
    for (int it = 0; it < 64; ++it) {
      switch (kind) {
      case 0: acc += (*reinterpret_cast<volatile u32x4 *>(at)).x; break;
      case 1: *reinterpret_cast<volatile u32x4 *>(at) = u32x4{acc, 1, 2, 3}; break;
      case 2: acc += (*reinterpret_cast<volatile u32x2 *>(at)).x; break;
      case 3: *reinterpret_cast<volatile u32x2 *>(at) = u32x2{acc, 1}; break;
      case 4: acc += *at; break;
      default: *at = acc; break;
      }
    }
  }
  if (acc == 0x9e3779b9u) // keeps the reads alive; practically never taken
    out[me] = acc;
}
