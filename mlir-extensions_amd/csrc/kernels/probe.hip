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
    if (mode == 2) { // random sign and mantissa, exponent field 0..14, i.e. |v| < 1
      lo = (x & 0x83ffu) | (((x >> 10) % 15u) << 10);
      hi = ((x >> 16) & 0x83ffu) | (((x >> 26) % 15u) << 10);
    } else {         // h / 32768 - 1 for each 16-bit half h: uniform in [-1, 1), exact in f32, one rounding to f16
      lo = imexhip::float_to_half_bits(static_cast<float>(x & 0xffffu) * (1.0f / 32768.0f) - 1.0f);
      hi = imexhip::float_to_half_bits(static_cast<float>(x >> 16) * (1.0f / 32768.0f) - 1.0f);
    }
    lds[i] = mode == 1 ? 0u : (lo | (hi << 16));
  }
  __syncthreads();

  f32x4 acc[kFragsA * kFragsB];
  for (int i = 0; i < kFragsA * kFragsB; ++i)
    for (int r = 0; r < 4; ++r)
      acc[i][r] = 0.0f;

  const f16x8 *slots = reinterpret_cast<const f16x8 *>(lds);
  const int lane = threadIdx.x;
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

  float s = 0.0f;
  for (int i = 0; i < kFragsA * kFragsB; ++i)
    for (int r = 0; r < 4; ++r)
      s += acc[i][r];
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx < outCount)
    out[idx] = s;
}

// ---- the GEMM's tile code with parts switched off (arguments and launch as imex_gemm_f16_f16_f32) ----
#define IMEX_GEMM_PROBE(name, switches)                                                                               \
  extern "C" __global__ __launch_bounds__(imexhip_gemm::kThreads) void name(                                          \
      const uint16_t *A, const uint16_t *B, float *C, int64_t M, int64_t N, int64_t K) {                              \
    imexhip_gemm::gemm_entry<imexhip_gemm::F16, false, false, (switches)>(A, B, M, N, K, imexhip_gemm::StoreF32{C});  \
  }
IMEX_GEMM_PROBE(imex_gemm_probe_no_loop_copies, imexhip_gemm::kProbeNoLoopCopies)
IMEX_GEMM_PROBE(imex_gemm_probe_no_epilogue, imexhip_gemm::kProbeNoEpilogue)
IMEX_GEMM_PROBE(imex_gemm_probe_multiply_only, imexhip_gemm::kProbeNoLoopCopies | imexhip_gemm::kProbeNoEpilogue)
IMEX_GEMM_PROBE(imex_gemm_probe_copies_only, imexhip_gemm::kProbeCopiesOnly)
IMEX_GEMM_PROBE(imex_gemm_probe_copies_only_a, imexhip_gemm::kProbeCopiesOnly | imexhip_gemm::kProbeNoCopyB)
IMEX_GEMM_PROBE(imex_gemm_probe_copies_only_b, imexhip_gemm::kProbeCopiesOnly | imexhip_gemm::kProbeNoCopyA)
