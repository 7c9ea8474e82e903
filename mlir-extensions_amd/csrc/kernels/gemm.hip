// Tiled MFMA GEMM for gfx950: C[M,N] = A[M,K] . B[K,N], A and B f16 or bf16
// (row-major), f32 accumulate.
//
// Reference kernels (workgroup-level XeGPU, the role XeTile's
// load_tile / prefetch_tile / tile_mma played):
//   test/Integration/Dialect/XeGPU/WG/gemm_4kx4kx4k_f16_f16_f32.mlir:47-91
//     256x256 workgroup tile, K-step 32, three-deep prefetch, C += A.B;
//   test/Integration/Dialect/XeGPU/WG/gemm_4kx4kx4k_f16_f16_f32_bias.mlir:77-116
//     bias[n] broadcast over rows and added after the K loop;
//   benchmarks/silu/silu_gpu.mlir.in:3-19 for the activation fused below.
//
// Blocking on MI355X:
//   workgroup tile 256 x 256, K-step 64, 512 threads = 8 wavefronts in a 2 x 4
//   grid (two per SIMD), each owning 128 x 64 = 4 x 2 MFMA 32x32x16 tiles;
//   A and B tiles go from global memory STRAIGHT into LDS (buffer_load ... lds,
//   16 bytes per lane, no register staging), double-buffered: the copies for
//   step k+1 are issued at the top of step k and awaited just before the
//   step's single barrier;
//   the LDS images are swizzled -- A [256 rows][64 k] by 16-byte group, B
//   [64 k][256 n] by 32-byte pair -- and because a direct copy fixes each lane's
//   LDS position, the swizzle is applied to the lane's GLOBAL address instead;
//   A fragments are 128-bit LDS reads; B is row-major [K,N] while the MFMA wants
//   eight consecutive k per lane, so B fragments use the LDS transpose read
//   (ds_read_b64_tr_b16) -- no permutes, no transposed writes; neither side has
//   LDS bank conflicts (SQ_LDS_BANK_CONFLICT = 0);
//   fragments are double-buffered in registers: the LDS reads of slice s+1 run
//   under the MFMAs of slice s (sched_group_barrier pins the interleaving);
//   workgroup ids are remapped so that the 32 workgroups resident on one XCD
//   (ids congruent mod 8) cover a compact 4 x 8 block of tiles and share A and
//   B panels in that XCD's L2 (L2 hit rate 78%, fabric fetch 1.5x the minimum).
//
// Shapes that are not multiples of the tile (M%256, N%256, K%64) take the
// one-thread-per-output path of the same kernels, which adds in ascending k
// like the reference's CPU loop (lib/ExecutionEngine/ImexRunnerUtils.cpp:308-317).
//
// Launch: block (512,1,1); grid (tiles,1,1) with tiles = (M/256)*(N/256) when
// the shape is tileable, else (ceil(M*N/512),1,1).  The fixed-shape 4096^3 entry
// points take the reference's own launch: blocks (16,16,1), threads (512,1,1).

#include "device_common.h"

using namespace imexhip;

namespace {

// Wavefront grid inside the 256 x 256 workgroup tile: 2 x 4 (eight wavefronts,
// two per SIMD, each 128 x 64) or 2 x 2 (four wavefronts, each 128 x 128).
#ifndef IMEX_GEMM_WAVES_N
#define IMEX_GEMM_WAVES_N 4
#endif
constexpr int kWavesM = 2, kWavesN = IMEX_GEMM_WAVES_N;
constexpr int kThreads = 64 * kWavesM * kWavesN;
constexpr int BM = 256, BN = 256, BK = 64;
constexpr int WM = BM / kWavesM, WN = BN / kWavesN; // wavefront tile
constexpr int TI = WM / 32, TJ = WN / 32;           // MFMA 32x32 tiles per wavefront
constexpr int kWaves = kWavesM * kWavesN;
constexpr int kADma = BM * BK * 2 / 1024 / kWaves;  // 1 KiB global->LDS copies per wavefront and K-step (A)
constexpr int kBDma = BK * BN * 2 / 1024 / kWaves;  // ... (B)
constexpr int kABytes = BM * BK * 2;                // A image: [256 rows][64 k], 16-byte groups swizzled
constexpr int kBBytes = BK * BN * 2;                // B image: [64 k][256 n], 32-byte pairs swizzled
constexpr int kStageBytes = kABytes + kBBytes;     // 64 KiB; two stages = 128 KiB of the 160 KiB LDS
constexpr int kGroupM = 4;                         // tile rows per L2-sharing group

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4 LdsI16x4; // operand type of the LDS transpose read
typedef __attribute__((address_space(3))) char LdsChar;

struct Stage0 { static constexpr int value = 0; };
struct Stage1 { static constexpr int value = 1; };

struct F16 {
  using Frag = f16x8;
  static __device__ __forceinline__ f32x16 mfma(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float widen(uint16_t h) { return half_bits_to_float(h); }
};
struct BF16 {
  using Frag = bf16x8;
  static __device__ __forceinline__ f32x16 mfma(Frag a, Frag b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float widen(uint16_t h) { return bf16_bits_to_float(h); }
};

// Byte offset of 16-byte group `chunk` (0..7) of row `row` in a [rows][64]
// 16-bit LDS image.  The xor spreads both "same chunk, consecutive rows"
// (fragment reads) and "same chunk, rows 8 apart" (transposed B writes) over
// all banks.
__device__ __forceinline__ int lds_off(int row, int chunk) {
  return row * (BK * 2) + (((chunk ^ row ^ (row >> 3)) & 7) << 4);
}

// Instruction-class masks of __builtin_amdgcn_sched_group_barrier.
#define IMEX_SG(mask, n) __builtin_amdgcn_sched_group_barrier(mask, n, 0)
#define IMEX_MFMA 0x008
#define IMEX_VALU 0x002
#define IMEX_VMEM_RD 0x020
#define IMEX_DS_RD 0x100
#define IMEX_DS_WR 0x200
#define IMEX_REP4(x) x x x x
#if IMEX_GEMM_WAVES_N == 2
// per slice: 16 MFMAs and 12 LDS reads (4 b128 for A, 8 transpose reads for B)
#define IMEX_SCHED_SLICE() IMEX_REP4(IMEX_SG(IMEX_MFMA, 1); IMEX_SG(IMEX_DS_RD, 1); IMEX_SG(IMEX_MFMA, 1); IMEX_SG(IMEX_DS_RD, 1); IMEX_SG(IMEX_MFMA, 1); IMEX_SG(IMEX_DS_RD, 1); IMEX_SG(IMEX_MFMA, 1);)
#else
// per slice: 8 MFMAs and 8 LDS reads (4 b128 for A, 4 transpose reads for B)
#define IMEX_SCHED_SLICE() IMEX_REP4(IMEX_SG(IMEX_MFMA, 1); IMEX_SG(IMEX_DS_RD, 1); IMEX_SG(IMEX_MFMA, 1); IMEX_SG(IMEX_DS_RD, 1);)
#endif

// ---- epilogues ------------------------------------------------------------------
struct StoreF32 {       // C = acc
  float *C;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    __builtin_nontemporal_store(acc, C + m * N + n);
  }
};
struct AccumulateF32 {  // C = C + acc   (the reference kernel loads C as its initial accumulator)
  float *C;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    C[m * N + n] = C[m * N + n] + acc;
  }
};
struct BiasAccumulateF32 { // C = bias[n] + (C + acc)  (bias.mlir:88-94,112-113)
  float *C;
  const float *bias;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    C[m * N + n] = bias[n] + (C[m * N + n] + acc);
  }
};
struct BiasSiluBF16 {   // out = bf16( silu( acc + bias[n] ) )
  uint16_t *out;
  const float *bias;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    const float v = acc + bias[n];
    const float y = v / (1.0f + __expf(-v));
    out[m * N + n] = static_cast<uint16_t>(float_to_bf16_bits(y));
  }
};
struct StoreF16 {       // C(f16) = acc   (WG/gemm_4kx4kx4k_f16_f16_f16.mlir)
  uint16_t *C;
  __device__ __forceinline__ void operator()(int64_t m, int64_t n, int64_t N, float acc) const {
    C[m * N + n] = static_cast<uint16_t>(float_to_half_bits(acc));
  }
};

// ---- one-thread-per-output path ---------------------------------------------------
template <typename T, typename Epi>
__device__ __forceinline__ void gemm_scalar(const uint16_t *A, const uint16_t *B, int64_t M, int64_t N, int64_t K,
                                            Epi epi) {
  const int64_t idx = int64_t(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= M * N)
    return;
  const int64_t m = idx / N, n = idx % N;
  float acc = 0.0f;
  for (int64_t k = 0; k < K; ++k) {
    const float p = T::widen(A[m * K + k]) * T::widen(B[k * N + n]);
    acc = acc + p; // rounded multiply, rounded add (file is built with contraction off)
  }
  epi(m, n, N, acc);
}

// ---- tiled MFMA path ----------------------------------------------------------------
// Buffer resource for raw buffer loads: base pointer, byte range, and the gfx9
// "32-bit data format" word; out-of-range lanes read zeros.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, int64_t bytes) {
  const int range = bytes > 0x7fffffff ? 0x7fffffff : int(bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, range, 0x00020000);
}

template <typename T, typename Epi>
__device__ __forceinline__ void gemm_tiled(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                                           int64_t M, int64_t N, int64_t K, Epi epi, char *lds) {
  LdsChar *lds_base = (LdsChar *)lds;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / kWavesN, wn = wave % kWavesN;

  // -- workgroup id -> tile, XCD-aware ------------------------------------------------
  const int tilesM = int(M / BM), tilesN = int(N / BN);
  const int tiles = tilesM * tilesN;
  int pid = blockIdx.y * gridDim.x + blockIdx.x;
  if (tiles % 8 == 0)
    pid = (pid % 8) * (tiles / 8) + pid / 8; // ids congruent mod 8 share an XCD
  const int group = kGroupM * tilesN;
  const int firstM = (pid / group) * kGroupM;
  const int groupRows = min(tilesM - firstM, kGroupM);
  const int tileM = firstM + (pid % group) % groupRows;
  const int tileN = (pid % group) / groupRows;
  const int64_t m0 = int64_t(tileM) * BM, n0 = int64_t(tileN) * BN;

  // -- global -> LDS, directly (no register staging) ------------------------------------
  // buffer_load_dwordx4 ... lds: each wavefront-level instruction moves 64 x 16 B
  // from global memory into 1 KiB of contiguous LDS (lane l lands at base + 16 l;
  // the LDS base is wave-uniform, in M0).  The LDS images are swizzled, so the
  // swizzle is applied on the GLOBAL side: a lane fetches the piece that belongs
  // at its fixed LDS position.
  //   A image [256 rows][64 k]: one instruction = 8 rows; 16-byte group c of row r
  //     lives at group c ^ ((r ^ r>>3) & 7).
  //   B image [64 k][256 n] (row-major, 512 B rows): one instruction = 2 k rows; the
  //     32-byte pair p of row r lives at pair p ^ g(r), g(r) = (r & 3) | ((r>>3 & 1) << 2),
  //     which spreads the rows a transpose read touches over all LDS banks.
  const int waveU = __builtin_amdgcn_readfirstlane(wave);
  const __amdgpu_buffer_rsrc_t aRsrc = make_rsrc(A + m0 * K, int64_t(BM) * K * 2);
  const __amdgpu_buffer_rsrc_t bRsrc = make_rsrc(B + n0, (K * N - n0) * 2);
  int aVoff[kADma], bVoff[kBDma];
#pragma unroll
  for (int q = 0; q < kADma; ++q) {
    const int row = wave * (BM / kWaves) + q * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);
    aVoff[q] = int((int64_t(row) * K + chunk * 8) * 2);
  }
#pragma unroll
  for (int q = 0; q < kBDma; ++q) {
    const int row = wave * (BK / kWaves) + q * 2 + (lane >> 5);
    const int g = (row & 3) | (((row >> 3) & 1) << 2);
    const int chunk = (((((lane & 31) >> 1) ^ g)) << 1) | (lane & 1);
    bVoff[q] = int((int64_t(row) * N + chunk * 8) * 2);
  }
  const int bStep = int(BK * N * 2); // bytes of B per K-step
  auto dma_tile = [&](int kt, int stage) {
    LdsChar *aDst = reinterpret_cast<LdsChar *>(lds_base) + stage * kStageBytes + waveU * (BM / kWaves) * 128;
    LdsChar *bDst = reinterpret_cast<LdsChar *>(lds_base) + stage * kStageBytes + kABytes + waveU * (BK / kWaves) * 512;
#pragma unroll
    for (int q = 0; q < kADma; ++q)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(aRsrc, aDst + q * 1024, 16, aVoff[q], kt * (BK * 2), 0, 0);
#pragma unroll
    for (int q = 0; q < kBDma; ++q)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(bRsrc, bDst + q * 1024, 16, bVoff[q], kt * bStep, 0, 0);
  };

  // -- LDS -> MFMA fragments ---------------------------------------------------------------
  // A: ds_read_b128 of row w*WM + i*32 + (lane&31), 16-byte group ks*2 + (lane>>5).  The
  // swizzled position is ((ks*2 ^ (i&1)*4) ^ z) with z per lane, so four per-lane
  // bases (c = 0,2,4,6) serve every (i, ks); the rest is an immediate.
  const int fragRow = lane & 31, fragHalf = lane >> 5;
  int aRd[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
    aRd[c] = lds_off(wm * WM + fragRow, 2 * c + fragHalf);
  // B: LDS transpose read (ds_read_b64_tr_b16).  Within each group of 16 lanes,
  // lane t supplies the address of 4 consecutive n at k row t/4 and receives 4
  // consecutive k of column n = t.  Lanes 0-31 cover k 0-7 of the slice, lanes
  // 32-63 k 8-15; two reads (k +0..3, +4..7) make one 8-wide MFMA operand.
  int bRd[TJ];
  {
    const int t = lane & 15, nblock = (lane >> 4) & 1, khalf = lane >> 5;
    const int g = (t >> 2) | (khalf << 2);                 // g(row) for row = ks*16 + khalf*8 + h*4 + t/4
    const int pair0 = (wn * WN) / 16 + nblock;             // 32-byte pair holding this lane's n, tile j = 0
#pragma unroll
    for (int j = 0; j < TJ; ++j)
      bRd[j] = kABytes + (khalf * 8 + (t >> 2)) * 512 + (((pair0 + 2 * j) ^ g) * 32) + (t & 3) * 8;
  }

  f32x16 acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0.0f;

  typename T::Frag af[2][TI], bf[2][TJ];
  auto read_frags = [&](int stage, int ks, int buf) {
    const char *base = lds + stage * kStageBytes;
#pragma unroll
    for (int i = 0; i < TI; ++i) {
      const int c = (ks ^ ((i & 1) << 1)) & 3; // which per-lane base: (ks*2 ^ (i&1)*4) / 2
      af[buf][i] = *reinterpret_cast<const typename T::Frag *>(base + aRd[c] + i * 32 * 128);
    }
#pragma unroll
    for (int j = 0; j < TJ; ++j) {
      const char *p = base + bRd[j] + ks * 16 * 512;
      const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsI16x4 *)(p));
      const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsI16x4 *)(p + 4 * 512));
      bf[buf][j] = __builtin_bit_cast(typename T::Frag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    }
  };
  auto mfma_slice = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j)
        acc[i][j] = T::mfma(af[buf][i], bf[buf][j], acc[i][j]);
  };

  // One K-step = four 16-wide slices; fragments are double-buffered in
  // registers (the reads of slice s+1 run under the MFMAs of slice s).  The
  // asynchronous copies of tile kt+1 into the other LDS stage are issued at the
  // top of step kt and awaited (vmcnt) just before the step's closing barrier.
  // Past the end of K they re-fetch the last tile into the stage nobody reads, so
  // every step is the same branch-free code.
  const int kTiles = int(K / BK);
  const int lastTile = kTiles - 1;
  auto k_step = [&](int kt, auto stageTag) {
    constexpr int cur = decltype(stageTag)::value;
    dma_tile(min(kt + 1, lastTile), cur ^ 1);
    read_frags(cur, 1, 1);
    mfma_slice(0);
    IMEX_SCHED_SLICE();
    read_frags(cur, 2, 0);
    mfma_slice(1);
    IMEX_SCHED_SLICE();
    read_frags(cur, 3, 1);
    mfma_slice(0);
    IMEX_SCHED_SLICE();
    mfma_slice(1);
    __builtin_amdgcn_s_waitcnt(0x0f70); // vmcnt(0): this wavefront's copies have landed
    __syncthreads();                    // ... and so have everyone else's
    read_frags(cur ^ 1, 0, 0);
  };

  dma_tile(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();
  read_frags(0, 0, 0);
  int kt = 0;
  for (; kt + 1 < kTiles; kt += 2) { // two steps per trip: the LDS stage is a compile-time constant
    k_step(kt, Stage0{});
    k_step(kt + 1, Stage1{});
  }
  if (kt < kTiles)
    k_step(kt, Stage0{});

  // -- epilogue: lane holds, for tile (i,j), column n = lane%32 and rows
  //    (r/4)*8 + (lane/32)*4 + r%4, r = 0..15.
#pragma unroll
  for (int i = 0; i < TI; ++i)
#pragma unroll
    for (int j = 0; j < TJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = m0 + wm * WM + i * 32 + (r >> 2) * 8 + fragHalf * 4 + (r & 3);
        const int64_t n = n0 + wn * WN + j * 32 + fragRow;
        epi(m, n, N, acc[i][j][r]);
      }
}

template <typename T, typename Epi>
__device__ __forceinline__ void gemm_entry(const uint16_t *A, const uint16_t *B, int64_t M, int64_t N, int64_t K,
                                           Epi epi) {
  // 2 stages x (256 + 256) rows x 64 k x 2 B = 128 KiB of the CU's 160 KiB LDS.
  __shared__ __attribute__((aligned(16))) char lds[2 * kStageBytes];
  const bool tileable = (M % BM == 0) && (N % BN == 0) && (K % BK == 0) && M > 0 && N > 0 && K > 0 &&
                        ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0;
  if (tileable)
    gemm_tiled<T, Epi>(A, B, M, N, K, epi, lds);
  else
    gemm_scalar<T, Epi>(A, B, M, N, K, epi);
}

} // namespace

// C = A.B
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_f16_f16_f32(const uint16_t *A, const uint16_t *B,
                                                                            float *C, int64_t M, int64_t N,
                                                                            int64_t K) {
  gemm_entry<F16>(A, B, M, N, K, StoreF32{C});
}
// C += A.B
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_f16_f16_f32_acc(const uint16_t *A,
                                                                                const uint16_t *B, float *C,
                                                                                int64_t M, int64_t N, int64_t K) {
  gemm_entry<F16>(A, B, M, N, K, AccumulateF32{C});
}
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_bf16_bf16_f32(const uint16_t *A,
                                                                              const uint16_t *B, float *C,
                                                                              int64_t M, int64_t N, int64_t K) {
  gemm_entry<BF16>(A, B, M, N, K, StoreF32{C});
}
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_bf16_bf16_f32_acc(const uint16_t *A,
                                                                                  const uint16_t *B, float *C,
                                                                                  int64_t M, int64_t N,
                                                                                  int64_t K) {
  gemm_entry<BF16>(A, B, M, N, K, AccumulateF32{C});
}
// C(f16) = A.B
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_f16_f16_f16(const uint16_t *A, const uint16_t *B,
                                                                            uint16_t *C, int64_t M, int64_t N,
                                                                            int64_t K) {
  gemm_entry<F16>(A, B, M, N, K, StoreF16{C});
}
// out(bf16) = silu(A.B + bias[n])
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_bf16_bias_silu_bf16(const uint16_t *A,
                                                                                    const uint16_t *B,
                                                                                    const float *bias,
                                                                                    uint16_t *out, int64_t M,
                                                                                    int64_t N, int64_t K) {
  gemm_entry<BF16>(A, B, M, N, K, BiasSiluBF16{out, bias});
}

// Fixed-shape entry points with the reference kernels' own signatures, so the
// reference's host code can launch them unchanged apart from the block size:
//   gemm_4kx4kx4k_f16_f16_f32.mlir:38,48   args (A, B, C), grid (16,16,1), C += A.B
//   gemm_4kx4kx4k_f16_f16_f32_bias.mlir:44,78 args (bias, C, A, B), C = bias + (C + A.B)
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_4kx4kx4k_f16_f16_f32(const uint16_t *A,
                                                                                     const uint16_t *B,
                                                                                     float *C) {
  gemm_entry<F16>(A, B, 4096, 4096, 4096, AccumulateF32{C});
}
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_4kx4kx4k_f16_f16_f32_bias(const float *bias,
                                                                                          float *C,
                                                                                          const uint16_t *A,
                                                                                          const uint16_t *B) {
  gemm_entry<F16>(A, B, 4096, 4096, 4096, BiasAccumulateF32{C, bias});
}
