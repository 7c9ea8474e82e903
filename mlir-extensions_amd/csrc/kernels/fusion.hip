// Fused element-wise chains of the reference's kLoopFusion / kInputFusion
// benchmarks, each as ONE pass over HBM.
//
// Reference op bodies:
//   benchmarks/kLoopFusion/kLoopFusion.mlir.in:4-30
//       t1 = log(a); t2 = |b|; t3 = t1 + t2; out = t3 - a          (four generics,
//       three full-size temporaries in the reference's lowering)
//   benchmarks/kInputFusion/kInputFusion.mlir.in:6-40
//       t = log(b) + |a|  (same first three generics, on swapped arguments), then
//       out[j] = 0 + sum_i t[i][j]: a reduction over the ROWS, one output per
//       column, added in ascending i (indexing maps (d1,d0) -> (d0), :29-39).
//
// Every operation is a separately rounded f32 one, as in the reference; log is
// the host libm's logf (benchmarks/pipelines/linalg-to-cpu.pp:18-19 lowers
// math.log to it), restated below so that the device lands on the same bits.
// 16-bit variants widen to f32, run the same chain and round once at the end
// (the policy the reference applies to 16-bit types on the GPU,
// docs/Transforms/BF16ToGpu.md:17-26).
//
// Arguments:  loop fusion  (a, b, out, n: i64)              dims = {n}
//             input fusion (a, b, out, rows: i64, cols: i64) dims = {rows, cols}
// Launch: block (256,1,1); loop fusion grid ceil(n / 4096) (f32) or ceil(n / 8192)
// (16-bit), a quarter of that per workgroup below 4 Mi elements.  Input fusion, by shape: below 4096 columns
// block (320,1,1), grid ceil(cols / 4); from 2048 rows and 128 row segments of 128 bytes on block (576,1,1),
// grid ceil(cols * element bytes / 128); otherwise block (256,1,1), grid ceil(cols / c), a workgroup per
// block of c = 64 .. 8 columns (the widest that leaves 512 workgroups).  A launch with 256 lanes always gets
// the last form.  Workgroups stride, so any grid is correct.

#include "device_common.h"

using namespace imexhip;
using namespace imexhip::io;

namespace {

constexpr int kThreads = 256;

// ---------------------------------------------------------------------------
// logf as glibc computes it (Arm Optimized Routines logf: x = 2^k z with z in
// [0x3f330000, ...), c = table centre of z's 1/16 sub-interval, r = z/c - 1,
// log x = k ln2 + log c + r + r^2 (A2 + A1 r + A0 r^2); all in f64 with IEEE
// operations, one final rounding).  A host build of this function agrees with
// libm's logf on every positive finite f32.
// ---------------------------------------------------------------------------
struct LogfEntry {
  double invc, logc;
};
__device__ const LogfEntry kLogfTable[16] = {
    {0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2}, {0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2},
    {0x1.49539f0f010bp+0, -0x1.01eae7f513a67p-2},  {0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3},
    {0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3}, {0x1.25e227b0b8eap+0, -0x1.1aa2bc79c81p-3},
    {0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4}, {0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4},
    {0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5}, {0x1p+0, 0x0p+0},
    {0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5},  {0x1.ca4b31f026aap-1, 0x1.c5e53aa362eb4p-4},
    {0x1.b2036576afce6p-1, 0x1.526e57720db08p-3},  {0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3},
    {0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2},  {0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2},
};

// The arithmetic of logf on the bits of a positive normal number (libm's main path).
__device__ __forceinline__ float logf_libm_core(uint32_t ix, const LogfEntry *table) {
  const uint32_t tmp = ix - 0x3f330000u;
  const int i = (tmp >> 19) & 15;
  const int k = static_cast<int32_t>(tmp) >> 23;
  const uint32_t iz = ix - (tmp & 0xff800000u);
  const double invc = table[i].invc, logc = table[i].logc;
  const double z = static_cast<double>(u2f(iz));
  const double r = z * invc - 1.0;
  const double y0 = logc + static_cast<double>(k) * 0x1.62e42fefa39efp-1;
  const double r2 = r * r;
  double y = 0x1.5575b0be00b6ap-2 * r + -0x1.ffffef20a4123p-2;
  y = -0x1.00ea348b88334p-2 * r2 + y;
  y = y * r2 + (y0 + r);
  return static_cast<float>(y);
}

// Positive, normal, finite and not 1.0: what libm sends straight down its main path.
__device__ __forceinline__ bool logf_ordinary(float x) {
  const uint32_t ix = f2u(x);
  return ix - 0x00800000u < 0x7f800000u - 0x00800000u && ix != 0x3f800000u;
}

__device__ __forceinline__ float logf_libm(float x, const LogfEntry *table) {
  uint32_t ix = f2u(x);
  if (ix == 0x3f800000u)
    return 0.0f;
  if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u) {
    if (ix * 2 == 0)
      return -__builtin_inff(); // log(+-0)
    if (ix == 0x7f800000u)
      return x;                 // log(inf)
    if (ix * 2 > 0xff000000u)
      return x + x;             // NaN: quieted, sign and payload kept
    if (ix & 0x80000000u)
      return u2f(0xffc00000u);  // log of a negative number: libm's (x - x) / 0, the x86 default NaN
    ix = f2u(x * 0x1p23f);      // subnormal: normalise
    ix -= 23u << 23;
  }
  return logf_libm_core(ix, table);
}

__device__ __forceinline__ void stage_table(LogfEntry *lds) {
  if (threadIdx.x < 16)
    lds[threadIdx.x] = kLogfTable[threadIdx.x];
  __syncthreads();
}

// the chains, on f32 values
// kOrdinary: the caller has checked logf_ordinary() for the logarithm's argument in every lane of the
// wavefront, so the chain is straight-line code (libm's special cases cost a masked region per element,
// which keeps the f64 chains of a vector's elements from interleaving).
template <bool kOrdinary = false>
__device__ __forceinline__ float loop_chain(float a, float b, const LogfEntry *table) {
  const float t1 = kOrdinary ? logf_libm_core(f2u(a), table) : logf_libm(a, table);
  const float t2 = __builtin_fabsf(b);
  const float t3 = t1 + t2;
  return t3 - a;
}
template <bool kOrdinary = false>
__device__ __forceinline__ float input_chain(float a, float b, const LogfEntry *table) {
  const float t1 = kOrdinary ? logf_libm_core(f2u(b), table) : logf_libm(b, table);
  const float t2 = __builtin_fabsf(a);
  return t1 + t2;
}

// Elem<Dt>: element access, 16-byte vector unpack / pack to f32 (device_common.h).

// ---- kLoopFusion: two streams in, one out ------------------------------------------
// kVecs 16-byte vectors per lane and pass: four for tensors that stream from HBM, one for small
// ones, where the logarithms of a lane are the critical path and spreading them over more
// workgroups is what shortens it.
constexpr int64_t kSmallFusion = int64_t(1) << 22; // elements

template <Dt D, int kVecs>
__device__ __forceinline__ void loop_fusion_pass(const void *__restrict__ a, const void *__restrict__ b,
                                                 void *__restrict__ out, int64_t n, const LogfEntry *table) {
  using E = Elem<D>;
  constexpr int kVecsPerThread = kVecs;
  constexpr int64_t kElemsPerBlock = int64_t(kThreads) * kVecsPerThread * E::kPerVec;
  const bool aligned = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
                         reinterpret_cast<uintptr_t>(out)) & 15) == 0;
  // workgroups stride over the blocks, so any grid covers n
  for (int64_t base = int64_t(blockIdx.x) * kElemsPerBlock; base < n; base += int64_t(gridDim.x) * kElemsPerBlock) {
    if (aligned && base + kElemsPerBlock <= n) {
      const u32x4 *pa = reinterpret_cast<const u32x4 *>(static_cast<const char *>(a) + base * E::kBytes);
      const u32x4 *pb = reinterpret_cast<const u32x4 *>(static_cast<const char *>(b) + base * E::kBytes);
      u32x4 *po = reinterpret_cast<u32x4 *>(static_cast<char *>(out) + base * E::kBytes);
      u32x4 va[kVecsPerThread], vb[kVecsPerThread];
#pragma unroll
      for (int j = 0; j < kVecsPerThread; ++j) {
        va[j] = load128<true>(pa + j * kThreads + threadIdx.x);
        vb[j] = load128<true>(pb + j * kThreads + threadIdx.x);
      }
#pragma unroll
      for (int j = 0; j < kVecsPerThread; ++j) {
        float fa[E::kPerVec], fb[E::kPerVec];
        E::unpack(va[j], fa);
        E::unpack(vb[j], fb);
        bool ordinary = true;
#pragma unroll
        for (int i = 0; i < E::kPerVec; ++i)
          ordinary = ordinary && logf_ordinary(fa[i]);
        if (__builtin_amdgcn_ballot_w64(!ordinary) == 0) { // uniform over the wavefront
#pragma unroll
          for (int i = 0; i < E::kPerVec; ++i)
            fa[i] = loop_chain<true>(fa[i], fb[i], table);
        } else {
#pragma unroll
          for (int i = 0; i < E::kPerVec; ++i)
            fa[i] = loop_chain(fa[i], fb[i], table);
        }
        store128<true>(E::pack(fa), po + j * kThreads + threadIdx.x);
      }
    } else {
      for (int64_t i = base + threadIdx.x; i < base + kElemsPerBlock && i < n; i += kThreads)
        E::put(out, i, loop_chain(E::get(a, i), E::get(b, i), table));
    }
  }
}

template <Dt D>
__device__ __forceinline__ void loop_fusion(const void *__restrict__ a, const void *__restrict__ b,
                                            void *__restrict__ out, int64_t n) {
  __shared__ LogfEntry table[16];
  stage_table(table);
  if (n < kSmallFusion)
    loop_fusion_pass<D, 1>(a, b, out, n, table);
  else
    loop_fusion_pass<D, 4>(a, b, out, n, table);
}

// ---- kInputFusion: chain + column sums ------------------------------------------------
// out[j] = sum over rows i, in ascending order from +0.0, of chain(a[i,j], b[i,j]) -- the
// reference's order of additions, so the f32 result is the same bits.  Only the additions are
// ordered; the chain (a logarithm per element) is not.  A workgroup owns kCols adjacent columns
// and walks the rows in tiles of 4096 / kCols: all 256 lanes evaluate the chain of a tile into
// LDS (coalesced along the rows), then lane j < kCols adds column j's values of the tile to its
// running sum, in row order.  The tile is double-buffered, so the ordered additions of one tile
// run under the loads and logarithms of the next, with one barrier per tile.  Short matrices
// (up to 1024 rows, the reference's 512 x 1024 among them) use tiles of 1024 elements, so that
// there is a next tile to overlap with; tall ones are faster with fewer barriers.
constexpr int kTileElems = 4096, kSmallTileElems = 1024;

// acc + t[0] + t[stride] + ... + t[(n-1) stride], added in that order: sixteen LDS reads are in flight
// while the previous sixteen values are added.
__device__ __forceinline__ float add_in_row_order(float acc, const float *t, int n, int stride) {
  float v[16], w[16];
  int r = 0;
  if (n >= 16) {
#pragma unroll
    for (int u = 0; u < 16; ++u)
      v[u] = t[u * stride];
    for (r = 16; r + 16 <= n; r += 16) {
#pragma unroll
      for (int u = 0; u < 16; ++u)
        w[u] = t[(r + u) * stride];
#pragma unroll
      for (int u = 0; u < 16; ++u)
        acc = acc + v[u];
#pragma unroll
      for (int u = 0; u < 16; ++u)
        v[u] = w[u];
    }
#pragma unroll
    for (int u = 0; u < 16; ++u)
      acc = acc + v[u];
  }
  for (; r < n; ++r)
    acc = acc + t[r * stride];
  return acc;
}

template <Dt D, int kCols, int kTileElems = ::kTileElems>
__device__ __forceinline__ void input_fusion_cols(const void *__restrict__ a, const void *__restrict__ b,
                                                  void *__restrict__ out, int64_t rows, int64_t cols,
                                                  const LogfEntry *table, float *tile) {
  using E = Elem<D>;
  constexpr int kTileRows = kTileElems / kCols;
  constexpr int kPerLane = kTileElems / kThreads;
  const int tid = threadIdx.x;
  const bool worker = tid < kThreads; // a launch with more lanes: the others only take part in the barriers
  for (int64_t c0 = int64_t(blockIdx.x) * kCols; c0 < cols; c0 += int64_t(gridDim.x) * kCols) {
    float acc = 0.0f;
    int buf = 0;
    for (int64_t r0 = 0; r0 < rows; r0 += kTileRows, buf ^= 1) {
      float *t = tile + buf * kTileElems;
      float xa[kPerLane], xb[kPerLane];
#pragma unroll
      for (int u = 0; u < kPerLane; ++u) {
        const int e = u * kThreads + tid;
        const int64_t r = r0 + e / kCols, c = c0 + e % kCols;
        const bool ok = worker && r < rows && c < cols;
        xa[u] = ok ? E::get(a, r * cols + c) : 2.0f; // positions outside the matrix: any ordinary value, never added
        xb[u] = ok ? E::get(b, r * cols + c) : 2.0f;
      }
      bool ordinary = true;
#pragma unroll
      for (int u = 0; u < kPerLane; ++u)
        ordinary = ordinary && logf_ordinary(xb[u]);
      if (__builtin_amdgcn_ballot_w64(!ordinary) == 0) { // uniform over the wavefront
#pragma unroll
        for (int u = 0; u < kPerLane; ++u)
          if (worker && r0 + (u * kThreads) / kCols < rows) // passes that lie wholly below the last row are skipped
            t[u * kThreads + tid] = input_chain<true>(xa[u], xb[u], table);
      } else {
#pragma unroll
        for (int u = 0; u < kPerLane; ++u)
          if (worker && r0 + (u * kThreads) / kCols < rows)
            t[u * kThreads + tid] = input_chain(xa[u], xb[u], table);
      }
      __syncthreads(); // the tile is complete; the other buffer was consumed before the previous barrier
      if (tid < kCols && c0 + tid < cols) {
        const int n = rows - r0 < kTileRows ? int(rows - r0) : kTileRows;
        acc = add_in_row_order(acc, t + tid, n, kCols);
      }
    }
    if (tid < kCols && c0 + tid < cols)
      E::put(out, c0 + tid, acc);
    __syncthreads(); // both buffers are free for the next block of columns
  }
}

// ---- kInputFusion on tall, wide matrices: the streaming form --------------------------------
// With 4 .. 64 columns per workgroup the form above reads 16 .. 64-byte row segments, computes and adds
// in turn, and is bound by memory latency (17 % of HBM at 8192 x 8192).  Here a workgroup of 576 lanes
// owns the columns of one 128-byte row segment (32 f32 or 64 16-bit columns).  Its first 512 lanes are
// workers: 16 bytes per lane and access, 8 lanes per row, 64 rows per access; a tile is 8192 elements
// (256 or 128 rows), the next tile's loads are issued before this tile's chains are evaluated, and the
// results go into one of two LDS tiles.  The ninth wavefront does nothing but the ordered additions, one
// lane per column, a tile behind the workers: one barrier per tile, passed by everybody, hands a tile
// over and returns the other one.
// The same structure serves narrow matrices (fewer than 4096 columns, the reference's 512 x 1024 among them):
// 256 workers + the adder wavefront = 320 lanes own 4 columns, one element per lane and access, 64 rows per
// tile, eight tiles' loads in flight together.  There the ordered additions are the critical path
// (a lone wavefront issues a dependent addition every ~8 cycles), and what this form buys is that nothing
// else is ever on it: the adder never loads or evaluates, and the workers are always a tile ahead.
constexpr int kStreamWorkers = 512, kStreamThreads = kStreamWorkers + 64;
constexpr int kNarrowWorkers = 256, kNarrowThreads = kNarrowWorkers + 64;
constexpr int kStreamTileElems = 8192;
constexpr int kStreamTileFloats = 64 * (128 + 16); // the largest padded tile: 64 columns of 128 rows
constexpr int64_t kStreamFromRows = 2048;

// kLanesPerRow worker lanes cover a row segment, each with one 16-byte vector (kVec) or one element; an access
// of all workers is a pass, kTilePasses passes make a tile (what is handed to the adder at one barrier), and
// the loads of kGroupTiles tiles are issued together, one such group ahead of the one being evaluated.
template <Dt D, int kLanesPerRow, int kWorkers, int kTilePassesT, int kGroupTilesT, bool kVecT> struct StreamShape {
  static constexpr bool kVec = kVecT;
  static constexpr int kLanes = kLanesPerRow, kWork = kWorkers, kTilePasses = kTilePassesT, kGroupTiles = kGroupTilesT;
  static constexpr int kPer = kVec ? Elem<D>::kPerVec : 1;      // elements per lane and access
  static constexpr int kCols = kLanesPerRow * kPer;             // columns per workgroup
  static constexpr int kRowsPerPass = kWorkers / kLanesPerRow;
  static constexpr int kTileRows = kTilePasses * kRowsPerPass;
  static constexpr int kGroupPasses = kTilePasses * kGroupTiles;
  // A tile lies in LDS COLUMN by column, kTileRows + 16 floats apart, and row r of column c sits at position
  // r ^ row_swizzle(c), a multiple of 4 below 32: blocks of four rows trade places inside their block of 32,
  // so the adder still reads four consecutive rows of its column with one 128-bit access.  Pitch and swizzle
  // follow from how the LDS serves the two kinds of access (measured with two-lane probes): a 32-bit write is
  // served 32 lanes at a time (0-31, 32-63) over banks that repeat every 32 words; a 128-bit read sixteen
  // lanes at a time (0-3 with 12-15, 20-23 and 24-27; 4-11 with 16-19 and 28-31; the same + 32) over banks
  // that repeat every 64 words.  A worker half-wavefront writes four rows of eight column groups with one
  // instruction: the pitch (16 modulo 32 words) puts odd and even groups 16 banks apart, the swizzle
  // 4 x (group index) spreads the four groups of each kind over the four 4-bank blocks.  The adder's sixteen
  // lanes then read sixteen different 16-byte bank groups for every row block.
  static constexpr int kColPitch = kTileRows + 16;
  static __device__ __forceinline__ int row_swizzle(int col) { return 4 * ((col / kPer) & 7); }
  static constexpr int kTileFloats = kCols * kColPitch;
  static_assert(kTileRows % 32 == 0 && kTileFloats <= kStreamTileFloats, "the LDS tiles are sized for 9216 floats");
};
// wide: 128-byte row segments, 8192-element tiles (256 rows of 32 f32, 128 rows of 64 16-bit columns)
template <Dt D>
using WideShape = StreamShape<D, 8, kStreamWorkers, kStreamTileElems / (128 / Elem<D>::kBytes) / (kStreamWorkers / 8), 1, true>;
// narrow: four columns, one element per lane, 64 rows per tile (a lane's first result is ready after ONE chain),
// the loads of eight tiles -- 512 rows -- in flight together
template <Dt D> using NarrowShape = StreamShape<D, 4, kNarrowWorkers, 1, 8, false>;

// what the launch and the kernel both decide on: enough column blocks for the chip, enough rows for a pipeline
template <Dt D> __device__ __forceinline__ bool input_fusion_streams(int64_t rows, int64_t cols) {
  return rows >= kStreamFromRows && cols >= int64_t(WideShape<D>::kCols) * 128;
}
// ... and the narrow form wherever the form above would take four columns per workgroup
__device__ __forceinline__ bool input_fusion_narrow(int64_t cols) { return cols < 8 * 512; }

// acc + c[0] + c[1] + ... + c[n-1], added in that order, for a column c of kTileRows consecutive floats
// (16-byte aligned, all of them readable): sixteen rows arrive as four 128-bit LDS reads while the previous
// sixteen are added, so the adder issues 1.25 instructions per row.
// swz: row r is kept at position r ^ swz (a multiple of 4 below 32: blocks of four rows trade places).
template <int kTileRows>
__device__ __forceinline__ float add_column_in_row_order(float acc, const float *c, int n, int swz = 0) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  f32x4 x[4], y[4];
  auto read16 = [&](f32x4(&v)[4], int r) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      v[q] = *reinterpret_cast<const f32x4 *>(c + ((r + 4 * q) ^ swz));
  };
  auto add16 = [&](const f32x4(&v)[4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      acc = acc + v[q].x;
      acc = acc + v[q].y;
      acc = acc + v[q].z;
      acc = acc + v[q].w;
    }
  };
  int r = 0;
  read16(x, 0);
  for (; r + 32 <= n; r += 32) {
    read16(y, r + 16);
    add16(x);
    read16(x, r + 32 < kTileRows ? r + 32 : 0); // past the tile's last row: any readable rows, not added
    add16(y);
  }
  // x holds rows r .. r + 15; fewer than 32 rows are left
  if (r + 16 <= n) {
    read16(y, r + 16);
    add16(x);
    r += 16;
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (r + 4 * q + e < n)
          acc = acc + y[q][e];
  } else {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (r + 4 * q + e < n)
          acc = acc + x[q][e];
  }
  return acc;
}

// The hand-over of a tile between the worker wavefronts and the adder wavefront.  The two roles run
// different code and meet here from different places, which the hardware barrier allows (it counts
// wavefronts that have arrived, wherever each one arrives from); what makes it correct is that both roles
// pass it exactly once per tile -- `tiles` times per block of columns, the workers after writing tile t,
// the adder before reading it -- and once more together when the block of columns is done.  Written as
// the instruction with the LDS release / acquire around it, not as a call the compiler may treat as
// convergent across the two branches.  The workgroup must be exactly kWork + 64 lanes (the entry checks).
__device__ __forceinline__ void tile_handover() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
}

template <Dt D, typename S>
__device__ __forceinline__ void input_fusion_stream(const void *__restrict__ a, const void *__restrict__ b,
                                                    void *__restrict__ out, int64_t rows, int64_t cols,
                                                    const LogfEntry *table, float *tile) {
  using E = Elem<D>;
  constexpr int kCols = S::kCols, kTileRows = S::kTileRows, kWorkers = S::kWork, kPer = S::kPer;
  constexpr int kGroupPasses = S::kGroupPasses;
  struct Raw { // what one load brings: a 16-byte vector, or one element already widened
    u32x4 v;
    float f;
  };
  const int tid = threadIdx.x;
  const int64_t tiles = (rows + kTileRows - 1) / kTileRows;
  const int64_t groups = (tiles + S::kGroupTiles - 1) / S::kGroupTiles;
  for (int64_t c0 = int64_t(blockIdx.x) * kCols; c0 < cols; c0 += int64_t(gridDim.x) * kCols) {
    if (tid < kWorkers) {
      const int lr = tid / S::kLanes, lc = (tid % S::kLanes) * kPer; // row within a pass, the lane's first column
      // Rows past the end and, in a partial last block, columns past the end re-read a position inside the
      // matrix instead (their results are never added): the loads are then unconditional, straight-line
      // code, and the wait for a tile's data leaves the next group's loads in flight.
      const int64_t col = c0 + lc < cols ? c0 + lc : c0; // vectors: cols is a multiple of the vector, all of it or none
      Raw ca[kGroupPasses], cb[kGroupPasses], na[kGroupPasses], nb[kGroupPasses];
      auto load_group = [&](int64_t g, Raw(&va)[kGroupPasses], Raw(&vb)[kGroupPasses]) {
#pragma unroll
        for (int p = 0; p < kGroupPasses; ++p) {
          const int64_t r = min((g * kGroupPasses + p) * S::kRowsPerPass + lr, rows - 1);
          if constexpr (S::kVec) {
            va[p].v = load128<true>(reinterpret_cast<const u32x4 *>(static_cast<const char *>(a) + (r * cols + col) * E::kBytes));
            vb[p].v = load128<true>(reinterpret_cast<const u32x4 *>(static_cast<const char *>(b) + (r * cols + col) * E::kBytes));
          } else {
            va[p].f = E::get(a, r * cols + col);
            vb[p].f = E::get(b, r * cols + col);
          }
        }
      };
      if (groups > 0) // (no rows: nothing to read, the sums are +0.0)
        load_group(0, ca, cb);
      for (int64_t g = 0; g < groups; ++g) {
        load_group(g + 1 < groups ? g + 1 : g, na, nb); // past the last group: the last one again, unused
#pragma unroll
        for (int j = 0; j < S::kGroupTiles; ++j) {
          const int64_t t = g * S::kGroupTiles + j;
          if (t < tiles) { // uniform
            float *dst = tile + (t & 1) * S::kTileFloats + lc * S::kColPitch;
#pragma unroll
            for (int q = 0; q < S::kTilePasses; ++q) {
              const int p = j * S::kTilePasses + q;
              float fa[kPer], fb[kPer];
              if constexpr (S::kVec) {
                E::unpack(ca[p].v, fa);
                E::unpack(cb[p].v, fb);
              } else {
                fa[0] = ca[p].f;
                fb[0] = cb[p].f;
              }
              bool ordinary = true;
#pragma unroll
              for (int i = 0; i < kPer; ++i)
                ordinary = ordinary && logf_ordinary(fb[i]);
              if (__builtin_amdgcn_ballot_w64(!ordinary) == 0) { // uniform over the wavefront
#pragma unroll
                for (int i = 0; i < kPer; ++i)
                  fa[i] = input_chain<true>(fa[i], fb[i], table);
              } else {
#pragma unroll
                for (int i = 0; i < kPer; ++i)
                  fa[i] = input_chain(fa[i], fb[i], table);
              }
#pragma unroll
              for (int i = 0; i < kPer; ++i)
                dst[i * S::kColPitch + q * S::kRowsPerPass + (lr ^ S::row_swizzle(lc + i))] = fa[i];
            }
            tile_handover(); // tile t is complete; the adder is done with tile t-1, whose buffer tile t+1 goes into
          }
        }
#pragma unroll
        for (int p = 0; p < kGroupPasses; ++p) {
          ca[p] = na[p];
          cb[p] = nb[p];
        }
      }
    } else {
      const int col = tid - kWorkers;
      const bool active = col < kCols && c0 + col < cols;
      float acc = 0.0f;
      for (int64_t t = 0; t < tiles; ++t) {
        tile_handover(); // tile t is complete
        const int n = rows - t * kTileRows < kTileRows ? int(rows - t * kTileRows) : kTileRows;
        if (active)
          acc = add_column_in_row_order<kTileRows>(acc, tile + (t & 1) * S::kTileFloats + col * S::kColPitch, n,
                                                   S::row_swizzle(col));
      }
      if (active)
        E::put(out, c0 + col, acc);
    }
    __syncthreads(); // both tiles are free for the next block of columns
  }
}

// Columns per workgroup: as many as still leave every CU a couple of workgroups (wide blocks read
// longer row segments), down to 4.
__device__ __forceinline__ int input_fusion_block_cols(int64_t cols) {
  return cols >= 64 * 512 ? 64 : cols >= 32 * 512 ? 32 : cols >= 16 * 512 ? 16 : cols >= 8 * 512 ? 8 : 4;
}

template <Dt D>
__device__ __forceinline__ void input_fusion(const void *__restrict__ a, const void *__restrict__ b,
                                             void *__restrict__ out, int64_t rows, int64_t cols) {
  __shared__ LogfEntry table[16];
  __shared__ __attribute__((aligned(16))) float tile[2 * kStreamTileFloats];
  stage_table(table);
  // The launch says which form: 576 or 320 lanes ask for a streaming one, which needs whole aligned vectors.
  const bool vectors = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0 &&
                       cols % Elem<D>::kPerVec == 0;
  if (blockDim.x == kStreamThreads && vectors && input_fusion_streams<D>(rows, cols)) {
    input_fusion_stream<D, WideShape<D>>(a, b, out, rows, cols, table, tile);
    return;
  }
  if (blockDim.x == kNarrowThreads && input_fusion_narrow(cols)) {
    input_fusion_stream<D, NarrowShape<D>>(a, b, out, rows, cols, table, tile);
    return;
  }
  switch (input_fusion_block_cols(cols)) {
  case 64: input_fusion_cols<D, 64>(a, b, out, rows, cols, table, tile); break;
  case 32: input_fusion_cols<D, 32>(a, b, out, rows, cols, table, tile); break;
  case 16: input_fusion_cols<D, 16>(a, b, out, rows, cols, table, tile); break;
  case 8: input_fusion_cols<D, 8>(a, b, out, rows, cols, table, tile); break;
  default:
    if (rows <= 1024)
      input_fusion_cols<D, 4, kSmallTileElems>(a, b, out, rows, cols, table, tile);
    else
      input_fusion_cols<D, 4>(a, b, out, rows, cols, table, tile);
    break;
  }
}

} // namespace

#define IMEX_FUSION_KERNELS(SUFFIX, DT, CTYPE)                                                                       \
  extern "C" __global__ __launch_bounds__(kThreads) void imex_loop_fusion_##SUFFIX(                                  \
      const CTYPE *a, const CTYPE *b, CTYPE *out, int64_t n) {                                                       \
    loop_fusion<DT>(a, b, out, n);                                                                                   \
  }                                                                                                                  \
  extern "C" __global__ __launch_bounds__(kStreamThreads) void imex_input_fusion_##SUFFIX(                                 \
      const CTYPE *a, const CTYPE *b, CTYPE *out, int64_t rows, int64_t cols) {                                      \
    input_fusion<DT>(a, b, out, rows, cols);                                                                         \
  }

IMEX_FUSION_KERNELS(f32, Dt::F32, float)
IMEX_FUSION_KERNELS(f16, Dt::F16, uint16_t)
IMEX_FUSION_KERNELS(bf16, Dt::BF16, uint16_t)
