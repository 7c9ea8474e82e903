// 2-D transpose (and the 3-D full reversal built from it), 16- and 32-bit
// elements, bit-exact moves.
//
// Reference: benchmarks/transpose/transpose2d_gpu.mlir.in:4-11 (out[j,i] = in[i,j])
// and transpose3d_gpu.mlir.in:4-11 (out[k,j,i] = in[i,j,k]); the reference's
// generated kernel moves one element per work-group
// (test/SPIRV/OpTest.Transpose_FLOAT32.mlir:55-57).
//
// Here a workgroup moves a tile through LDS so that both the HBM reads and the
// HBM writes are 128-bit per lane and contiguous per row segment:
//  * 32-bit: R x C tile kept transposed in LDS in 16-byte groups of four input
//    rows; a lane's four row loads give it a 4 x 4 block that it transposes by
//    picking components, so both LDS sides are 128-bit accesses, XOR-swizzled by
//    group so neither side has bank conflicts.
//  * 16-bit: R x 128 tile (or two of them side by side, loaded together), the
//    same scheme on 8 x 8 blocks: a lane's eight row loads are repacked with
//    v_perm_b32 into eight 128-bit groups of the transposed image, one per
//    column; 128-bit LDS accesses on both sides, XOR-swizzled by group.  Problems
//    made of whole 256 x 256 tiles send a tile through LDS a quarter (64 columns)
//    at a time, while the later quarters are still arriving from memory.
//  * Tile size: the WRITE side of a transpose is the scattered one, and its row
//    segments are R elements long.  Measured streaming from HBM, 512-byte write
//    segments reach 74-78% of peak where 256-byte ones stop at 67-70%, so large
//    problems (>= 2^24 elements) use 128 x 128 (32-bit) or 256 x 256 (16-bit) tiles
//    -- 512-byte segments on both sides; smaller ones keep 64 x 64 / 128 x 128
//    tiles, which give more workgroups.
//  * Workgroups walk the tile grid diagonal by diagonal, so that the workgroups
//    in flight together cover every tile row AND every tile column: both strided
//    sides of the transpose are spread over all memory channels.
//  * Loads and stores are non-temporal: each byte is touched once, and keeping
//    the streams out of the caches is what holds up when the tensors are not
//    already cache-resident; cached accesses are faster only when the same
//    buffers are transposed again and again inside the 256 MiB Infinity Cache.
//  * 32-bit problems made of whole 128 x 128 tiles are walked by 512 workgroups (two per CU, what the
//    LDS tile allows), each of which issues the loads of its next tile before the current one goes
//    through LDS and out: a workgroup always has a tile's reads in flight (4096 x 4096 streaming
//    from HBM: 22.9 us against 24.0 us with one workgroup per tile).  The same walk for the 16-bit
//    256 x 256 tile (512 lanes, so that two tiles fit the registers) gained 1.5 % and is not used.
// Shapes or bases that break 16-byte alignment use the scalar 64 x 64 tile path
// of the same kernel.
//
// Arguments: 2-D (in, out, rows: i64, cols: i64); 3-D (in, out, d0, d1, d2: i64).
// Launch: block (256,1,1); one workgroup per tile, grid 2-D (ceil(cols/C),
// ceil(rows/R), 1), 3-D (ceil(d2/C), ceil(d0/R), d1) with (R, C) as above -- for 32-bit
// problems of whole 128 x 128 tiles at most 512 workgroups in all; any
// other grid is also correct (workgroups stride over the tiles).

#include "device_common.h"

using namespace imexhip;

namespace {

constexpr int kThreads = 256;
constexpr int64_t kBigProblem = int64_t(1) << 24; // elements from which the large tiles are used

// in element (i, j) lives at in[i * ldIn + j]; it goes to out[j * ldOut + i].
struct View {
  int64_t rows, cols, ldIn, ldOut;
};

// A workgroup barrier that orders LDS traffic only: global loads stay in flight across it.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---- 32-bit elements: R x C tile ----------------------------------------------------
// LDS holds the tile TRANSPOSED, T[C][R] words, in 16-byte groups of four consecutive input rows.
// A lane loads four consecutive rows (4 b .. 4 b + 3) at four consecutive columns (4 v .. 4 v + 3),
// one 128-bit load per row with whole 512-byte row segments per wavefront; the 4 x 4 block is then
// transposed by picking components -- no data moves between lanes -- and goes to LDS as four 128-bit
// writes, T[4 v + k][group b].  Output rows leave LDS as 128-bit reads of consecutive groups.  Group g
// of row c is kept at position g ^ ((c / 4) % 16): the lanes an LDS access serves together (eight consecutive
// lanes over 128 bytes of banks for a 128-bit write, sixteen lanes over 256 bytes for a 128-bit read) then
// touch different 16-byte bank groups on the write side (consecutive v) and on the read side (consecutive
// g) alike.
template <int R, int C> struct Tile32 {
  static constexpr int VR = C / 4, BP = kThreads / VR, LP = R / 4 / BP; // load: vectors per row, row blocks per pass, passes
  static constexpr int G = R / 4;                                      // 16-byte groups per LDS row
  static_assert(G >= 16 && (G & (G - 1)) == 0 && LP >= 1, "the group swizzle needs at least 16 groups per row");
  u32x4 x[LP][4];

  // kFull: the tile lies wholly inside the matrix, so the loads are unconditional straight-line code
  template <bool kFull>
  __device__ __forceinline__ void load(const uint32_t *__restrict__ in, const View &v, int64_t r0, int64_t c0) {
    const int cv = threadIdx.x % VR, bb = threadIdx.x / VR;
#pragma unroll
    for (int p = 0; p < LP; ++p) {
      const int b = bb + BP * p; // row block: input rows 4 b .. 4 b + 3
      if (kFull || (r0 + 4 * b < v.rows && c0 + cv * 4 < v.cols)) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          x[p][j] = load128<true>(reinterpret_cast<const u32x4 *>(in + (r0 + 4 * b + j) * v.ldIn + c0 + cv * 4));
      }
    }
  }
  __device__ __forceinline__ void store(uint32_t *__restrict__ out, const View &v, int64_t r0, int64_t c0, u32x4 *tile) {
    const int cv = threadIdx.x % VR, bb = threadIdx.x / VR;
#pragma unroll
    for (int p = 0; p < LP; ++p) {
      const int b = bb + BP * p;
      const int pos = b ^ (cv & 15); // (c / 4) % 16 is the same for the four columns of this vector
      tile[(cv * 4 + 0) * G + pos] = u32x4{x[p][0].x, x[p][1].x, x[p][2].x, x[p][3].x};
      tile[(cv * 4 + 1) * G + pos] = u32x4{x[p][0].y, x[p][1].y, x[p][2].y, x[p][3].y};
      tile[(cv * 4 + 2) * G + pos] = u32x4{x[p][0].z, x[p][1].z, x[p][2].z, x[p][3].z};
      tile[(cv * 4 + 3) * G + pos] = u32x4{x[p][0].w, x[p][1].w, x[p][2].w, x[p][3].w};
    }
    lds_barrier();
    constexpr int CP = kThreads / G, SP = C / CP; // store: output rows per pass, passes
    const int g = threadIdx.x % G, cc = threadIdx.x / G;
#pragma unroll
    for (int p = 0; p < SP; ++p) {
      const int c = cc + CP * p; // output row within the tile
      if (c0 + c < v.cols && r0 + g * 4 < v.rows)
        store128<true>(tile[c * G + (g ^ ((c >> 2) & 15))], reinterpret_cast<u32x4 *>(out + (c0 + c) * v.ldOut + r0 + g * 4));
    }
  }
};

// ---- 16-bit elements: R x 128 tile (or two of them side by side) ---------------------------
// The same scheme as the 32-bit tile with blocks of 8 x 8 elements: a lane loads eight consecutive rows
// (8 b .. 8 b + 7) at eight consecutive columns, one 128-bit load per row; for each of its eight columns it
// packs the eight row values into four words (v_perm_b32 on the words of two adjacent rows) and writes
// them as one 128-bit group of the transposed LDS image T[128 columns][R elements].  Output rows leave
// LDS as 128-bit reads.  Group g of LDS row c sits at position g ^ ((c / 8) % 16).
// kHalves = 2: the tile is R x 256; the loads of both 128-column halves are issued together (512-byte row
// segments on the read side as well), then each half takes its turn through the LDS image.
template <int R, int kHalves>
__device__ __forceinline__ void tile16_fast(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                            const View &v, int64_t r0, int64_t c0, u32x4 *tile) {
  constexpr int G = R / 8;               // 16-byte groups per LDS row
  constexpr int BP = kThreads / 16;      // row blocks per pass (16 column groups of 8 across 128 columns)
  constexpr int LP = G / BP;             // passes
  static_assert(G >= 16 && (G & (G - 1)) == 0 && LP >= 1, "the group swizzle needs at least 16 groups per row");
  const int cg = threadIdx.x % 16, bb = threadIdx.x / 16;
  u32x4 x[kHalves][LP][8];
#pragma unroll
  for (int p = 0; p < LP; ++p) {
    const int b = bb + BP * p; // input rows 8 b .. 8 b + 7
#pragma unroll
    for (int h = 0; h < kHalves; ++h)
      if (r0 + 8 * b < v.rows && c0 + h * 128 + cg * 8 < v.cols) {
        const uint16_t *src = in + (r0 + 8 * b) * v.ldIn + c0 + h * 128 + cg * 8;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          x[h][p][j] = load128<true>(reinterpret_cast<const u32x4 *>(src + j * v.ldIn));
      }
  }
  constexpr int CP = kThreads / G, SP = 128 / CP; // store: output rows per pass, passes
  const int g = threadIdx.x % G, cc = threadIdx.x / G;
#pragma unroll
  for (int h = 0; h < kHalves; ++h) {
    if (h > 0)
      __syncthreads(); // the previous half has left LDS
#pragma unroll
    for (int p = 0; p < LP; ++p) {
      const int pos = (bb + BP * p) ^ cg; // (c / 8) % 16 = cg for this lane's eight columns
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        // column 2 m of the group: the low halves of word m of each row; column 2 m + 1: the high halves
        u32x4 lo, hi;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          lo[q] = __builtin_amdgcn_perm(x[h][p][2 * q + 1][m], x[h][p][2 * q][m], 0x05040100u);
          hi[q] = __builtin_amdgcn_perm(x[h][p][2 * q + 1][m], x[h][p][2 * q][m], 0x07060302u);
        }
        tile[(cg * 8 + 2 * m) * G + pos] = lo;
        tile[(cg * 8 + 2 * m + 1) * G + pos] = hi;
      }
    }
    __syncthreads();
#pragma unroll
    for (int p = 0; p < SP; ++p) {
      const int c = cc + CP * p; // output row within this half
      if (c0 + h * 128 + c < v.cols && r0 + g * 8 < v.rows)
        store128<true>(tile[c * G + (g ^ ((c >> 3) & 15))],
                       reinterpret_cast<u32x4 *>(out + (c0 + h * 128 + c) * v.ldOut + r0 + g * 8));
    }
  }
}

// ---- 16-bit elements, whole 256 x 256 tiles: the tile goes through LDS a quarter at a time ------------
// A copy with this kernel's memory traffic reaches 4 points more of the HBM peak when every row segment is
// written out as soon as it has arrived than when a workgroup first waits for its whole tile (measured:
// 71.7 % against 67.7 % on 8192 x 8192).  A transpose cannot write anything before 256 input rows are there,
// but it need not wait for all 256 columns: the 32 loads of a lane are issued together, quarter by quarter
// (64 columns = one 8 x 8 block per lane and quarter), and each quarter is repacked, staged and written out
// while the later quarters are still arriving.  Two 32 KiB LDS images take the quarters in turn, so one
// barrier per quarter is enough: when a wavefront writes quarter q + 2 into an image, every wavefront has
// passed the barrier of quarter q + 1 and with it its last read of quarter q.  Loads and stores are
// unconditional straight-line code, so the waits are exact counts ("all but the 24, 16, 8 youngest").
// LDS image T[64 columns][256 rows]: group g (eight rows) of column c at position g ^ (c / 8).  A 128-bit LDS
// write is served eight consecutive lanes at a time over 128 bytes of banks: those eight lanes are the eight
// column blocks of one row block, whose positions differ in their low three bits.  A 128-bit read is served
// sixteen lanes at a time over 256 bytes of banks: one output row's groups, sixteen different positions.
__device__ __forceinline__ void tile16_quarters(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                                const View &v, int64_t r0, int64_t c0, u32x4 *lds) {
  constexpr int G = 32;            // 16-byte groups per LDS row (256 rows of the tile)
  constexpr int kImage = 64 * G;   // groups per quarter image: 32 KiB
  const int cg = threadIdx.x % 8, b = threadIdx.x / 8; // load side: column group within the quarter, row block
  const int g = threadIdx.x % G, cc = threadIdx.x / G;  // store side: group within the output row, output row
  u32x4 x[4][8];
  const uint16_t *src = in + (r0 + 8 * b) * v.ldIn + c0 + cg * 8;
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int j = 0; j < 8; ++j)
      x[q][j] = load128<true>(reinterpret_cast<const u32x4 *>(src + j * v.ldIn + q * 64));
  const int pos = b ^ cg;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    u32x4 *img = lds + (q & 1) * kImage;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      // column 2 m of the block: the low halves of word m of each row; column 2 m + 1: the high halves
      u32x4 lo, hi;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        lo[k] = __builtin_amdgcn_perm(x[q][2 * k + 1][m], x[q][2 * k][m], 0x05040100u);
        hi[k] = __builtin_amdgcn_perm(x[q][2 * k + 1][m], x[q][2 * k][m], 0x07060302u);
      }
      img[(cg * 8 + 2 * m) * G + pos] = lo;
      img[(cg * 8 + 2 * m + 1) * G + pos] = hi;
    }
    lds_barrier();
    u32x4 y[8];
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const int c = cc + 8 * p; // output row within the quarter
      y[p] = img[c * G + (g ^ (c >> 3))];
    }
#pragma unroll
    for (int p = 0; p < 8; ++p)
      store128<true>(y[p], reinterpret_cast<u32x4 *>(out + (c0 + q * 64 + cc + 8 * p) * v.ldOut + r0 + g * 8));
  }
}

// ---- any shape / alignment ------------------------------------------------------
template <typename T, int kTile>
__device__ __forceinline__ void tile_scalar(const T *__restrict__ in, T *__restrict__ out, const View &v,
                                            int64_t r0, int64_t c0, T (*tile)[kTile + 1]) {
  const int tx = threadIdx.x % kTile;
  const int ty = threadIdx.x / kTile;
  for (int r = ty; r < kTile; r += kThreads / kTile)
    if (r0 + r < v.rows && c0 + tx < v.cols)
      tile[r][tx] = in[(r0 + r) * v.ldIn + c0 + tx];
  __syncthreads();
  for (int c = ty; c < kTile; c += kThreads / kTile)
    if (c0 + c < v.cols && r0 + tx < v.rows)
      out[(c0 + c) * v.ldOut + r0 + tx] = tile[tx][c];
}

// Walks tiles id, id + (number of workgroups), ... of a (planes x tilesY x tilesX)
// grid, diagonal-major inside a plane: id -> tile row id % tilesY, diagonal
// k = id / tilesY, tile column (row + k) % tilesX.  One diagonal holds every tile
// row once, so the ~1000 workgroups in flight spread BOTH the reads (strided by
// the input pitch) and the writes (strided by the output pitch) over all tile
// rows and tile columns, i.e. over all memory channels.  A row-major walk keeps
// the in-flight writes inside a few tile columns of the output (57% of HBM peak
// against 69% for this order, 8192 x 8192 bf16 with 128 x 128 tiles).
template <int R, int C, typename Body>
__device__ __forceinline__ void for_each_tile(const View &v, int64_t planes, Body body) {
  const int64_t tilesX = (v.cols + C - 1) / C, tilesY = (v.rows + R - 1) / R;
  const int64_t perPlane = tilesX * tilesY, total = perPlane * planes;
  const int64_t first = (int64_t(blockIdx.z) * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
  const int64_t stride = int64_t(gridDim.x) * gridDim.y * gridDim.z;
  for (int64_t t = first; t < total; t += stride) {
    const int64_t plane = t / perPlane, rem = t % perPlane;
    const int64_t ty = rem % tilesY;
    const int64_t tx = (ty + rem / tilesY) % tilesX;
    body(plane, ty * R, tx * C);
    __syncthreads(); // the tile has left LDS before the next one is staged
  }
}

// The pipelined walk: the loads of a workgroup's next tile are issued before the current tile goes through LDS
// and out, so a workgroup always has a tile's reads in flight.  Tiles that lie wholly inside the matrix only
// (the caller checks that every tile does).
template <int R, int C, typename Tile, typename T>
__device__ __forceinline__ void pipelined_tiles(const T *in, T *out, const View &v, int64_t planes, int64_t inPlane,
                                                int64_t outPlane, u32x4 *lds) {
  const int64_t tilesX = v.cols / C, tilesY = v.rows / R;
  const int64_t perPlane = tilesX * tilesY, total = perPlane * planes;
  const int64_t first = (int64_t(blockIdx.z) * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
  const int64_t stride = int64_t(gridDim.x) * gridDim.y * gridDim.z;
  struct Where { int64_t plane, r0, c0; };
  auto where = [&](int64_t t) {
    const int64_t plane = t / perPlane, rem = t % perPlane;
    const int64_t ty = rem % tilesY;
    const int64_t tx = (ty + rem / tilesY) % tilesX;
    return Where{plane, ty * R, tx * C};
  };
  if (first >= total)
    return;
  Tile a, b;
  Where wa = where(first), wb = wa;
  a.template load<true>(in + wa.plane * inPlane, v, wa.r0, wa.c0);
  for (int64_t t = first;;) {
    // a holds tile t
    if (t + stride < total) {
      wb = where(t + stride);
      b.template load<true>(in + wb.plane * inPlane, v, wb.r0, wb.c0);
      a.store(out + wa.plane * outPlane, v, wa.r0, wa.c0, lds);
      lds_barrier();
    } else {
      a.store(out + wa.plane * outPlane, v, wa.r0, wa.c0, lds);
      return;
    }
    t += stride;
    // b holds tile t
    if (t + stride < total) {
      wa = where(t + stride);
      a.template load<true>(in + wa.plane * inPlane, v, wa.r0, wa.c0);
      b.store(out + wb.plane * outPlane, v, wb.r0, wb.c0, lds);
      lds_barrier();
    } else {
      b.store(out + wb.plane * outPlane, v, wb.r0, wb.c0, lds);
      return;
    }
    t += stride;
  }
}

// planes: number of 2-D problems (1, or d1 for the 3-D reversal) with element
// strides inPlane / outPlane between them.
template <typename T>
__device__ __forceinline__ void transpose_block(const T *in, T *out, const View &v, int64_t planes, int64_t inPlane,
                                                int64_t outPlane) {
  constexpr int kVec = 16 / sizeof(T);
  // 32-bit: 128 x 128 words.  16-bit: 128 rows x 128 words.  The scalar path's 64 x 65 elements fit as well.
  constexpr int kLdsBytes = 128 * 128 * 4;
  __shared__ __attribute__((aligned(16))) char lds[kLdsBytes];
  const bool fast = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 &&
                    v.rows % kVec == 0 && v.cols % kVec == 0 && v.ldIn % kVec == 0 && v.ldOut % kVec == 0 &&
                    inPlane % kVec == 0 && outPlane % kVec == 0;
  const bool big = v.rows * v.cols * planes >= kBigProblem;
  if (!fast) {
    for_each_tile<64, 64>(v, planes, [&](int64_t plane, int64_t r0, int64_t c0) {
      tile_scalar<T, 64>(in + plane * inPlane, out + plane * outPlane, v, r0, c0, reinterpret_cast<T(*)[65]>(lds));
    });
  } else if constexpr (sizeof(T) == 4) {
    if (big && v.rows % 128 == 0 && v.cols % 128 == 0)
      pipelined_tiles<128, 128, Tile32<128, 128>>(in, out, v, planes, inPlane, outPlane, reinterpret_cast<u32x4 *>(lds));
    else if (big)
      for_each_tile<128, 128>(v, planes, [&](int64_t plane, int64_t r0, int64_t c0) {
        Tile32<128, 128> t;
        t.template load<false>(in + plane * inPlane, v, r0, c0);
        t.store(out + plane * outPlane, v, r0, c0, reinterpret_cast<u32x4 *>(lds));
      });
    else
      for_each_tile<64, 64>(v, planes, [&](int64_t plane, int64_t r0, int64_t c0) {
        Tile32<64, 64> t;
        t.template load<false>(in + plane * inPlane, v, r0, c0);
        t.store(out + plane * outPlane, v, r0, c0, reinterpret_cast<u32x4 *>(lds));
      });
  } else {
    if (big && v.rows % 256 == 0 && v.cols % 256 == 0)
      for_each_tile<256, 256>(v, planes, [&](int64_t plane, int64_t r0, int64_t c0) {
        tile16_quarters(in + plane * inPlane, out + plane * outPlane, v, r0, c0, reinterpret_cast<u32x4 *>(lds));
      });
    else if (big)
      for_each_tile<256, 256>(v, planes, [&](int64_t plane, int64_t r0, int64_t c0) {
        tile16_fast<256, 2>(in + plane * inPlane, out + plane * outPlane, v, r0, c0, reinterpret_cast<u32x4 *>(lds));
      });
    else
      for_each_tile<128, 128>(v, planes, [&](int64_t plane, int64_t r0, int64_t c0) {
        tile16_fast<128, 1>(in + plane * inPlane, out + plane * outPlane, v, r0, c0, reinterpret_cast<u32x4 *>(lds));
      });
  }
}

} // namespace

extern "C" __global__ __launch_bounds__(kThreads) void imex_transpose2d_b32(const uint32_t *in, uint32_t *out,
                                                                           int64_t rows, int64_t cols) {
  transpose_block<uint32_t>(in, out, View{rows, cols, cols, rows}, 1, 0, 0);
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_transpose2d_b16(const uint16_t *in, uint16_t *out,
                                                                           int64_t rows, int64_t cols) {
  transpose_block<uint16_t>(in, out, View{rows, cols, cols, rows}, 1, 0, 0);
}

// out[k, j, i] = in[i, j, k]: for each j (blockIdx.z) a 2-D transpose of the
// (i, k) plane with leading dimensions d1*d2 (in) and d1*d0 (out).
extern "C" __global__ __launch_bounds__(kThreads) void imex_transpose3d_b32(const uint32_t *in, uint32_t *out,
                                                                           int64_t d0, int64_t d1, int64_t d2) {
  transpose_block<uint32_t>(in, out, View{d0, d2, d1 * d2, d1 * d0}, d1, d2, d0);
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_transpose3d_b16(const uint16_t *in, uint16_t *out,
                                                                           int64_t d0, int64_t d1, int64_t d2) {
  transpose_block<uint16_t>(in, out, View{d0, d2, d1 * d2, d1 * d0}, d1, d2, d0);
}
