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
//  * 32-bit: R x C tile in tile[R][C+1] words; the odd pitch makes the row-wise
//    scalar LDS writes and the column-wise scalar LDS reads conflict-free.
//  * 16-bit: R x 128 tile (or two of them side by side, loaded together).  Two
//    vertically adjacent rows are interleaved in
//    registers into 32-bit words (in[2p][c], in[2p+1][c]) -- two neighbouring
//    elements of output row c -- and stored transposed; output rows then leave
//    LDS as 128-bit reads.  The 16-byte groups of each LDS row are XOR-swizzled
//    with the column group so neither side has bank conflicts.
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
// Shapes or bases that break 16-byte alignment use the scalar 64 x 64 tile path
// of the same kernel.
//
// Arguments: 2-D (in, out, rows: i64, cols: i64); 3-D (in, out, d0, d1, d2: i64).
// Launch: block (256,1,1); one workgroup per tile, grid 2-D (ceil(cols/C),
// ceil(rows/R), 1), 3-D (ceil(d2/C), ceil(d0/R), d1) with (R, C) as above; any
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

// ---- 32-bit elements: R x C tile ----------------------------------------------------
template <int R, int C>
__device__ __forceinline__ void tile32_fast(const uint32_t *__restrict__ in, uint32_t *__restrict__ out,
                                            const View &v, int64_t r0, int64_t c0, uint32_t (*tile)[C + 1]) {
  constexpr int VR = C / 4, RP = kThreads / VR, LP = R / RP; // load: vectors per row, rows per pass, passes
  const int cv = threadIdx.x % VR, rr = threadIdx.x / VR;
  u32x4 x[LP];
#pragma unroll
  for (int p = 0; p < LP; ++p) {
    const int r = rr + RP * p;
    if (r0 + r < v.rows && c0 + cv * 4 < v.cols)
      x[p] = load128<true>(reinterpret_cast<const u32x4 *>(in + (r0 + r) * v.ldIn + c0 + cv * 4));
  }
#pragma unroll
  for (int p = 0; p < LP; ++p) {
    const int r = rr + RP * p;
    tile[r][cv * 4 + 0] = x[p].x;
    tile[r][cv * 4 + 1] = x[p].y;
    tile[r][cv * 4 + 2] = x[p].z;
    tile[r][cv * 4 + 3] = x[p].w;
  }
  __syncthreads();
  constexpr int VO = R / 4, CP = kThreads / VO, SP = C / CP; // store: vectors per output row, rows per pass, passes
  const int iv = threadIdx.x % VO, cc = threadIdx.x / VO;    // 4 input rows -> one output vector
#pragma unroll
  for (int p = 0; p < SP; ++p) {
    const int c = cc + CP * p; // output row within the tile
    if (c0 + c < v.cols && r0 + iv * 4 < v.rows) {
      u32x4 y = {tile[iv * 4 + 0][c], tile[iv * 4 + 1][c], tile[iv * 4 + 2][c], tile[iv * 4 + 3][c]};
      store128<true>(y, reinterpret_cast<u32x4 *>(out + (c0 + c) * v.ldOut + r0 + iv * 4));
    }
  }
}

// ---- 16-bit elements: R x 128 tile ------------------------------------------------------
// LDS image: [128 output rows][R/2 words]; word w of output row c holds input
// rows 2w, 2w+1 at column c.  16-byte group g of row c is stored at group
// g ^ (c/8).
template <int R> __device__ __forceinline__ int swz16(int col, int rowPair) {
  constexpr int W = R / 2; // words per output row
  return col * W + ((((rowPair >> 2) ^ (col >> 3)) & (W / 4 - 1)) << 2) + (rowPair & 3);
}

// kHalves = 2: the tile is R x 256; the loads of both 128-column halves are issued
// together (512-byte row segments on the read side as well), then each half takes
// its turn through the LDS image.
template <int R, int kHalves>
__device__ __forceinline__ void tile16_fast(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                            const View &v, int64_t r0, int64_t c0, uint32_t *words) {
  constexpr int LP = R / 32; // 16 row pairs per pass
  const int cg = threadIdx.x % 16; // 8-element column group
  const int rq = threadIdx.x / 16; // row pair within a pass
  u32x4 a[kHalves][LP], b[kHalves][LP];
#pragma unroll
  for (int pass = 0; pass < LP; ++pass) {
    const int rp = rq + 16 * pass;
#pragma unroll
    for (int h = 0; h < kHalves; ++h)
      if (r0 + 2 * rp < v.rows && c0 + h * 128 + cg * 8 < v.cols) {
        const uint16_t *p = in + (r0 + 2 * rp) * v.ldIn + c0 + h * 128 + cg * 8;
        a[h][pass] = load128<true>(reinterpret_cast<const u32x4 *>(p));
        b[h][pass] = load128<true>(reinterpret_cast<const u32x4 *>(p + v.ldIn));
      }
  }
  constexpr int VO = R / 8, CP = kThreads / VO, SP = 128 / CP; // vectors per output row, rows per pass, passes
  const int g = threadIdx.x % VO; // 8 consecutive input rows
#pragma unroll
  for (int h = 0; h < kHalves; ++h) {
    if (h > 0)
      __syncthreads(); // the previous half has left LDS
#pragma unroll
    for (int pass = 0; pass < LP; ++pass) {
      const int rp = rq + 16 * pass;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        // even column: low halves of both rows; odd column: high halves
        words[swz16<R>(cg * 8 + 2 * k, rp)] = __builtin_amdgcn_perm(b[h][pass][k], a[h][pass][k], 0x05040100u);
        words[swz16<R>(cg * 8 + 2 * k + 1, rp)] = __builtin_amdgcn_perm(b[h][pass][k], a[h][pass][k], 0x07060302u);
      }
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < SP; ++pass) {
      const int c = threadIdx.x / VO + CP * pass; // output row within this half
      if (c0 + h * 128 + c < v.cols && r0 + g * 8 < v.rows) {
        u32x4 y = *reinterpret_cast<const u32x4 *>(words + swz16<R>(c, g * 4));
        store128<true>(y, reinterpret_cast<u32x4 *>(out + (c0 + h * 128 + c) * v.ldOut + r0 + g * 8));
      }
    }
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

// planes: number of 2-D problems (1, or d1 for the 3-D reversal) with element
// strides inPlane / outPlane between them.
template <typename T>
__device__ __forceinline__ void transpose_block(const T *in, T *out, const View &v, int64_t planes, int64_t inPlane,
                                                int64_t outPlane) {
  constexpr int kVec = 16 / sizeof(T);
  // 32-bit: 128 x 129 words = 66048 B.  16-bit: 128 rows x 128 words = 65536 B.
  constexpr int kLdsBytes = sizeof(T) == 4 ? 128 * 129 * 4 : 128 * 128 * 4;
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
    if (big)
      for_each_tile<128, 128>(v, planes, [&](int64_t plane, int64_t r0, int64_t c0) {
        tile32_fast<128, 128>(in + plane * inPlane, out + plane * outPlane, v, r0, c0,
                              reinterpret_cast<uint32_t(*)[129]>(lds));
      });
    else
      for_each_tile<64, 64>(v, planes, [&](int64_t plane, int64_t r0, int64_t c0) {
        tile32_fast<64, 64>(in + plane * inPlane, out + plane * outPlane, v, r0, c0,
                            reinterpret_cast<uint32_t(*)[65]>(lds));
      });
  } else {
    if (big)
      for_each_tile<256, 256>(v, planes, [&](int64_t plane, int64_t r0, int64_t c0) {
        tile16_fast<256, 2>(in + plane * inPlane, out + plane * outPlane, v, r0, c0, reinterpret_cast<uint32_t *>(lds));
      });
    else
      for_each_tile<128, 128>(v, planes, [&](int64_t plane, int64_t r0, int64_t c0) {
        tile16_fast<128, 1>(in + plane * inPlane, out + plane * outPlane, v, r0, c0, reinterpret_cast<uint32_t *>(lds));
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
