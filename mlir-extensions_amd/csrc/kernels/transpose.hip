// 2-D transpose (and the 3-D full reversal built from it), 16- and 32-bit
// elements, bit-exact moves.
//
// Reference: benchmarks/transpose/transpose2d_gpu.mlir.in:4-11 (out[j,i] = in[i,j])
// and transpose3d_gpu.mlir.in:4-11 (out[k,j,i] = in[i,j,k]); the reference's
// generated kernel moves one element per work-group
// (test/SPIRV/OpTest.Transpose_FLOAT32.mlir:55-57).
//
// Here a workgroup moves a tile through LDS so that both the HBM reads and the
// HBM writes are 128-bit per lane and 256 B contiguous per row segment:
//  * 32-bit: 64 x 64 tile, tile[64][65] words; the odd pitch makes the row-wise
//    scalar LDS writes and the column-wise scalar LDS reads conflict-free.
//  * 16-bit: 128 x 128 tile.  Two vertically adjacent rows are interleaved in
//    registers into 32-bit words (in[2p][c], in[2p+1][c]) -- two neighbouring
//    elements of output row c -- and stored transposed; output rows then leave
//    LDS as 128-bit reads.  The 16-byte groups of each LDS row are XOR-swizzled
//    with the column group so neither side has bank conflicts.
//  * Workgroups walk the tile grid diagonal by diagonal, so that the workgroups
//    in flight together cover every tile row AND every tile column: both strided
//    sides of the transpose are spread over all memory channels.
//  * Loads and stores are non-temporal: each byte is touched once, and keeping
//    the streams out of the caches is what holds up when the tensors are not
//    already cache-resident (69% of HBM peak streaming from memory, 65% right
//    after a cache flush; cached accesses are faster only when the same buffers
//    are transposed again and again inside the 256 MiB Infinity Cache).
// Shapes or bases that break 16-byte alignment use the scalar tile path of the
// same kernel.
//
// Arguments: 2-D (in, out, rows: i64, cols: i64); 3-D (in, out, d0, d1, d2: i64).
// Launch: block (256,1,1); tile T = 64 (32-bit) or 128 (16-bit);
//         grid 2-D (ceil(cols/T), ceil(rows/T), 1); 3-D (ceil(d2/T), ceil(d0/T), d1).

#include "device_common.h"

using namespace imexhip;

namespace {

constexpr int kThreads = 256;
constexpr int kTile32 = 64;
constexpr int kTile16 = 128;

// in element (i, j) lives at in[i * ldIn + j]; it goes to out[j * ldOut + i].
struct View {
  int64_t rows, cols, ldIn, ldOut;
};

// Diagonal-major walk over the tile grid.  Workgroup ids run down a diagonal
// first: id -> tile row id % ny, diagonal k = id / ny, tile column (row + k) % nx.
// One diagonal holds every tile row once and (for nx >= ny) distinct tile
// columns, so the ~1000 workgroups in flight at any moment spread BOTH the reads
// (strided by the input pitch) and the writes (strided by the output pitch) over
// all tile rows and tile columns, i.e. over all memory channels.  A row-major
// walk keeps the in-flight writes inside a few tile columns of the output, which
// measured 57% of HBM peak against 69% for this order (8192 x 8192 bf16).
__device__ __forceinline__ void tile_coords(int &tx, int &ty) {
  const int lin = blockIdx.y * gridDim.x + blockIdx.x;
  ty = lin % gridDim.y;
  tx = (ty + lin / gridDim.y) % gridDim.x;
}

// ---- 32-bit elements ----------------------------------------------------------
template <bool kStream>
__device__ __forceinline__ void tile32_fast(const uint32_t *__restrict__ in, uint32_t *__restrict__ out,
                                            const View &v, int64_t r0, int64_t c0, uint32_t (*tile)[kTile32 + 1]) {
  const int cv = threadIdx.x % 16; // 16-byte vector within a 64-element row
  const int rr = threadIdx.x / 16; // 16 rows per pass
  u32x4 x[4];
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int r = rr + 16 * pass;
    if (r0 + r < v.rows && c0 + cv * 4 < v.cols)
      x[pass] = load128<kStream>(reinterpret_cast<const u32x4 *>(in + (r0 + r) * v.ldIn + c0 + cv * 4));
  }
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int r = rr + 16 * pass;
    tile[r][cv * 4 + 0] = x[pass].x;
    tile[r][cv * 4 + 1] = x[pass].y;
    tile[r][cv * 4 + 2] = x[pass].z;
    tile[r][cv * 4 + 3] = x[pass].w;
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int c = rr + 16 * pass; // output row within the tile
    const int iv = cv;            // 4 input rows -> one output vector
    if (c0 + c < v.cols && r0 + iv * 4 < v.rows) {
      u32x4 y = {tile[iv * 4 + 0][c], tile[iv * 4 + 1][c], tile[iv * 4 + 2][c], tile[iv * 4 + 3][c]};
      store128<kStream>(y, reinterpret_cast<u32x4 *>(out + (c0 + c) * v.ldOut + r0 + iv * 4));
    }
  }
}

// ---- 16-bit elements ----------------------------------------------------------
// LDS image: [128 output rows][64 words]; word w of output row c holds input
// rows 2w, 2w+1 at column c.  16-byte group g of row c is stored at group
// g ^ (c/8 mod 16).
__device__ __forceinline__ int swz16(int col, int rowPair) {
  return col * 64 + ((((rowPair >> 2) ^ (col >> 3)) & 15) << 2) + (rowPair & 3);
}

template <bool kStream>
__device__ __forceinline__ void tile16_fast(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                            const View &v, int64_t r0, int64_t c0, uint32_t *words) {
  const int cg = threadIdx.x % 16; // 8-element column group
  const int rq = threadIdx.x / 16; // row pair within a pass (16 per pass)
  u32x4 a[4], b[4];
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int rp = rq + 16 * pass;
    if (r0 + 2 * rp < v.rows && c0 + cg * 8 < v.cols) {
      const uint16_t *p = in + (r0 + 2 * rp) * v.ldIn + c0 + cg * 8;
      a[pass] = load128<kStream>(reinterpret_cast<const u32x4 *>(p));
      b[pass] = load128<kStream>(reinterpret_cast<const u32x4 *>(p + v.ldIn));
    }
  }
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int rp = rq + 16 * pass;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      // even column: low halves of both rows; odd column: high halves
      words[swz16(cg * 8 + 2 * k, rp)] = __builtin_amdgcn_perm(b[pass][k], a[pass][k], 0x05040100u);
      words[swz16(cg * 8 + 2 * k + 1, rp)] = __builtin_amdgcn_perm(b[pass][k], a[pass][k], 0x07060302u);
    }
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 8; ++pass) {
    const int g = threadIdx.x % 16;            // 8 consecutive input rows
    const int c = threadIdx.x / 16 + 16 * pass; // output row within the tile
    if (c0 + c < v.cols && r0 + g * 8 < v.rows) {
      u32x4 y = *reinterpret_cast<const u32x4 *>(words + swz16(c, g * 4));
      store128<kStream>(y, reinterpret_cast<u32x4 *>(out + (c0 + c) * v.ldOut + r0 + g * 8));
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

template <typename T> __device__ __forceinline__ void transpose_block(const T *in, T *out, const View &v) {
  constexpr int kVec = 16 / sizeof(T);
  constexpr int kTile = sizeof(T) == 4 ? kTile32 : kTile16;
  // 32-bit: 64 x 65 words = 16640 B.  16-bit: 128 x 64 words = 32768 B (fast path),
  // 128 x 129 halfwords = 33024 B (scalar path).
  constexpr int kLdsBytes = sizeof(T) == 4 ? kTile32 * (kTile32 + 1) * 4 : kTile16 * (kTile16 + 1) * 2;
  __shared__ __attribute__((aligned(16))) char lds[kLdsBytes];
  int tx, ty;
  tile_coords(tx, ty);
  const int64_t r0 = int64_t(ty) * kTile;
  const int64_t c0 = int64_t(tx) * kTile;
  const bool fast = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 &&
                    v.rows % kVec == 0 && v.cols % kVec == 0 && v.ldIn % kVec == 0 && v.ldOut % kVec == 0;
  if constexpr (sizeof(T) == 4) {
    if (fast)
      tile32_fast<true>(in, out, v, r0, c0, reinterpret_cast<uint32_t(*)[kTile32 + 1]>(lds));
    else
      tile_scalar<uint32_t, kTile32>(in, out, v, r0, c0, reinterpret_cast<uint32_t(*)[kTile32 + 1]>(lds));
  } else {
    if (fast)
      tile16_fast<true>(in, out, v, r0, c0, reinterpret_cast<uint32_t *>(lds));
    else
      tile_scalar<uint16_t, kTile16>(in, out, v, r0, c0, reinterpret_cast<uint16_t(*)[kTile16 + 1]>(lds));
  }
}

} // namespace

extern "C" __global__ __launch_bounds__(kThreads) void imex_transpose2d_b32(const uint32_t *in, uint32_t *out,
                                                                           int64_t rows, int64_t cols) {
  transpose_block<uint32_t>(in, out, View{rows, cols, cols, rows});
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_transpose2d_b16(const uint16_t *in, uint16_t *out,
                                                                           int64_t rows, int64_t cols) {
  transpose_block<uint16_t>(in, out, View{rows, cols, cols, rows});
}

// out[k, j, i] = in[i, j, k]: for each j (blockIdx.z) a 2-D transpose of the
// (i, k) plane with leading dimensions d1*d2 (in) and d1*d0 (out).
extern "C" __global__ __launch_bounds__(kThreads) void imex_transpose3d_b32(const uint32_t *in, uint32_t *out,
                                                                           int64_t d0, int64_t d1, int64_t d2) {
  const int64_t j = blockIdx.z;
  transpose_block<uint32_t>(in + j * d2, out + j * d0, View{d0, d2, d1 * d2, d1 * d0});
}

extern "C" __global__ __launch_bounds__(kThreads) void imex_transpose3d_b16(const uint16_t *in, uint16_t *out,
                                                                           int64_t d0, int64_t d1, int64_t d2) {
  const int64_t j = blockIdx.z;
  transpose_block<uint16_t>(in + j * d2, out + j * d0, View{d0, d2, d1 * d2, d1 * d0});
}
