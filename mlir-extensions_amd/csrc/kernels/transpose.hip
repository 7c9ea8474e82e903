// 2-D transpose (and the 3-D full reversal built from it), 16- and 32-bit
// elements, bit-exact moves.
//
// Reference: benchmarks/transpose/transpose2d_gpu.mlir.in:4-11 (out[j,i] = in[i,j])
// and transpose3d_gpu.mlir.in:4-11 (out[k,j,i] = in[i,j,k]); the reference's
// generated kernel moves one element per work-group
// (test/SPIRV/OpTest.Transpose_FLOAT32.mlir:55-57).
//
// Here a workgroup moves a 64x64 tile through LDS so that both the HBM reads
// and the HBM writes are 128-bit and row-contiguous:
//  * 32-bit: tile[64][65] words; the odd pitch makes the row-wise scalar LDS
//    writes and the column-wise scalar LDS reads both conflict-free.
//  * 16-bit: two vertically adjacent rows are interleaved in registers into
//    32-bit words (in[2p][c], in[2p+1][c]) -- two neighbouring elements of
//    output row c -- and stored transposed; output rows then leave LDS as
//    128-bit reads.  The 16-byte groups of each LDS row are XOR-swizzled with
//    the column group so neither side has bank conflicts.
// Shapes or bases that break 16-byte alignment use the scalar tile path of the
// same kernel.
//
// Arguments: 2-D (in, out, rows: i64, cols: i64); 3-D (in, out, d0, d1, d2: i64).
// Launch: block (256,1,1); grid 2-D (ceil(cols/64), ceil(rows/64), 1);
//         3-D (ceil(d2/64), ceil(d0/64), d1).

#include "device_common.h"

using namespace imexhip;

namespace {

constexpr int kThreads = 256;
constexpr int kTile = 64;

// in element (i, j) lives at in[i * ldIn + j]; it goes to out[j * ldOut + i].
struct View {
  int64_t rows, cols, ldIn, ldOut;
};

// ---- 32-bit elements ----------------------------------------------------------
__device__ __forceinline__ void tile32_fast(const uint32_t *__restrict__ in, uint32_t *__restrict__ out,
                                            const View &v, int64_t r0, int64_t c0, uint32_t (*tile)[kTile + 1]) {
  const int cv = threadIdx.x % 16; // 16-byte vector within a 64-element row
  const int rr = threadIdx.x / 16; // 16 rows per pass
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int r = rr + 16 * pass;
    if (r0 + r < v.rows && c0 + cv * 4 < v.cols) {
      u32x4 x = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(in + (r0 + r) * v.ldIn + c0 + cv * 4));
      tile[r][cv * 4 + 0] = x.x;
      tile[r][cv * 4 + 1] = x.y;
      tile[r][cv * 4 + 2] = x.z;
      tile[r][cv * 4 + 3] = x.w;
    }
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int c = rr + 16 * pass; // output row within the tile
    const int iv = cv;            // 4 input rows -> one output vector
    if (c0 + c < v.cols && r0 + iv * 4 < v.rows) {
      u32x4 y = {tile[iv * 4 + 0][c], tile[iv * 4 + 1][c], tile[iv * 4 + 2][c], tile[iv * 4 + 3][c]};
      __builtin_nontemporal_store(y, reinterpret_cast<u32x4 *>(out + (c0 + c) * v.ldOut + r0 + iv * 4));
    }
  }
}

// ---- 16-bit elements ----------------------------------------------------------
__device__ __forceinline__ int swz16(int col, int rowPair) {
  // word index of (output row `col`, row pair `rowPair`) in the LDS image
  return col * 32 + ((((rowPair >> 2) ^ (col >> 3)) & 7) << 2) + (rowPair & 3);
}

__device__ __forceinline__ void tile16_fast(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                            const View &v, int64_t r0, int64_t c0, uint32_t *words) {
  {
    const int cg = threadIdx.x % 8; // 8-element column group
    const int rp = threadIdx.x / 8; // row pair 0..31
    if (r0 + 2 * rp < v.rows && c0 + cg * 8 < v.cols) {
      const uint16_t *p = in + (r0 + 2 * rp) * v.ldIn + c0 + cg * 8;
      u32x4 a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
      u32x4 b = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p + v.ldIn));
      const uint32_t aw[4] = {a.x, a.y, a.z, a.w};
      const uint32_t bw[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        // even column: low halves of both rows; odd column: high halves
        words[swz16(cg * 8 + 2 * k, rp)] = (aw[k] & 0xffffu) | (bw[k] << 16);
        words[swz16(cg * 8 + 2 * k + 1, rp)] = (aw[k] >> 16) | (bw[k] & 0xffff0000u);
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int g = threadIdx.x % 8;             // 8 consecutive input rows
    const int c = threadIdx.x / 8 + 32 * pass; // output row within the tile
    if (c0 + c < v.cols && r0 + g * 8 < v.rows) {
      u32x4 y = *reinterpret_cast<const u32x4 *>(words + swz16(c, g * 4));
      __builtin_nontemporal_store(y, reinterpret_cast<u32x4 *>(out + (c0 + c) * v.ldOut + r0 + g * 8));
    }
  }
}

// ---- any shape / alignment ------------------------------------------------------
template <typename T>
__device__ __forceinline__ void tile_scalar(const T *__restrict__ in, T *__restrict__ out, const View &v,
                                            int64_t r0, int64_t c0, T (*tile)[kTile + 1]) {
  const int tx = threadIdx.x % kTile;
  const int ty = threadIdx.x / kTile; // 4 rows per pass
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
  __shared__ __attribute__((aligned(16))) uint32_t lds[kTile * (kTile + 1)];
  const int64_t r0 = int64_t(blockIdx.y) * kTile;
  const int64_t c0 = int64_t(blockIdx.x) * kTile;
  const bool fast = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0 &&
                    v.rows % kVec == 0 && v.cols % kVec == 0 && v.ldIn % kVec == 0 && v.ldOut % kVec == 0;
  if constexpr (sizeof(T) == 4) {
    if (fast)
      tile32_fast(in, out, v, r0, c0, reinterpret_cast<uint32_t(*)[kTile + 1]>(lds));
    else
      tile_scalar<uint32_t>(in, out, v, r0, c0, reinterpret_cast<uint32_t(*)[kTile + 1]>(lds));
  } else {
    if (fast)
      tile16_fast(in, out, v, r0, c0, lds);
    else
      tile_scalar<uint16_t>(in, out, v, r0, c0, reinterpret_cast<uint16_t(*)[kTile + 1]>(lds));
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
