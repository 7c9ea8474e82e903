//===- KernelCatalog.cpp - embedded gfx950 code objects + launch shapes ----===//
//
// Host-side table of the hand-written kernels: which embedded code object
// holds each one and the grid/block it is launched with.  This plays the part
// of the `gpu.binary` blob plus the `blocks in (...) threads in (...)` operands
// that IMEX's lowering bakes into host code
// (lib/Conversion/GPUXToLLVM/GPUXToLLVMPass.cpp:456-713).
//
//===----------------------------------------------------------------------===//

#include "imex_hip_kernels.h"

#include <algorithm>
#include <cstring>

// Blob symbols come from the assembler stub generated at build time
// (one .incbin per code object).
extern "C" {
extern const unsigned char imex_blob_eltwise[], imex_blob_eltwise_end[];
extern const unsigned char imex_blob_softmax[], imex_blob_softmax_end[];
extern const unsigned char imex_blob_reduce[], imex_blob_reduce_end[];
extern const unsigned char imex_blob_transpose[], imex_blob_transpose_end[];
extern const unsigned char imex_blob_gemm[], imex_blob_gemm_end[];
extern const unsigned char imex_blob_fusion[], imex_blob_fusion_end[];
extern const unsigned char imex_blob_attention[], imex_blob_attention_end[];
}

namespace {

enum class Module { Eltwise, Softmax, Reduce, Transpose, Gemm, Fusion, Attention };
enum class Shape { Eltwise32, Eltwise16, Fusion32, Fusion16, SoftmaxRows32, SoftmaxRows16, RowSum, ReduceOuter, ReduceOuter16, Transpose2D32, Transpose2D16, Transpose3D32, Transpose3D16, Gemm, GemmStreamK, GemmTA, GemmTB, GemmFixed4k, ColumnThreads, ColumnThreads16, Attention };

struct Entry {
  const char *name;
  const char *signature;
  Module module;
  Shape shape;
  int ndims;
};

const Entry kEntries[] = {
    {"imex_relu_f32", "(in: f32*, out: f32*, n: i64)", Module::Eltwise, Shape::Eltwise32, 1},
    {"imex_relu_f16", "(in: f16*, out: f16*, n: i64)", Module::Eltwise, Shape::Eltwise16, 1},
    {"imex_relu_bf16", "(in: bf16*, out: bf16*, n: i64)", Module::Eltwise, Shape::Eltwise16, 1},
    {"imex_silu_f32", "(in: f32*, out: f32*, n: i64)", Module::Eltwise, Shape::Fusion32, 1},
    {"imex_silu_f16", "(in: f16*, out: f16*, n: i64)", Module::Eltwise, Shape::Fusion16, 1},
    {"imex_silu_bf16", "(in: bf16*, out: bf16*, n: i64)", Module::Eltwise, Shape::Fusion16, 1},
    {"imex_exp_f32", "(in: f32*, out: f32*, n: i64)", Module::Eltwise, Shape::Fusion32, 1},
    {"imex_maximum_f32", "(a: f32*, b: f32*, out: f32*, n: i64)", Module::Eltwise, Shape::Eltwise32, 1},
    {"imex_softmax_f32", "(in: f32*, out: f32*, rows: i64, cols: i64)", Module::Softmax, Shape::SoftmaxRows32, 2},
    {"imex_softmax_f16", "(in: f16*, out: f16*, rows: i64, cols: i64)", Module::Softmax, Shape::SoftmaxRows16, 2},
    {"imex_softmax_bf16", "(in: bf16*, out: bf16*, rows: i64, cols: i64)", Module::Softmax, Shape::SoftmaxRows16, 2},
    {"imex_rowsum_f32", "(in: f32*, out: f32*, rows: i64, cols: i64, init: f32)", Module::Reduce, Shape::RowSum, 2},
    {"imex_rowmean_f32", "(in: f32*, out: f32*, rows: i64, cols: i64)", Module::Reduce, Shape::RowSum, 2},
    {"imex_reduce_outer_f32", "(in: f32*, out: f32*, outer: i64, inner: i64, init: f32)", Module::Reduce,
     Shape::ReduceOuter, 2},
    {"imex_reduce_outer_f16", "(in: f16*, out: f16*, outer: i64, inner: i64, init: f32)", Module::Reduce,
     Shape::ReduceOuter16, 2},
    {"imex_reduce_outer_bf16", "(in: bf16*, out: bf16*, outer: i64, inner: i64, init: f32)", Module::Reduce,
     Shape::ReduceOuter16, 2},
    {"imex_transpose2d_b32", "(in: b32*, out: b32*, rows: i64, cols: i64)", Module::Transpose, Shape::Transpose2D32, 2},
    {"imex_transpose2d_b16", "(in: b16*, out: b16*, rows: i64, cols: i64)", Module::Transpose, Shape::Transpose2D16, 2},
    {"imex_transpose3d_b32", "(in: b32*, out: b32*, d0: i64, d1: i64, d2: i64)", Module::Transpose,
     Shape::Transpose3D32, 3},
    {"imex_transpose3d_b16", "(in: b16*, out: b16*, d0: i64, d1: i64, d2: i64)", Module::Transpose,
     Shape::Transpose3D16, 3},
    {"imex_loop_fusion_f32", "(a: f32*, b: f32*, out: f32*, n: i64)", Module::Fusion, Shape::Fusion32, 1},
    {"imex_loop_fusion_f16", "(a: f16*, b: f16*, out: f16*, n: i64)", Module::Fusion, Shape::Fusion16, 1},
    {"imex_loop_fusion_bf16", "(a: bf16*, b: bf16*, out: bf16*, n: i64)", Module::Fusion, Shape::Fusion16, 1},
    {"imex_input_fusion_f32", "(a: f32*, b: f32*, out: f32*, rows: i64, cols: i64)", Module::Fusion,
     Shape::ColumnThreads, 2},
    {"imex_input_fusion_f16", "(a: f16*, b: f16*, out: f16*, rows: i64, cols: i64)", Module::Fusion,
     Shape::ColumnThreads16, 2},
    {"imex_input_fusion_bf16", "(a: bf16*, b: bf16*, out: bf16*, rows: i64, cols: i64)", Module::Fusion,
     Shape::ColumnThreads16, 2},
    {"imex_flash_attention_fwd_f16",
     "(Q: f16*, K: f16*, V: f16*, Out: f16*, sm_scale: f32, ZH: i64, N_CTX: i64)", Module::Attention,
     Shape::Attention, 2},
    {"imex_gemm_f16_f16_f32", "(A: f16*, B: f16*, C: f32*, M: i64, N: i64, K: i64)", Module::Gemm, Shape::Gemm, 3},
    {"imex_gemm_f16_f16_f32_acc", "(A: f16*, B: f16*, C: f32*, M: i64, N: i64, K: i64)", Module::Gemm, Shape::Gemm, 3},
    {"imex_gemm_bf16_bf16_f32", "(A: bf16*, B: bf16*, C: f32*, M: i64, N: i64, K: i64)", Module::Gemm, Shape::Gemm, 3},
    {"imex_gemm_bf16_bf16_f32_acc", "(A: bf16*, B: bf16*, C: f32*, M: i64, N: i64, K: i64)", Module::Gemm,
     Shape::Gemm, 3},
    {"imex_gemm_f16_f16_f16", "(A: f16*, B: f16*, C: f16*, M: i64, N: i64, K: i64)", Module::Gemm, Shape::Gemm, 3},
    {"imex_gemm_bf16_bias_silu_bf16", "(A: bf16*, B: bf16*, bias: f32*, out: bf16*, M: i64, N: i64, K: i64)",
     Module::Gemm, Shape::Gemm, 3},
    {"imex_gemm_bf16_bias_silu_bf16_streamk",
     "(A: bf16*, B: bf16*, bias: f32*, out: bf16*, M: i64, N: i64, K: i64, workspace: i8*, epoch: i64, spin_limit: i64)",
     Module::Gemm, Shape::GemmStreamK, 3},
    {"imex_gemm_f16_f16_f32_tb", "(A: f16*, Bt: f16* [N,K], C: f32*, M: i64, N: i64, K: i64)", Module::Gemm,
     Shape::GemmTB, 3},
    {"imex_gemm_f16_f16_f32_ta", "(At: f16* [K,M], B: f16*, C: f32*, M: i64, N: i64, K: i64)", Module::Gemm,
     Shape::GemmTA, 3},
    {"imex_gemm_4kx4kx4k_f16_f16_f32", "(A: f16*, B: f16*, C: f32*)", Module::Gemm, Shape::GemmFixed4k, 0},
    {"imex_gemm_4kx4kx4k_transpose_b", "(A: f16*, Bt: f16* [N,K], C: f32*)", Module::Gemm, Shape::GemmFixed4k, 0},
    {"imex_gemm_4kx4kx4k_transpose_a", "(At: f16* [K,M], B: f16*, C: f32*)", Module::Gemm, Shape::GemmFixed4k, 0},
    {"imex_gemm_4kx4kx4k_f16_f16_f32_bias", "(bias: f32*, C: f32*, A: f16*, B: f16*)", Module::Gemm,
     Shape::GemmFixed4k, 0},
};
constexpr int kEntryCount = sizeof(kEntries) / sizeof(kEntries[0]);

const Entry *find(const char *name) {
  if (!name)
    return nullptr;
  for (const Entry &e : kEntries)
    if (strcmp(e.name, name) == 0)
      return &e;
  return nullptr;
}

size_t ceilDiv(int64_t a, int64_t b) { return static_cast<size_t>((a + b - 1) / b); }

} // namespace

extern "C" int imexHipKernelCount(void) { return kEntryCount; }

extern "C" const char *imexHipKernelName(int index) {
  return (index >= 0 && index < kEntryCount) ? kEntries[index].name : nullptr;
}

extern "C" const char *imexHipKernelSignature(int index) {
  return (index >= 0 && index < kEntryCount) ? kEntries[index].signature : nullptr;
}

extern "C" const void *imexHipKernelModule(const char *kernel, size_t *size) {
  const Entry *e = find(kernel);
  if (!e)
    return nullptr;
  const unsigned char *begin = nullptr, *end = nullptr;
  switch (e->module) {
  case Module::Eltwise: begin = imex_blob_eltwise; end = imex_blob_eltwise_end; break;
  case Module::Softmax: begin = imex_blob_softmax; end = imex_blob_softmax_end; break;
  case Module::Reduce: begin = imex_blob_reduce; end = imex_blob_reduce_end; break;
  case Module::Transpose: begin = imex_blob_transpose; end = imex_blob_transpose_end; break;
  case Module::Gemm: begin = imex_blob_gemm; end = imex_blob_gemm_end; break;
  case Module::Fusion: begin = imex_blob_fusion; end = imex_blob_fusion_end; break;
  case Module::Attention: begin = imex_blob_attention; end = imex_blob_attention_end; break;
  }
  if (size)
    *size = static_cast<size_t>(end - begin);
  return begin;
}

extern "C" size_t imexHipStreamKWorkspaceBytes(size_t workgroups) { return 4096 + (size_t(256) * 256 * 4) * workgroups; }

extern "C" int imexHipKernelLaunchShape(const char *kernel, const int64_t *dims, int ndims, size_t grid[3],
                                        size_t block[3], size_t *sharedMemBytes) {
  const Entry *e = find(kernel);
  if (!e)
    return -1;
  if (ndims != e->ndims || (ndims > 0 && !dims))
    return -2;
  for (int i = 0; i < ndims; ++i)
    if (dims[i] < 0 || dims[i] > (int64_t(1) << 40))
      return -2;
  grid[0] = grid[1] = grid[2] = 1;
  block[0] = 256;
  block[1] = block[2] = 1;
  if (sharedMemBytes)
    *sharedMemBytes = 0;
  switch (e->shape) {
  case Shape::Eltwise32: // 256 lanes x 4 vectors x 4 elements
    grid[0] = ceilDiv(dims[0], 4096);
    break;
  case Shape::Eltwise16: // 256 lanes x 4 vectors x 8 elements
    grid[0] = ceilDiv(dims[0], 8192);
    break;
  case Shape::Fusion32: // SiLU and the fused chains: as Eltwise32 / 16, but one vector per lane below 4 Mi elements
    grid[0] = ceilDiv(dims[0], dims[0] < (int64_t(1) << 22) ? 1024 : 4096);
    break;
  case Shape::Fusion16:
    grid[0] = ceilDiv(dims[0], dims[0] < (int64_t(1) << 22) ? 2048 : 8192);
    break;
  case Shape::SoftmaxRows32:
  case Shape::SoftmaxRows16: {
    // Rows of up to 128 x 16 B stay in registers, one per wavefront (four per workgroup); longer rows take
    // a workgroup each.  The kernels stride over the rows, so any grid is correct.  f32 and bf16 register
    // rows: one pass (two rows per wavefront from 16384 rows on).  f16 register rows: a wavefront walks
    // its rows with the next row's loads in flight, and 2048 workgroups give every wavefront slot of the
    // chip (256 CUs x 4 SIMDs x 8) one wavefront.
    const int64_t regCols = e->shape == Shape::SoftmaxRows16 ? 1024 : 512;
    const bool f16 = std::strcmp(e->name, "imex_softmax_f16") == 0;
    if (dims[1] > regCols)
      grid[0] = static_cast<size_t>(dims[0] < 1048560 ? dims[0] : 1048560);
    else if (f16)
      grid[0] = std::min<size_t>(ceilDiv(dims[0], 4), 2048);
    else
      grid[0] = ceilDiv(dims[0], dims[0] >= 16384 ? 8 : 4);
    if (dims[1] == 0)
      grid[0] = 0;
    break;
  }
  case Shape::RowSum: // workgroup per row above 2048 columns, else wavefront per row
    grid[0] = dims[1] > 2048 ? static_cast<size_t>(dims[0]) : ceilDiv(dims[0], 4);
    break;
  case Shape::ReduceOuter:
  case Shape::ReduceOuter16: { // 256 lanes x v vectors of 4 (8) outputs, v = 8, 4, 2, 1: the widest that leaves 512 workgroups
    const int64_t inner = dims[1], perVec = e->shape == Shape::ReduceOuter ? 1024 : 2048;
    const int64_t v = inner >= 512 * 8 * perVec ? 8 : inner >= 512 * 4 * perVec ? 4 : inner >= 512 * 2 * perVec ? 2 : 1;
    grid[0] = ceilDiv(inner, perVec * v);
    break;
  }
  case Shape::Transpose2D32:
  case Shape::Transpose2D16:
  case Shape::Transpose3D32:
  case Shape::Transpose3D16: {
    // One workgroup per R x C tile.  Problems of 2^24 elements and more use the
    // large tiles (512-byte row segments): 128 x 128 for 32-bit, 256 x 256 for
    // 16-bit elements; smaller ones 64 x 64 / 128 x 128.  The kernels apply the same
    // rule, and stride over the tiles if the grid is any different.
    const bool is32 = e->shape == Shape::Transpose2D32 || e->shape == Shape::Transpose3D32;
    const bool is3d = e->shape == Shape::Transpose3D32 || e->shape == Shape::Transpose3D16;
    const int64_t rows = dims[0], cols = is3d ? dims[2] : dims[1], planes = is3d ? dims[1] : 1;
    const bool big = rows * cols * planes >= (int64_t(1) << 24);
    const int64_t tileR = is32 ? (big ? 128 : 64) : (big ? 256 : 128);
    const int64_t tileC = is32 ? (big ? 128 : 64) : (big ? 256 : 128);
    grid[0] = ceilDiv(cols, tileC);
    grid[1] = ceilDiv(rows, tileR);
    grid[2] = static_cast<size_t>(planes);
    if (grid[1] > 65535) // the kernels stride over the tiles a smaller grid leaves out
      grid[1] = 65535;
    if (grid[2] > 65535)
      grid[2] = 65535;
    // 32-bit problems made of whole 128 x 128 tiles: 512 workgroups (two per CU), each of which walks its
    // share of the tiles with the next tile's loads in flight while the current one is written
    if (is32 && big && rows % 128 == 0 && cols % 128 == 0) {
      const size_t budget = 512;
      if (grid[0] >= budget) {
        grid[0] = budget;
        grid[1] = grid[2] = 1;
      } else {
        grid[1] = std::min(grid[1], std::max<size_t>(1, budget / grid[0]));
        grid[2] = std::min(grid[2], std::max<size_t>(1, budget / (grid[0] * grid[1])));
      }
    }
    break;
  }
  case Shape::Attention: {
    // dims = {ZH, N_CTX}.  A workgroup takes 64, 128 or 256 queries of one (batch, head); the kernel reads
    // the choice off the grid and the block.  More queries per workgroup mean less K / V traffic, so: the
    // largest of the three that still gives every one of the 256 CUs a workgroup.  256 queries run as
    // sixteen wavefronts (8 query blocks x 2 key groups), the others as eight.  N_CTX need not divide.
    const int64_t ZH = dims[0], N = dims[1];
    block[0] = 512;
    if (N > 0 && N < (int64_t(1) << 24) && ZH > 0 && ZH <= 65535) {
      int64_t queries = 256;
      while (queries > 64 && ((N + queries - 1) / queries) * ZH < 256)
        queries /= 2;
      grid[0] = ceilDiv(N, queries);
      grid[1] = static_cast<size_t>(ZH);
      if (queries == 256)
        block[0] = 1024;
    } else {
      grid[0] = ceilDiv(ZH * N, 512); // one lane per query
    }
    break;
  }
  case Shape::ColumnThreads:
  case Shape::ColumnThreads16: {
    const int64_t rows = dims[0], cols = dims[1];
    // From 2048 rows and 128 row segments of 128 bytes on: the streaming form, 576 lanes per segment's
    // columns (32 f32 or 64 16-bit ones).  The kernel applies the same rule, and falls back by itself when
    // the rows are not made of whole aligned 16-byte vectors.
    const int64_t segment_cols = e->shape == Shape::ColumnThreads ? 32 : 64;
    if (rows >= 2048 && cols >= segment_cols * 128) {
      block[0] = 576;
      grid[0] = ceilDiv(cols, segment_cols);
      break;
    }
    // Fewer than 4096 columns (the reference's 512 x 1024): the same form with 256 workers and the adder
    // wavefront = 320 lanes per four columns.
    if (cols < 8 * 512) {
      block[0] = 320;
      grid[0] = ceilDiv(cols, 4);
      break;
    }
    // otherwise a workgroup per block of 64 .. 8 columns: the widest that leaves 512 workgroups
    const int64_t block_cols = cols >= 64 * 512 ? 64 : cols >= 32 * 512 ? 32 : cols >= 16 * 512 ? 16 : cols >= 8 * 512 ? 8 : 4;
    grid[0] = ceilDiv(cols, block_cols);
    break;
  }
  case Shape::Gemm:
  case Shape::GemmTA:
  case Shape::GemmTB: {
    // 512 lanes: eight wavefronts per 256 x 256 tile of C, edge tiles included.  The MFMA path
    // needs 16-byte aligned rows in memory, i.e. K % 8 == 0, N % 8 == 0 where B is [K,N] and
    // M % 8 == 0 where A is [K,M]; everything else runs 128 x 128 tiles on the vector ALUs.
    const int64_t M = dims[0], N = dims[1], K = dims[2];
    const bool rowsB = e->shape == Shape::GemmTB || N % 8 == 0;
    const bool rowsA = e->shape != Shape::GemmTA || M % 8 == 0;
    // operands addressed through one 32-bit-offset buffer descriptor must stay below 2 GiB
    const int64_t twoGiB = int64_t(1) << 31, maxRow = int64_t(1) << 22;
    const bool fitsA = e->shape == Shape::GemmTA ? K * M * 2 < twoGiB : K < maxRow;
    const bool fitsB = e->shape == Shape::GemmTB ? K < maxRow : K * N * 2 < twoGiB;
    const bool tileable = M > 0 && N > 0 && K > 0 && K % 8 == 0 && rowsA && rowsB && fitsA && fitsB;
    block[0] = 512;
    grid[0] = tileable ? ceilDiv(M, 256) * ceilDiv(N, 256) : ceilDiv(M, 128) * ceilDiv(N, 128);
    break;
  }
  case Shape::GemmStreamK: {
    // One workgroup per CU at most (256 on this part): the kernel's finishing workgroups wait for partial sums
    // of others, which have to be resident.  A problem with fewer tiles than CUs still gets more workgroups
    // than tiles -- its K loops are split -- as long as each one has 1024 k or more to do.
    const int64_t M = dims[0], N = dims[1], K = dims[2];
    const bool streams = M > 0 && N > 0 && K > 0 && K % 64 == 0 && N % 8 == 0;
    const size_t tiles = ceilDiv(M, 256) * ceilDiv(N, 256);
    const size_t shares = K >= 2048 ? static_cast<size_t>(K / 1024) : 1;
    block[0] = 512;
    grid[0] = !streams ? (K % 8 == 0 && N % 8 == 0 ? tiles : ceilDiv(M, 128) * ceilDiv(N, 128))
                       : std::min<size_t>(imexHipStreamKMaxWorkgroups, tiles * shares);
    break;
  }
  case Shape::GemmFixed4k: // the reference's own launch: blocks (16,16,1), threads (512,1,1)
    block[0] = 512;
    grid[0] = 16;
    grid[1] = 16;
    break;
  }
  // A grid component of 0 means there is nothing to launch.
  return 0;
}
