// Entry points of the tiled MFMA GEMM for gfx950: C[M,N] = A[M,K] . B[K,N], A and B f16 or bf16
// (row-major), f32 accumulate; also with A stored [K,M] or B stored [N,K].  The tile code, its
// blocking and the reference kernels it stands for are described in gemm_tile.h.
//
// Launch: block (512,1,1); grid (tiles,1,1) with tiles = ceil(M/256)*ceil(N/256) on
// the MFMA path, else (ceil(M/128)*ceil(N/128),1,1); workgroups stride, so any grid is correct.  The fixed-shape
// 4096^3 entry points take the reference's own launch: blocks (16,16,1), threads (512,1,1).

#include "gemm_tile.h"

using namespace imexhip;
using namespace imexhip_gemm;

// C = A.B
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_f16_f16_f32(const uint16_t *A, const uint16_t *B,
                                                                            float *C, int64_t M, int64_t N,
                                                                            int64_t K) {
  gemm_entry<F16, false, false>(A, B, M, N, K, StoreF32{C});
}
// C += A.B
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_f16_f16_f32_acc(const uint16_t *A,
                                                                                const uint16_t *B, float *C,
                                                                                int64_t M, int64_t N, int64_t K) {
  gemm_entry<F16, false, false>(A, B, M, N, K, AccumulateF32{C});
}
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_bf16_bf16_f32(const uint16_t *A,
                                                                              const uint16_t *B, float *C,
                                                                              int64_t M, int64_t N, int64_t K) {
  gemm_entry<BF16, false, false>(A, B, M, N, K, StoreF32{C});
}
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_bf16_bf16_f32_acc(const uint16_t *A,
                                                                                  const uint16_t *B, float *C,
                                                                                  int64_t M, int64_t N,
                                                                                  int64_t K) {
  gemm_entry<BF16, false, false>(A, B, M, N, K, AccumulateF32{C});
}
// C(f16) = A.B
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_f16_f16_f16(const uint16_t *A, const uint16_t *B,
                                                                            uint16_t *C, int64_t M, int64_t N,
                                                                            int64_t K) {
  gemm_entry<F16, false, false>(A, B, M, N, K, StoreF16{C});
}
// out(bf16) = silu(A.B + bias[n])
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_bf16_bias_silu_bf16(const uint16_t *A,
                                                                                    const uint16_t *B,
                                                                                    const float *bias,
                                                                                    uint16_t *out, int64_t M,
                                                                                    int64_t N, int64_t K) {
  gemm_entry<BF16, false, false>(A, B, M, N, K, BiasSiluBF16{out, bias});
}

// The same with a workspace: the tiles that are left after the last full round of one tile per workgroup
// have their K loops dealt out evenly over all workgroups (stream-K, gemm_tile.h).  Launch with at most
// one workgroup per CU.  workspace: 4096 + 262144 * workgroups bytes, 16-byte aligned, not shared with a
// launch that may overlap this one; epoch: differs from the previous launch's on the same workspace;
// spin_limit: how long a finishing workgroup waits for the others' partial sums before it computes them
// itself, in ~1 us units (0: about a second).  Null workspace: the kernel above.
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_bf16_bias_silu_bf16_streamk(
    const uint16_t *A, const uint16_t *B, const float *bias, uint16_t *out, int64_t M, int64_t N, int64_t K,
    void *workspace, int64_t epoch, int64_t spin_limit) {
  gemm_entry_streamk<BF16>(A, B, M, N, K, BiasSiluBF16{out, bias}, workspace, epoch, spin_limit);
}

// C = A . B^T with B stored [N,K] (WG/gemm_4kx4kx4k_transpose_b.mlir:16,70-83: the
// B tile is loaded k-contiguous and transposed in registers before the dpas)
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_f16_f16_f32_tb(const uint16_t *A, const uint16_t *Bt,
                                                                               float *C, int64_t M, int64_t N,
                                                                               int64_t K) {
  gemm_entry<F16, false, true>(A, Bt, M, N, K, StoreF32{C});
}
// C = A^T . B with A stored [K,M] (WG/gemm_4kx4kx4k_transpose_a.mlir:41-47)
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_f16_f16_f32_ta(const uint16_t *At, const uint16_t *B,
                                                                               float *C, int64_t M, int64_t N,
                                                                               int64_t K) {
  gemm_entry<F16, true, false>(At, B, M, N, K, StoreF32{C});
}

// Fixed-shape entry points with the reference kernels' own signatures, so the
// reference's host code can launch them unchanged apart from the block size:
//   gemm_4kx4kx4k_f16_f16_f32.mlir:38,48   args (A, B, C), grid (16,16,1), C += A.B
//   gemm_4kx4kx4k_f16_f16_f32_bias.mlir:44,78 args (bias, C, A, B), C = bias + (C + A.B)
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_4kx4kx4k_f16_f16_f32(const uint16_t *A,
                                                                                     const uint16_t *B,
                                                                                     float *C) {
  gemm_entry<F16, false, false>(A, B, 4096, 4096, 4096, AccumulateF32{C});
}
//   gemm_4kx4kx4k_transpose_b.mlir:40,53   args (A, B[N,K], C), C += A.B^T
//   gemm_4kx4kx4k_transpose_a.mlir:21,31   args (A[K,M], B, C), C += A^T.B
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_4kx4kx4k_transpose_b(const uint16_t *A,
                                                                                     const uint16_t *Bt,
                                                                                     float *C) {
  gemm_entry<F16, false, true>(A, Bt, 4096, 4096, 4096, AccumulateF32{C});
}
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_4kx4kx4k_transpose_a(const uint16_t *At,
                                                                                     const uint16_t *B,
                                                                                     float *C) {
  gemm_entry<F16, true, false>(At, B, 4096, 4096, 4096, AccumulateF32{C});
}
extern "C" __global__ __launch_bounds__(kThreads) void imex_gemm_4kx4kx4k_f16_f16_f32_bias(const float *bias,
                                                                                          float *C,
                                                                                          const uint16_t *A,
                                                                                          const uint16_t *B) {
  gemm_entry<F16, false, false>(A, B, 4096, 4096, 4096, BiasAccumulateF32{C, bias});
}
