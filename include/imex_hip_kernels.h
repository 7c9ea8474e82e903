/*
 * imex_hip_kernels.h -- catalogue of the hand-written gfx950 kernels that stand
 * in for the device code IMEX generates (SPIR-V / XeVM) for its benchmark
 * workloads, and the launch shape each one expects.
 *
 * libimex-hip-kernels.so embeds the code objects (what a `gpu.binary`
 * attribute would hold, cf. lib/Transforms/SerializeSPIRV.cpp:65-69) and
 * answers two questions host code has to settle before calling
 * gpuModuleLoad / gpuKernelGet / gpuLaunchKernel (imex_hip_runtime.h):
 * which blob holds a kernel, and with what grid and block it is launched.
 *
 * Kernel argument convention (lib/Conversion/GPUXToLLVM/GPUXToLLVMPass.cpp:571-584):
 * one raw aligned base pointer per memref, scalars by value; `index` is i64.
 *
 * Kernels (name : arguments : reference op body it replaces)
 *   imex_relu_f32 / _f16 / _bf16   (in, out, n:i64)
 *       benchmarks/relu/relu_gpu.mlir.in:3-13            dims = {n}
 *   imex_silu_f32 / _f16 / _bf16   (in, out, n:i64)
 *       benchmarks/silu/silu_gpu.mlir.in:3-19            dims = {n}
 *   imex_exp_f32                   (in, out, n:i64)                 out = expf(in), libm's
 *       test/Integration/Dialect/XeGPU/WG/math_exp.mlir:49-62    dims = {n}
 *   imex_maximum_f32               (a, b, out, n:i64)               out = maximumf(a, b): NaN if either is
 *       test/Integration/Dialect/XeGPU/WG/arith_maximumf.mlir:51-66   dims = {n}
 *   imex_softmax_f32 / _f16 / _bf16 (in, out, rows:i64, cols:i64)
 *       benchmarks/softmax/softmax_gpu.mlir.in:4-44      dims = {rows, cols}
 *   imex_rowsum_f32                (in, out, rows:i64, cols:i64, init:f32)
 *       WG/reduction_2D_1D_cross_sg_cross_lane.mlir:31-37 dims = {rows, cols}
 *   imex_rowmean_f32               (in, out, rows:i64, cols:i64)   out[r] = (sum_c in[r,c]) / cols
 *       WG/reduction_4D_3D_mean_intra_sg_intra_lane.mlir:51-52   dims = {rows, cols}
 *   imex_reduce_outer_f32 / _f16 / _bf16  (in, out, outer:i64, inner:i64, init:f32)
 *       benchmarks/reduce/reduce_gpu.mlir.in:4-21        dims = {outer, inner}
 *   imex_transpose2d_b16 / _b32    (in, out, rows:i64, cols:i64)
 *       benchmarks/transpose/transpose2d_gpu.mlir.in:4-11 dims = {rows, cols}
 *   imex_transpose3d_b16 / _b32    (in, out, d0:i64, d1:i64, d2:i64)
 *       benchmarks/transpose/transpose3d_gpu.mlir.in:4-11 dims = {d0, d1, d2}
 *   imex_loop_fusion_f32 / _f16 / _bf16   (a, b, out, n:i64)         out = (log a + |b|) - a
 *       benchmarks/kLoopFusion/kLoopFusion.mlir.in:4-30  dims = {n}
 *   imex_input_fusion_f32 / _f16 / _bf16  (a, b, out, rows:i64, cols:i64)
 *       out[j] = sum_i (log b[i,j] + |a[i,j]|)
 *       benchmarks/kInputFusion/kInputFusion.mlir.in:6-40 dims = {rows, cols}
 *   imex_flash_attention_fwd_f16   (Q, K, V, Out, sm_scale:f32, ZH:i64, N_CTX:i64)
 *       softmax(sm_scale Q K^T) V per (batch, head), head dim 64, tensors [(ZH*N_CTX), 64]
 *       WG/flash_attention_fwd.mlir:25-307               dims = {ZH, N_CTX}
 *   imex_gemm_f16_f16_f32[_acc], imex_gemm_bf16_bf16_f32[_acc], imex_gemm_f16_f16_f16
 *                                  (A, B, C, M:i64, N:i64, K:i64)
 *       WG/gemm_4kx4kx4k_f16_f16_f32.mlir:47-91          dims = {M, N, K}
 *   imex_gemm_f16_f16_f32_tb       (A, Bt, C, M:i64, N:i64, K:i64)   B stored [N,K]: C = A.B^T
 *       WG/gemm_4kx4kx4k_transpose_b.mlir:53-88          dims = {M, N, K}
 *   imex_gemm_f16_f16_f32_ta       (At, B, C, M:i64, N:i64, K:i64)   A stored [K,M]: C = A^T.B
 *       WG/gemm_4kx4kx4k_transpose_a.mlir:31-55          dims = {M, N, K}
 *   imex_gemm_bf16_bias_silu_bf16  (A, B, bias, out, M:i64, N:i64, K:i64)
 *       WG/gemm_4kx4kx4k_f16_f16_f32_bias.mlir:88-113 + silu_gpu.mlir.in:3-19
 *   imex_gemm_bf16_bias_silu_bf16_streamk  (A, B, bias, out, M:i64, N:i64, K:i64, workspace, epoch:i64, spin_limit:i64)
 *       the same operator with the last, partial round of tiles split along K over all workgroups (no
 *       counterpart in the reference); workspace: imexHipStreamKWorkspaceBytes(grid) bytes of device
 *       memory, 16-byte aligned, contents irrelevant, not shared with an overlapping launch; epoch: any
 *       value other than the one of the previous launch on that workspace; spin_limit: 0, or how many
 *       ~1 us waits a workgroup spends on another's partial sums before computing them itself
 *                                                          dims = {M, N, K}
 *   imex_gemm_4kx4kx4k_f16_f16_f32       (A, B, C)        dims = {}
 *   imex_gemm_4kx4kx4k_f16_f16_f32_bias  (bias, C, A, B)  dims = {}
 *   imex_gemm_4kx4kx4k_transpose_b       (A, Bt, C)       dims = {}   C += A.B^T
 *   imex_gemm_4kx4kx4k_transpose_a       (At, B, C)       dims = {}   C += A^T.B
 *       the reference kernels' own signatures (WG/...f32.mlir:48, ...bias.mlir:78,
 *       ...transpose_b.mlir:53, ...transpose_a.mlir:31)
 */
#ifndef IMEX_HIP_KERNELS_H
#define IMEX_HIP_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Number of kernels in the catalogue and the i-th one's name / argument list. */
int imexHipKernelCount(void);
const char *imexHipKernelName(int index);
const char *imexHipKernelSignature(int index);

/* The code object that contains `kernel` (the `data`/`dataSize` to give
 * gpuModuleLoad).  The pointer is stable for the life of the process, so the
 * runtime's by-pointer module cache hits.  NULL if the name is unknown. */
const void *imexHipKernelModule(const char *kernel, size_t *size);

/* Grid (in workgroups), block and dynamic shared memory for `kernel` on a
 * problem of the given dims (see the table above).  Returns 0 on success,
 * -1 unknown kernel, -2 wrong number of dims or a negative / overflowing dim. */
int imexHipKernelLaunchShape(const char *kernel, const int64_t *dims, int ndims, size_t grid[3],
                             size_t block[3], size_t *sharedMemBytes);

/* Stream-K kernels (imex_gemm_bf16_bias_silu_bf16_streamk): the most workgroups their launch shape
 * ever asks for -- one per CU of the part -- and the workspace a launch of `workgroups` needs:
 * 4096 bytes of flags and 256 KiB of partial sums per workgroup (64 MiB + 4 KiB at 256). */
enum { imexHipStreamKMaxWorkgroups = 256 };
size_t imexHipStreamKWorkspaceBytes(size_t workgroups);

#ifdef __cplusplus
}
#endif
#endif
