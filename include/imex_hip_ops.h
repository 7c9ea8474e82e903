/*
 * imex_hip_ops.h -- one-call operator entry points on top of the runtime ABI (imex_hip_runtime.h) and the
 * kernel catalogue (imex_hip_kernels.h), exported by libimex-hip-ops.so.
 *
 * No counterpart in the reference: its host code always goes through gpuModuleLoad / gpuKernelGet /
 * gpuLaunchKernel itself.  These entries exist for the one operator here whose kernel needs device memory
 * beyond its inputs and outputs -- the K-splitting form of out = bf16(silu(A.B + bias)),
 * imex_gemm_bf16_bias_silu_bf16_streamk, which passes partial sums between workgroups through a
 * workspace -- so that a caller does not have to size, allocate and stamp that workspace.
 *
 * Every function returns 0 on success and a negative number on failure; imexHipOpsLastError() then
 * describes the failure of the calling thread's last call.  `queue` is a queue of gpuCreateStream; the
 * launch is asynchronous on it (gpuWait orders after it).  A, B bf16 row-major [M,K], [K,N]; bias f32
 * [N]; out bf16 [M,N]; all device pointers.
 */
#ifndef IMEX_HIP_OPS_H
#define IMEX_HIP_OPS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* out = bf16(silu(A.B + bias[n])) with the K loops split over the chip's CUs.  The workspace
 * (imexHipStreamKWorkspaceBytes of the launch's workgroups: at most 64 MiB + 4 KiB) is allocated by the
 * library on the first call on a device and kept for the life of the process.  Calls on one device that may
 * overlap in time (different queues) must not be made: they would share the workspace. */
int imexHipGemmBiasSiluBf16SplitK(void *queue, const void *A, const void *B, const void *bias, void *out,
                                  int64_t M, int64_t N, int64_t K);

/* What went wrong in the calling thread's last failing call ("" if none has failed). */
const char *imexHipOpsLastError(void);

#ifdef __cplusplus
}
#endif
#endif
