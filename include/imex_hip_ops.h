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

/* Once per device before the first imexHipGemmBiasSiluBf16SplitKNoAlloc on it (further calls do nothing):
 * loads the code object, resolves the kernel and this device's copy of the library's fixed workspace.
 * May allocate (the HIP runtime places the code object in device memory). */
int imexHipOpsInit(void *queue);

/* out = bf16(silu(A.B + bias[n])) with the K loops split over the chip's CUs.  The workspace
 * (imexHipStreamKWorkspaceBytes of the launch's workgroups: at most 64 MiB + 4 KiB) is allocated by the
 * library on the first call on a device and kept for the life of the process.  Calls on one device that may
 * overlap in time (different queues) must not be made: they would share the workspace. */
int imexHipGemmBiasSiluBf16SplitK(void *queue, const void *A, const void *B, const void *bias, void *out,
                                  int64_t M, int64_t N, int64_t K);

/* The same operator for callers that cannot allocate device memory at the point of the call -- code under
 * HIP graph capture, tight serving loops, harnesses that forbid it.  No counterpart in the reference.
 * Allocates nothing and calls nothing that allocates: the workspace is a fixed array of 64 MiB + 4 KiB in
 * the library's own device image (every GPU the library runs on holds one until the process ends), which
 * is the most the kernel's launch shape ever needs; a launch that would need more is refused (-3).
 * (With the runtime's profiling mode switched off, as it is by default: IMEX_ENABLE_PROFILING makes every
 * gpuLaunchKernel time its kernel first, and that loop allocates.)
 * Requires imexHipOpsInit on the queue's device (-2 otherwise).  All calls on one GPU share that array:
 * calls that overlap in time race, and nothing in it has to be cleared between calls (the flags in it are
 * stamped with a per-device launch counter). */
int imexHipGemmBiasSiluBf16SplitKNoAlloc(void *queue, const void *A, const void *B, const void *bias,
                                         void *out, int64_t M, int64_t N, int64_t K);

/* The bytes of the fixed workspace behind the NoAlloc entry. */
size_t imexHipOpsFixedWorkspaceBytes(void);

/* What went wrong in the calling thread's last failing call ("" if none has failed). */
const char *imexHipOpsLastError(void);

#ifdef __cplusplus
}
#endif
#endif
