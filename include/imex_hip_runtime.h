/*
 * imex_hip_runtime.h -- the IMEX ExecutionEngine runtime-wrapper C ABI, served
 * by HIP on AMD Instinct MI355X (gfx950).
 *
 * libimex-hip-runtime.so exports exactly the symbols that host code emitted by
 * IMEX's `convert-gpux-to-llvm` pass calls (callee names and LLVM types fixed at
 * lib/Conversion/GPUXToLLVM/GPUXToLLVMPass.cpp:120-209 and pinned by
 * the .mlir files under test/Conversion/GPUXToLLVM), with the semantics of the Level Zero
 * implementation they replace
 * (lib/ExecutionEngine/LEVELZERORUNTIME/LevelZeroRuntimeWrappers.cpp:606-671).
 * It is passed to `mlir-runner --shared-libs=` in place of
 * liblevel-zero-runtime.so / libsycl-runtime.so.
 *
 * Error convention (LevelZeroRuntimeWrappers.cpp:41-53): no return codes; any
 * failure prints "An exception was thrown: <what>" on stdout, flushes, and
 * calls abort().
 *
 * All signatures are plain C: opaque pointers, sizes, no C++ or framework
 * types.  `module` blobs are gfx950 code objects (ELF or clang offload
 * bundle); a SPIR-V blob is rejected with the error convention above.
 */
#ifndef IMEX_HIP_RUNTIME_H
#define IMEX_HIP_RUNTIME_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Kernel-argument and dependency lists handed to gpuLaunchKernel.
 * LevelZeroRuntimeWrappers.cpp:80-97; built by GPUXToLLVMPass.cpp:534-677.
 * `data` points at storage holding the argument VALUE (for a memref: its
 * aligned base pointer only), `size` is that value's byte size.  Arrays end
 * with {NULL, 0} / {NULL}. */
typedef struct ImexParamDesc {
  void *data;
  size_t size;
} ImexParamDesc;

typedef struct ImexEventDesc {
  void *event;
} ImexEventDesc;

/* ---- IMEX gpux ABI ------------------------------------------------------ */

/* LevelZeroRuntimeWrappers.cpp:606-622.  (NULL, NULL) -> stream on the default
 * GPU (ordinal from env IMEX_HIP_DEVICE, default 0).  Non-NULL `device` is an
 * `int *` device ordinal; non-NULL `context` is an existing hipStream_t to
 * adopt (not destroyed by gpuStreamDestroy). */
void *gpuCreateStream(void *device, void *context);

/* LevelZeroRuntimeWrappers.cpp:624-626.  Waits for the stream, releases the
 * events it handed out, destroys the stream it created. */
void gpuStreamDestroy(void *queue);

/* LevelZeroRuntimeWrappers.cpp:628-632 (call site passes isShared as i32,
 * GPUXToLLVMPass.cpp:183-191: only the low byte is tested).  isShared ->
 * host-dereferenceable, device-accessible memory; else device HBM.  The
 * pointer is at least 256-byte aligned; larger power-of-two alignments are
 * honoured.  size 0 yields a valid, freeable pointer. */
void *gpuMemAlloc(void *queue, size_t size, size_t alignment, int isShared);

/* LevelZeroRuntimeWrappers.cpp:634-637; NULL queue or pointer is ignored
 * (SyclRuntimeWrappers.cpp:452-458). */
void gpuMemFree(void *queue, void *ptr);

/* LevelZeroRuntimeWrappers.cpp:639-642.  Blocking; direction inferred from
 * the pointers (H2D, D2H, D2D, H2H). */
void gpuMemCopy(void *queue, void *dst, void *src, size_t bytes);

/* LevelZeroRuntimeWrappers.cpp:644-647,396-432.  Cached by `data` pointer for
 * the life of the process; called before every launch, so the hit path is
 * cheap. */
void *gpuModuleLoad(void *queue, const void *data, size_t dataSize);

/* LevelZeroRuntimeWrappers.cpp:649-652. */
void *gpuKernelGet(void *queue, void *module, const char *name);

/* LevelZeroRuntimeWrappers.cpp:654-664,445-480,507-603.  grid* = number of
 * workgroups.  If sharedMemBytes != 0 the last ParamDesc is the placeholder
 * for dynamic shared memory and is not passed as an argument.  Only the low 32
 * bits of sharedMemBytes are used (the call site passes i32).  Returns an
 * event that stands for "after this launch" on the stream, owned by the
 * stream; it can be listed in a later launch's depEvents (on any stream).
 * The handle is valid until the stream is destroyed; once 4096 further
 * launches have gone to the stream it stands for a later position of that
 * stream (a wait on it then waits longer than needed, never shorter).
 * Environment (LevelZeroRuntimeWrappers.cpp:521-597): IMEX_ENABLE_PROFILING,
 * IMEX_PROFILING_RUNS (default 1000), IMEX_PROFILING_WARMUPS (default 3),
 * IMEX_ENABLE_CACHE_FLUSHING, plus IMEX_CACHE_FLUSH_BYTES (default 512 MiB:
 * that many bytes are filled and as many of a second region read before each
 * timed run, so the caches hold neither the kernel's data nor dirty lines).
 * Each run's time is the dispatch's own start-to-end interval, as the
 * reference's is; IMEX_PROFILING_EVENT_PAIRS=1 records events around the
 * launch instead. */
void *gpuLaunchKernel(void *queue, void *kernel, size_t gridX, size_t gridY, size_t gridZ,
                      size_t blockX, size_t blockY, size_t blockZ, size_t sharedMemBytes,
                      void *params, void *depEvents);

/* LevelZeroRuntimeWrappers.cpp:666-671 (SYCL twin: queue.wait(),
 * SyclRuntimeWrappers.cpp:498-505).  Blocks until the stream is idle. */
void gpuWait(void *queue);

/* Declared by the lowering (GPUXToLLVMPass.cpp:129-134), exported by neither
 * reference wrapper; modules live for the process, so this is a no-op. */
void gpuModuleUnload(void *queue, void *module);

/* `count` 32-bit (16-bit) elements at `dst` set to `value`, asynchronously on the stream; gpuWait or a
 * later launch on the stream orders after it.  No reference line to cite: `gpux.memset` exists as an
 * op but convert-gpux-to-llvm has no pattern for it (lib/Conversion/GPUXToLLVM/GPUXToLLVMPass.cpp:828-840
 * lists the lowered ops), so these two names and signatures are this library's -- the stream-first
 * form of the upstream callees below, for a lowering to bind when one is added.  `dst` must be
 * aligned to the element size.  Runs as a kernel of this library, never as a memset on the stream. */
void gpuMemSet32(void *queue, void *dst, unsigned int value, size_t count);
void gpuMemSet16(void *queue, void *dst, unsigned short value, size_t count);

/* ---- upstream gpu-to-llvm ABI: the nine names the reference's wrapper exports
 *      (LevelZeroRuntimeWrappers.cpp:673-741) ---- */
void *mgpuStreamCreate(void);
void mgpuStreamSynchronize(void *stream);
void mgpuStreamDestroy(void *stream);
void mgpuLaunchKernel(void *kernel, size_t gridX, size_t gridY, size_t gridZ, size_t blockX,
                      size_t blockY, size_t blockZ, size_t sharedMemBytes, void *stream,
                      void **params, void **extra, size_t paramsCount);
void *mgpuMemAlloc(size_t size, void *stream, int isShared);
void mgpuMemFree(void *stream, void *ptr);
void *mgpuModuleLoad(const void *data, size_t dataSize);
void *mgpuModuleGetFunction(void *module, const char *name);
void mgpuModuleUnload(void *module);
/* Three more callee names of upstream MLIR's gpu-to-llvm lowering (gpu.memcpy, gpu.memset of 32-bit and
 * of 16-bit elements).  No reference line: the reference's wrapper exports the nine names above and none
 * of these three; they are here so that host code lowered by upstream's pass finds every callee it binds.
 * The fills run as a kernel of this library (not as a memset on the stream), so a caller that captures
 * the stream into a HIP graph gets an ordinary kernel node; `count` is in elements. */
void mgpuMemcpy(void *dst, void *src, size_t bytes, void *stream);
void mgpuMemset32(void *dst, unsigned int value, size_t count, void *stream);
void mgpuMemset16(void *dst, unsigned short value, size_t count, void *stream);

/* ---- measurement helpers (no counterpart in the reference ABI; they expose
 *      the profiling loop of launchKernel, LevelZeroRuntimeWrappers.cpp:521-597,
 *      to callers that want the numbers instead of the printed line) -------- */

/* Runs `warmups` untimed launches, then `rounds` timed ones.
 * mode 0: one event pair per launch, times_ms[0..rounds) = per-launch ms
 *         (the reference profiler's protocol); flushBytes > 0 writes that many
 *         bytes of a scratch buffer before each timed launch.
 * mode 1: one event pair around `rounds` back-to-back launches,
 *         times_ms[0] = total ms.
 * Returns 0. */
int imexHipProfileKernel(void *queue, void *kernel, size_t gridX, size_t gridY, size_t gridZ,
                         size_t blockX, size_t blockY, size_t blockZ, size_t sharedMemBytes,
                         void *params, int warmups, int rounds, size_t flushBytes, int mode,
                         float *times_ms);

/* Records a timestamp event at the stream's current tail (owned by the stream; the handle is good
 * until 1024 further timestamps have been recorded on that stream). */
void *imexHipRecordTimestamp(void *queue);

/* Milliseconds between two imexHipRecordTimestamp events of one stream.  An event returned by
 * gpuLaunchKernel is refused (error convention above): it is an ordering point whose HIP event
 * is only recorded when it is first waited on, so it carries no time of its own. */
float imexHipEventElapsedMs(void *startEvent, void *stopEvent);

/* out[9] = avg, min, max, median, stddev, variance, P95, P5, middle-third avg
 * (formulas of lib/ExecutionEngine/ExecutionEngineUtils/ExecutionEngineUtils.cpp:18-150;
 * the median is the textbook one, valid for every n). */
void imexHipComputeStats(const float *values, size_t n, float *out);

/* Device facts used for rooflines: CU count, clock (kHz), L2 bytes, total
 * global memory bytes.  Returns 0, or -1 without a usable GPU. */
int imexHipDeviceInfo(void *queue, int *cuCount, int *clockKHz, size_t *l2Bytes, size_t *globalBytes,
                      char *name, size_t nameLen);

/* The device ordinal a queue of gpuCreateStream runs on; -1 for NULL. */
int imexHipQueueDevice(void *queue);

#ifdef __cplusplus
}
#endif
#endif
