//===- GemmSplitK.hip - one-call entry points of the K-splitting GEMM + bias + SiLU ------------===//
//
// Host code (plus one device array) over the runtime ABI and the kernel catalogue: resolves
// imex_gemm_bf16_bias_silu_bf16_streamk, sizes its launch, stamps its workspace with a per-device launch
// counter and launches it through gpuLaunchKernel.  Two entries differ only in where the workspace lives:
// allocated by this library on first use, or the fixed device array below for callers that must not
// allocate.  There is no counterpart in the reference.
//
//===--------------------------------------------------------------------------------------------===//

#include "imex_hip_ops.h"

#include "imex_hip_kernels.h"
#include "imex_hip_runtime.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <mutex>

namespace {

constexpr const char *kKernelName = "imex_gemm_bf16_bias_silu_bf16_streamk";
// what imexHipStreamKWorkspaceBytes(imexHipStreamKMaxWorkgroups) comes to: 4 KiB of flags + 256 x 256 KiB
constexpr size_t kScratchBytes = 4096 + size_t(imexHipStreamKMaxWorkgroups) * 256 * 256 * 4;

// The fixed workspace.  In host code this name is only a handle for hipGetSymbolAddress: each GPU has its
// own copy at its own address, which devices[].scratch holds once imexHipOpsInit has run there.
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
struct PerDevice {
  bool ready = false;
  void *scratch = nullptr;   // this device's address of `scratch`
  void *kernel = nullptr;    // resolved through the runtime (cached there as well)
  void *allocated = nullptr; // workspace of the allocating entry
  size_t allocatedBytes = 0;
  int64_t launches = 0;      // the epoch stamped into the flags; never reused on a workspace
};
PerDevice devices[kMaxDevices];
std::mutex mutex;
thread_local char lastError[512] = "";

int fail(int code, const char *format, ...) {
  va_list ap;
  va_start(ap, format);
  vsnprintf(lastError, sizeof lastError, format, ap);
  va_end(ap);
  return code;
}

int deviceOf(void *queue) {
  const int device = imexHipQueueDevice(queue);
  return device >= 0 && device < kMaxDevices ? device : -1;
}

// Resolves kernel and scratch for `device` (mutex held).
int prepare(void *queue, int device) {
  PerDevice &d = devices[device];
  if (d.ready)
    return 0;
  size_t blobBytes = 0;
  const void *blob = imexHipKernelModule(kKernelName, &blobBytes);
  if (!blob)
    return fail(-4, "%s is not in the kernel catalogue", kKernelName);
  void *module = gpuModuleLoad(queue, blob, blobBytes);
  d.kernel = gpuKernelGet(queue, module, kKernelName);
  int previous = 0;
  if (hipGetDevice(&previous) != hipSuccess || hipSetDevice(device) != hipSuccess)
    return fail(-5, "cannot make device %d current", device);
  void *address = nullptr;
  const hipError_t rc = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
  (void)hipSetDevice(previous);
  if (rc != hipSuccess || !address)
    return fail(-5, "hipGetSymbolAddress(scratch) on device %d: %s", device, hipGetErrorString(rc));
  d.scratch = address;
  d.ready = true;
  return 0;
}

int launch(void *queue, PerDevice &d, void *workspace, size_t workspaceBytes, const void *A, const void *B,
           const void *bias, void *out, int64_t M, int64_t N, int64_t K, const size_t grid[3], const size_t block[3]) {
  int64_t epoch = ++d.launches, spinLimit = 0;
  (void)workspaceBytes;
  ImexParamDesc params[] = {{&A, sizeof A},       {&B, sizeof B},         {&bias, sizeof bias}, {&out, sizeof out},
                            {&M, sizeof M},       {&N, sizeof N},         {&K, sizeof K},       {&workspace, sizeof workspace},
                            {&epoch, sizeof epoch}, {&spinLimit, sizeof spinLimit}, {nullptr, 0}};
  ImexEventDesc noDeps[] = {{nullptr}};
  gpuLaunchKernel(queue, d.kernel, grid[0], grid[1], grid[2], block[0], block[1], block[2], 0, params, noDeps);
  return 0;
}

// grid / block of the launch and the workspace it needs; a negative code for shapes there is nothing to launch for
int shape(int64_t M, int64_t N, int64_t K, size_t grid[3], size_t block[3], size_t *bytes) {
  const int64_t dims[3] = {M, N, K};
  size_t smem = 0;
  if (M < 0 || N < 0 || K < 0 || imexHipKernelLaunchShape(kKernelName, dims, 3, grid, block, &smem) != 0)
    return fail(-1, "bad problem size %lld x %lld x %lld", (long long)M, (long long)N, (long long)K);
  *bytes = imexHipStreamKWorkspaceBytes(grid[0] * grid[1] * grid[2]);
  return 0;
}

} // namespace

extern "C" int imexHipOpsInit(void *queue) {
  const int device = deviceOf(queue);
  if (device < 0)
    return fail(-1, "not a queue of this runtime, or a device ordinal beyond %d", kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(mutex);
  return prepare(queue, device);
}

extern "C" int imexHipGemmBiasSiluBf16SplitK(void *queue, const void *A, const void *B, const void *bias, void *out,
                                             int64_t M, int64_t N, int64_t K) {
  const int device = deviceOf(queue);
  if (device < 0)
    return fail(-1, "not a queue of this runtime, or a device ordinal beyond %d", kMaxDevices - 1);
  size_t grid[3], block[3], bytes = 0;
  if (int rc = shape(M, N, K, grid, block, &bytes))
    return rc;
  if (grid[0] * grid[1] * grid[2] == 0)
    return 0; // an empty C
  std::lock_guard<std::mutex> lock(mutex);
  if (int rc = prepare(queue, device))
    return rc;
  PerDevice &d = devices[device];
  if (d.allocatedBytes < bytes) { // first use, or a larger launch than before: the queue is drained before the old one goes
    if (d.allocated) {
      gpuWait(queue);
      gpuMemFree(queue, d.allocated);
    }
    d.allocated = gpuMemAlloc(queue, bytes, 256, /*isShared=*/0);
    d.allocatedBytes = bytes;
  }
  return launch(queue, d, d.allocated, d.allocatedBytes, A, B, bias, out, M, N, K, grid, block);
}

extern "C" int imexHipGemmBiasSiluBf16SplitKNoAlloc(void *queue, const void *A, const void *B, const void *bias,
                                                    void *out, int64_t M, int64_t N, int64_t K) {
  const int device = deviceOf(queue);
  if (device < 0)
    return fail(-1, "not a queue of this runtime, or a device ordinal beyond %d", kMaxDevices - 1);
  size_t grid[3], block[3], bytes = 0;
  if (int rc = shape(M, N, K, grid, block, &bytes))
    return rc;
  if (grid[0] * grid[1] * grid[2] == 0)
    return 0;
  if (bytes > kScratchBytes)
    return fail(-3, "the launch needs a workspace of %zu bytes, the fixed one holds %zu", bytes, kScratchBytes);
  std::lock_guard<std::mutex> lock(mutex);
  PerDevice &d = devices[device];
  if (!d.ready)
    return fail(-2, "imexHipOpsInit has not run on device %d", device);
  // d.scratch, never the array's name: the name is not a device address in host code
  return launch(queue, d, d.scratch, kScratchBytes, A, B, bias, out, M, N, K, grid, block);
}

extern "C" size_t imexHipOpsFixedWorkspaceBytes(void) { return kScratchBytes; }

extern "C" const char *imexHipOpsLastError(void) { return lastError; }
