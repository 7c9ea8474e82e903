//===- HipRuntimeWrappers.cpp - IMEX gpu* runtime ABI over HIP ------------===//
//
// The extern "C" runtime-wrapper ABI that IMEX's convert-gpux-to-llvm lowering
// calls (lib/Conversion/GPUXToLLVM/GPUXToLLVMPass.cpp:120-209), implemented on
// HIP for MI355X.  Semantics follow the Level Zero implementation
// (lib/ExecutionEngine/LEVELZERORUNTIME/LevelZeroRuntimeWrappers.cpp:367-671)
// with the SYCL twin (lib/ExecutionEngine/SYCLRUNTIME/SyclRuntimeWrappers.cpp)
// as second witness where the two differ.
//
// Design notes (HIP-first, not a translation):
//  * a "queue" is {device ordinal, hipStream_t}; work is asynchronous on the
//    stream and gpuWait / gpuMemCopy synchronise it (the Level Zero wrapper
//    used a synchronous immediate command list instead);
//  * modules are gfx950 code objects loaded with hipModuleLoadData and cached
//    by blob address for the life of the process; kernels are cached per
//    (module, name), so the load+get pair that precedes every launch costs two
//    map lookups;
//  * events returned by gpuLaunchKernel are stream positions held in a ring of
//    slots owned by the stream (the reference never frees its events and draws
//    them from a 256-slot pool that overflows); the HIP event behind one is
//    recorded only when it is first used;
//  * profiling uses hipEvent pairs on the launch stream.
//
//===----------------------------------------------------------------------===//

#include "imex_hip_runtime.h"

#include "ProfilerStats.h"

#include <hip/hip_runtime_api.h>

// From <hip/hip_ext.h>, which a host compiler cannot include whole: a module launch that attaches a start
// and a stop event to the dispatch.  Global sizes are in work-items.
extern "C" hipError_t hipExtModuleLaunchKernel(hipFunction_t f, uint32_t globalWorkSizeX, uint32_t globalWorkSizeY,
                                               uint32_t globalWorkSizeZ, uint32_t localWorkSizeX,
                                               uint32_t localWorkSizeY, uint32_t localWorkSizeZ,
                                               size_t sharedMemBytes, hipStream_t hStream, void **kernelParams,
                                               void **extra, hipEvent_t startEvent, hipEvent_t stopEvent,
                                               uint32_t flags);

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace {

// LevelZeroRuntimeWrappers.cpp:41-53: report on stdout, flush, abort.
template <typename F> auto catchAll(F &&func) {
  try {
    return func();
  } catch (const std::exception &e) {
    fprintf(stdout, "An exception was thrown: %s\n", e.what());
    fflush(stdout);
    abort();
  } catch (...) {
    fprintf(stdout, "An unknown exception was thrown\n");
    fflush(stdout);
    abort();
  }
}

inline void checkHip(hipError_t res, const char *expr) {
  if (res != hipSuccess)
    throw std::runtime_error(std::string(expr) + " failed: " + std::to_string(static_cast<int>(res)) +
                             " (" + hipGetErrorString(res) + ")");
}
#define CHECK_HIP(expr) checkHip((expr), #expr)

struct GpuHipQueue;

// What gpuLaunchKernel returns: a position in a stream (after the launch with
// this sequence number).  No GPU-side marker is recorded at launch time -- a
// completion signal per kernel costs ~15 us of dispatch bubble between
// back-to-back launches, and host code that launches synchronously discards the
// event anyway.  The HIP event is materialised on first use: recording it then
// still places it after the launch it stands for (streams are in order), so a
// dependency on it is satisfied no earlier than the reference semantics demand.
struct LaunchEvent {
  GpuHipQueue *queue;
  uint64_t sequence;    // the launch this slot currently stands for
  hipEvent_t event;     // null until someone waits on or times a position of this slot
  uint64_t recordedFor; // sequence `event` was last recorded for (0: never)
  bool isTimestamp;     // recorded when it was handed out (imexHipRecordTimestamp), so it marks a point in time
};

// Launch events live in a ring: a handle stays valid for the life of its stream,
// and after kEventSlots further launches it stands for a LATER position of the
// same in-order stream -- waiting on a stale handle over-synchronises, it never
// under-synchronises -- so a process that launches for days does not grow.
constexpr size_t kEventSlots = 4096;
// Timestamps come from a ring of their own: a handle is good until kTimestampSlots further
// timestamps have been recorded on its stream, then its slot is recorded anew.
constexpr size_t kTimestampSlots = 1024;

struct GpuHipQueue {
  int device = 0;
  hipStream_t stream = nullptr;
  bool ownsStream = true;
  uint64_t launches = 0;
  std::vector<LaunchEvent> ring;          // handed out by gpuLaunchKernel, slot = launch number mod ring size
  std::vector<LaunchEvent> timestamps;    // handed out by imexHipRecordTimestamp, slot = timestamp number mod ring size
  uint64_t timestampCount = 0;
  void *flushBuffer = nullptr;    // scratch for the profiler's cache flush
  size_t flushBytes = 0;

  GpuHipQueue(int dev, hipStream_t adopt) : device(dev) {
    CHECK_HIP(hipSetDevice(device));
    if (adopt) {
      stream = adopt;
      ownsStream = false;
    } else {
      // Default priority on purpose: mixed-priority streams are not used anywhere.
      CHECK_HIP(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking));
    }
  }

  // Waits for the stream and releases what the queue owns; throws on a HIP error (the callers
  // run it under catchAll before deleting the queue).  Idempotent.
  void release() {
    if (!stream)
      return;
    CHECK_HIP(hipSetDevice(device));
    CHECK_HIP(hipStreamSynchronize(stream));
    for (std::vector<LaunchEvent> *events : {&ring, &timestamps}) {
      for (LaunchEvent &e : *events)
        if (e.event)
          CHECK_HIP(hipEventDestroy(e.event));
      events->clear();
    }
    if (flushBuffer)
      CHECK_HIP(hipFree(flushBuffer));
    flushBuffer = nullptr;
    if (ownsStream)
      CHECK_HIP(hipStreamDestroy(stream));
    stream = nullptr;
  }

  // A queue that was not released (a thread's default queue at thread exit): best effort, no throw.
  ~GpuHipQueue() {
    try {
      release();
    } catch (...) {
    }
  }
};

void destroyQueue(GpuHipQueue *queue) {
  if (!queue)
    return;
  queue->release();
  delete queue;
}

int defaultDeviceOrdinal() {
  if (const char *env = getenv("IMEX_HIP_DEVICE"))
    return static_cast<int>(strtol(env, nullptr, 10));
  return 0;
}

// ---- allocations -----------------------------------------------------------

enum class AllocKind { Device, HostShared };
struct AllocInfo {
  void *base;
  AllocKind kind;
};
std::map<void *, AllocInfo> allocRegistry;
std::mutex allocMutex;

constexpr size_t kNaturalAlignment = 256; // what hipMalloc / hipHostMalloc give

void *allocMemory(GpuHipQueue *queue, size_t size, size_t alignment, bool isShared) {
  if (!queue)
    throw std::runtime_error("gpuMemAlloc: null stream");
  if (alignment & (alignment - 1))
    throw std::runtime_error("gpuMemAlloc: alignment " + std::to_string(alignment) +
                             " is not a power of two");
  CHECK_HIP(hipSetDevice(queue->device));
  size_t bytes = size ? size : 1;
  if (alignment > kNaturalAlignment)
    bytes += alignment;
  void *base = nullptr;
  if (isShared) {
    // Host-dereferenceable and device-accessible, coherent: JIT'd host code
    // memref.copy's straight into it (test/SPIRV/OpTest.GEMM_F16_ACC_F32.mlir:43-48).
    CHECK_HIP(hipHostMalloc(&base, bytes, hipHostMallocMapped | hipHostMallocCoherent));
  } else {
    CHECK_HIP(hipMalloc(&base, bytes));
  }
  if (!base)
    throw std::runtime_error("gpuMemAlloc: allocation of " + std::to_string(size) + " bytes returned null");
  void *user = base;
  if (alignment > kNaturalAlignment) {
    uintptr_t p = reinterpret_cast<uintptr_t>(base);
    p = (p + alignment - 1) & ~(static_cast<uintptr_t>(alignment) - 1);
    user = reinterpret_cast<void *>(p);
  }
  std::lock_guard<std::mutex> lock(allocMutex);
  allocRegistry[user] = {base, isShared ? AllocKind::HostShared : AllocKind::Device};
  return user;
}

void freeMemory(GpuHipQueue *queue, void *ptr) {
  if (!queue || !ptr)
    return;
  AllocInfo info;
  {
    std::lock_guard<std::mutex> lock(allocMutex);
    auto it = allocRegistry.find(ptr);
    if (it == allocRegistry.end())
      throw std::runtime_error("gpuMemFree: pointer was not returned by gpuMemAlloc");
    info = it->second;
    allocRegistry.erase(it);
  }
  CHECK_HIP(hipSetDevice(queue->device));
  // Work that still uses the buffer may be in flight on the stream.
  CHECK_HIP(hipStreamSynchronize(queue->stream));
  if (info.kind == AllocKind::HostShared)
    CHECK_HIP(hipHostFree(info.base));
  else
    CHECK_HIP(hipFree(info.base));
}

void copyMemory(GpuHipQueue *queue, void *dst, void *src, size_t bytes) {
  if (!queue)
    throw std::runtime_error("gpuMemCopy: null stream");
  if (bytes == 0)
    return;
  if (!dst || !src)
    throw std::runtime_error("gpuMemCopy: null pointer with non-zero size");
  CHECK_HIP(hipSetDevice(queue->device));
  CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, queue->stream));
  CHECK_HIP(hipStreamSynchronize(queue->stream));
}

// ---- modules and kernels ---------------------------------------------------

std::map<std::pair<int, const void *>, hipModule_t> moduleCache; // (device, blob address)
std::map<std::pair<hipModule_t, std::string>, hipFunction_t> kernelCache;
std::mutex moduleMutex;

// Decide on the host, before any HIP call, whether the blob can be a gfx950
// code object.  The reference embeds SPIR-V (magic 0x07230203, visible as
// "\03\02#\07" in test/Conversion/GPUXToLLVM/launch-func-to-gpu-runtime.mlir:5).
void validateBlob(const void *data, size_t size) {
  if (!data)
    throw std::runtime_error("gpuModuleLoad: null module data");
  if (size < 4)
    throw std::runtime_error("gpuModuleLoad: module blob of " + std::to_string(size) + " bytes is too small");
  const unsigned char *b = static_cast<const unsigned char *>(data);
  const bool spirvLE = b[0] == 0x03 && b[1] == 0x02 && b[2] == 0x23 && b[3] == 0x07;
  const bool spirvBE = b[0] == 0x07 && b[1] == 0x23 && b[2] == 0x02 && b[3] == 0x03;
  if (spirvLE || spirvBE)
    throw std::runtime_error("gpuModuleLoad: blob is SPIR-V; this runtime loads gfx950 code objects "
                             "(ELF or clang offload bundle)");
  const bool elf = b[0] == 0x7f && b[1] == 'E' && b[2] == 'L' && b[3] == 'F';
  static const char bundleMagic[] = "__CLANG_OFFLOAD_BUNDLE__";
  const bool bundle = size >= sizeof(bundleMagic) - 1 && memcmp(b, bundleMagic, sizeof(bundleMagic) - 1) == 0;
  const bool compressedBundle = b[0] == 'C' && b[1] == 'C' && b[2] == 'O' && b[3] == 'B';
  if (!elf && !bundle && !compressedBundle)
    throw std::runtime_error("gpuModuleLoad: blob is not a code object (unknown magic)");
  if (elf) {
    // e_machine (bytes 18-19, little endian) must be EM_AMDGPU = 224
    if (size < 20)
      throw std::runtime_error("gpuModuleLoad: truncated ELF header");
    const unsigned machine = b[18] | (b[19] << 8);
    if (machine != 224)
      throw std::runtime_error("gpuModuleLoad: ELF blob is for machine " + std::to_string(machine) +
                               ", not an AMDGPU code object");
  }
}

hipModule_t loadModule(GpuHipQueue *queue, const void *data, size_t size) {
  validateBlob(data, size); // a few header bytes; before any HIP call and before the stream is looked at
  if (!queue)
    throw std::runtime_error("gpuModuleLoad: null stream");
  const std::pair<int, const void *> key(queue->device, data);
  {
    std::lock_guard<std::mutex> lock(moduleMutex);
    auto it = moduleCache.find(key);
    if (it != moduleCache.end())
      return it->second;
  }
  CHECK_HIP(hipSetDevice(queue->device));
  hipModule_t module = nullptr;
  CHECK_HIP(hipModuleLoadData(&module, data));
  std::lock_guard<std::mutex> lock(moduleMutex);
  auto inserted = moduleCache.emplace(key, module);
  if (!inserted.second) { // another thread won the race
    (void)hipModuleUnload(module);
    return inserted.first->second;
  }
  return module;
}

hipFunction_t getKernel(hipModule_t module, const char *name) {
  if (!module)
    throw std::runtime_error("gpuKernelGet: null module");
  if (!name)
    throw std::runtime_error("gpuKernelGet: null kernel name");
  std::pair<hipModule_t, std::string> key(module, name);
  {
    std::lock_guard<std::mutex> lock(moduleMutex);
    auto it = kernelCache.find(key);
    if (it != kernelCache.end())
      return it->second;
  }
  hipFunction_t fn = nullptr;
  hipError_t res = hipModuleGetFunction(&fn, module, name);
  if (res != hipSuccess)
    throw std::runtime_error(std::string("gpuKernelGet: kernel '") + name + "' not found in module (" +
                             hipGetErrorString(res) + ")");
  std::lock_guard<std::mutex> lock(moduleMutex);
  kernelCache.emplace(key, fn);
  return fn;
}

// ---- launch -----------------------------------------------------------------

// LevelZeroRuntimeWrappers.cpp:99-106.
template <typename T, typename Pred> size_t countUntil(T *ptr, Pred isEnd) {
  size_t n = 0;
  if (!ptr)
    return 0;
  while (!isEnd(ptr[n]))
    ++n;
  return n;
}

struct LaunchArgs {
  hipFunction_t fn;
  unsigned grid[3];
  unsigned block[3];
  unsigned sharedMemBytes;
  std::vector<void *> kernelParams;
};

LaunchArgs makeLaunch(void *kernel, size_t gx, size_t gy, size_t gz, size_t bx, size_t by, size_t bz,
                      size_t sharedMemBytes, ImexParamDesc *params) {
  if (!kernel)
    throw std::runtime_error("gpuLaunchKernel: null kernel");
  LaunchArgs la;
  la.fn = static_cast<hipFunction_t>(kernel);
  auto cast = [](size_t v, const char *what) {
    if (v == 0 || v > 0xffffffffull)
      throw std::runtime_error(std::string("gpuLaunchKernel: ") + what + " = " + std::to_string(v) +
                               " is outside [1, 2^32)");
    return static_cast<unsigned>(v);
  };
  la.grid[0] = cast(gx, "gridX");
  la.grid[1] = cast(gy, "gridY");
  la.grid[2] = cast(gz, "gridZ");
  la.block[0] = cast(bx, "blockX");
  la.block[1] = cast(by, "blockY");
  la.block[2] = cast(bz, "blockZ");
  if (static_cast<size_t>(la.block[0]) * la.block[1] * la.block[2] > 1024)
    throw std::runtime_error("gpuLaunchKernel: more than 1024 threads per workgroup");
  // The call site passes an i32 (GPUXToLLVMPass.cpp:157); ignore the upper half.
  la.sharedMemBytes = static_cast<unsigned>(sharedMemBytes & 0xffffffffull);
  size_t count = countUntil(params, [](const ImexParamDesc &p) { return p.data == nullptr && p.size == 0; });
  // LevelZeroRuntimeWrappers.cpp:462-475: the last entry stands for dynamic
  // shared memory; on HIP that is the launch's sharedMemBytes, not an argument.
  if (la.sharedMemBytes && count)
    count -= 1;
  la.kernelParams.reserve(count);
  for (size_t i = 0; i < count; ++i)
    la.kernelParams.push_back(params[i].data);
  return la;
}

void enqueue(GpuHipQueue *queue, LaunchArgs &la) {
  CHECK_HIP(hipModuleLaunchKernel(la.fn, la.grid[0], la.grid[1], la.grid[2], la.block[0], la.block[1],
                                  la.block[2], la.sharedMemBytes, queue->stream,
                                  la.kernelParams.empty() ? nullptr : la.kernelParams.data(), nullptr));
}

void fillMemory(GpuHipQueue *q, void *dst, unsigned value, size_t count, int bits);
hipModule_t runtimeModule(GpuHipQueue *q);

// The profiler's cache flush works on a buffer of twice `bytes` (as LevelZeroRuntimeWrappers.cpp:531-538
// allocates twice the cache size): the first half is filled before every timed launch, the second half,
// zeroed once here, is then read.
void ensureFlushBuffer(GpuHipQueue *queue, size_t bytes) {
  if (queue->flushBytes >= bytes)
    return;
  if (queue->flushBuffer)
    CHECK_HIP(hipFree(queue->flushBuffer));
  queue->flushBuffer = nullptr;
  queue->flushBytes = 0;
  CHECK_HIP(hipMalloc(&queue->flushBuffer, 2 * bytes + 256));
  queue->flushBytes = bytes;
  fillMemory(queue, queue->flushBuffer, 0, (2 * bytes + 256) / 4, 32);
}

// Evict the previous run's data (LevelZeroRuntimeWrappers.cpp:524-530,564-570: a cached fill larger than
// the last-level cache), then read the buffer's other half.  The fill alone leaves the caches full of
// DIRTY lines, and their write-back would share HBM with the timed kernel; after the read they hold
// clean lines of a region the kernel does not touch.
void flushCaches(GpuHipQueue *queue, size_t bytes) {
  bytes &= ~size_t(15);
  fillMemory(queue, queue->flushBuffer, 0, bytes / 4, 32);
  hipFunction_t sweep = getKernel(runtimeModule(queue), "imex_runtime_read_sweep");
  const void *src = static_cast<const char *>(queue->flushBuffer) + bytes;
  void *sink = static_cast<char *>(queue->flushBuffer) + 2 * bytes;
  int64_t vecs = static_cast<int64_t>(bytes / 16);
  void *params[] = {&src, &vecs, &sink};
  CHECK_HIP(hipModuleLaunchKernel(sweep, 2048, 1, 1, 256, 1, 1, 0, queue->stream, params, nullptr));
}

// The profiling loop of LevelZeroRuntimeWrappers.cpp:553-583 on HIP events.
void profile(GpuHipQueue *queue, LaunchArgs &la, int warmups, int rounds, size_t flushBytes, int mode,
             float *timesMs) {
  if (rounds <= 0)
    throw std::runtime_error("profiling needs at least one run");
  CHECK_HIP(hipSetDevice(queue->device));
  if (flushBytes)
    ensureFlushBuffer(queue, flushBytes);
  hipEvent_t start, stop;
  CHECK_HIP(hipEventCreate(&start));
  CHECK_HIP(hipEventCreate(&stop));
  for (int r = 0; r < warmups; ++r)
    enqueue(queue, la);
  if (mode == 1) {
    CHECK_HIP(hipEventRecord(start, queue->stream));
    for (int r = 0; r < rounds; ++r)
      enqueue(queue, la);
    CHECK_HIP(hipEventRecord(stop, queue->stream));
    CHECK_HIP(hipEventSynchronize(stop));
    CHECK_HIP(hipEventElapsedTime(&timesMs[0], start, stop));
  } else {
    // work-item counts of the launch must fit the 32-bit arguments of the launch that takes events
    bool timestampsOnLaunch = !getenv("IMEX_PROFILING_EVENT_PAIRS");
    for (int d = 0; d < 3; ++d)
      timestampsOnLaunch = timestampsOnLaunch && uint64_t(la.grid[d]) * la.block[d] <= 0xffffffffull;
    for (int r = 0; r < rounds; ++r) {
      if (flushBytes)
        flushCaches(queue, flushBytes);
      // The reference reads the kernel's own start and end timestamps (command_start / command_end of the
      // event attached to the launch, LevelZeroRuntimeWrappers.cpp:572-582).  The launch below attaches the
      // two events to the dispatch in the same way; events recorded around it would add the stream's
      // bookkeeping between commands to a 10-40 us kernel.
      if (timestampsOnLaunch) {
        CHECK_HIP(hipExtModuleLaunchKernel(la.fn, la.grid[0] * la.block[0], la.grid[1] * la.block[1],
                                           la.grid[2] * la.block[2], la.block[0], la.block[1], la.block[2],
                                           la.sharedMemBytes, queue->stream,
                                           la.kernelParams.empty() ? nullptr : la.kernelParams.data(), nullptr,
                                           start, stop, 0));
      } else {
        CHECK_HIP(hipEventRecord(start, queue->stream));
        enqueue(queue, la);
        CHECK_HIP(hipEventRecord(stop, queue->stream));
      }
      CHECK_HIP(hipEventSynchronize(stop));
      CHECK_HIP(hipEventElapsedTime(&timesMs[r], start, stop));
    }
  }
  CHECK_HIP(hipEventDestroy(start));
  CHECK_HIP(hipEventDestroy(stop));
}

// An integer environment variable; anything unparsable or below `least` gives the fallback.
long envLong(const char *name, long fallback, long least = 1) {
  if (const char *v = getenv(name)) {
    char *end = nullptr;
    long parsed = strtol(v, &end, 10);
    if (end != v && parsed >= least)
      return parsed;
  }
  return fallback;
}

hipEvent_t materialise(LaunchEvent *le) {
  if (!le->event || le->recordedFor != le->sequence) {
    CHECK_HIP(hipSetDevice(le->queue->device));
    if (!le->event)
      CHECK_HIP(hipEventCreate(&le->event));
    CHECK_HIP(hipEventRecord(le->event, le->queue->stream));
    le->recordedFor = le->sequence;
  }
  return le->event;
}

LaunchEvent *launchKernel(GpuHipQueue *queue, void *kernel, size_t gx, size_t gy, size_t gz, size_t bx,
                          size_t by, size_t bz, size_t sharedMemBytes, ImexParamDesc *params,
                          ImexEventDesc *depEvents) {
  if (!queue)
    throw std::runtime_error("gpuLaunchKernel: null stream");
  LaunchArgs la = makeLaunch(kernel, gx, gy, gz, bx, by, bz, sharedMemBytes, params);

  size_t depCount = countUntil(depEvents, [](const ImexEventDesc &e) { return e.event == nullptr; });
  for (size_t i = 0; i < depCount; ++i) {
    LaunchEvent *dep = static_cast<LaunchEvent *>(depEvents[i].event);
    if (dep->queue == queue)
      continue; // same in-order stream: already ordered
    hipEvent_t ev = materialise(dep);
    CHECK_HIP(hipSetDevice(queue->device));
    CHECK_HIP(hipStreamWaitEvent(queue->stream, ev, 0));
  }
  CHECK_HIP(hipSetDevice(queue->device));

  if (getenv("IMEX_ENABLE_PROFILING")) {
    // Defaults of LevelZeroRuntimeWrappers.cpp:521-523; a positive
    // IMEX_PROFILING_RUNS / IMEX_PROFILING_WARMUPS overrides them.
    const int rounds = static_cast<int>(envLong("IMEX_PROFILING_RUNS", 1000));
    const int warmups = static_cast<int>(envLong("IMEX_PROFILING_WARMUPS", 3, /*least=*/0)); // 0 = no warm-up (:547-551)
    size_t flushBytes = 0;
    if (getenv("IMEX_ENABLE_CACHE_FLUSHING"))
      flushBytes = static_cast<size_t>(envLong("IMEX_CACHE_FLUSH_BYTES", 512l << 20));
    std::vector<float> times(rounds, 0.0f);
    profile(queue, la, warmups, rounds, flushBytes, 0, times.data());
    imexhip::KernelTimeStats s = imexhip::computeStats(times);
    // Same line as LevelZeroRuntimeWrappers.cpp:587-596 with the runtime's name,
    // so a grep for "execution time" (benchmarks/bench_imex.in:87-91) still finds it.
    fprintf(stdout,
            "the kernel execution time is (ms, on HIP runtime):"
            "avg: %.4f, min: %.4f, max: %.4f, median: %4f, std_deviation: %4f, "
            "variance: %4f, P95: %4f, P5: %4f, median_one_third_avg: %4f (over "
            "%d runs)\n",
            s.avg, s.min, s.max, s.median, s.stddev, s.variance, s.p95, s.p5, s.middleThirdAvg, rounds);
    fflush(stdout);
  }

  enqueue(queue, la);
  if (queue->ring.empty())
    queue->ring.assign(kEventSlots, LaunchEvent{queue, 0, nullptr, 0, false});
  LaunchEvent *done = &queue->ring[queue->launches % kEventSlots];
  done->sequence = ++queue->launches; // a HIP event left from the slot's previous life is re-recorded on first use
  return done;
}

// Default stream for the mgpu* entry points that carry no stream
// (LevelZeroRuntimeWrappers.cpp:676).
GpuHipQueue *defaultQueue() {
  struct Holder { // released when the thread ends
    GpuHipQueue *q = nullptr;
    ~Holder() { delete q; }
  };
  thread_local Holder holder;
  if (!holder.q)
    holder.q = new GpuHipQueue(defaultDeviceOrdinal(), nullptr);
  return holder.q;
}

// The fill kernels this library carries (csrc/runtime/fill.hip), embedded at build time.
extern "C" const char imex_runtime_fill_blob[], imex_runtime_fill_blob_end[];

hipModule_t runtimeModule(GpuHipQueue *q) {
  return loadModule(q, imex_runtime_fill_blob, size_t(imex_runtime_fill_blob_end - imex_runtime_fill_blob));
}

// `count` elements of `bits` (16 or 32) wide, each set to the low bits of `value`.  A kernel launch, not
// a memset on the stream: memset nodes recorded into a captured HIP graph have replayed wrongly on this
// platform, and the queue may sit on a stream its owner captures.
void fillMemory(GpuHipQueue *q, void *dst, unsigned value, size_t count, int bits) {
  if (!q)
    throw std::runtime_error("memset: null stream");
  if (count == 0)
    return;
  if (!dst)
    throw std::runtime_error("memset: null pointer with non-zero count");
  if (reinterpret_cast<uintptr_t>(dst) % (bits / 8))
    throw std::runtime_error("memset: destination is not aligned to its " + std::to_string(bits) + "-bit elements");
  CHECK_HIP(hipSetDevice(q->device));
  hipFunction_t fill = getKernel(runtimeModule(q), bits == 32 ? "imex_runtime_fill_b32" : "imex_runtime_fill_b16");
  uint32_t word = value;
  int64_t n = static_cast<int64_t>(count);
  void *params[] = {&dst, &word, &n};
  const size_t perGroup = 256 * 4 * (128 / bits); // 256 lanes, about four 16-byte stores each
  const unsigned groups = static_cast<unsigned>(std::min<size_t>((count + perGroup - 1) / perGroup, 2048));
  CHECK_HIP(hipModuleLaunchKernel(fill, groups, 1, 1, 256, 1, 1, 0, q->stream, params, nullptr));
}

GpuHipQueue *asQueue(void *p) { return static_cast<GpuHipQueue *>(p); }

} // namespace

// ===========================================================================
// IMEX gpux ABI
// ===========================================================================

extern "C" void *gpuCreateStream(void *device, void *context) {
  return catchAll([&]() -> void * {
    int ordinal = device ? *static_cast<int *>(device) : defaultDeviceOrdinal();
    return new GpuHipQueue(ordinal, static_cast<hipStream_t>(context));
  });
}

extern "C" void gpuStreamDestroy(void *queue) {
  catchAll([&]() { destroyQueue(asQueue(queue)); });
}

extern "C" void *gpuMemAlloc(void *queue, size_t size, size_t alignment, int isShared) {
  return catchAll([&]() { return allocMemory(asQueue(queue), size, alignment, (isShared & 0xff) != 0); });
}

extern "C" void gpuMemFree(void *queue, void *ptr) {
  catchAll([&]() { freeMemory(asQueue(queue), ptr); });
}

extern "C" void gpuMemCopy(void *queue, void *dst, void *src, size_t bytes) {
  catchAll([&]() { copyMemory(asQueue(queue), dst, src, bytes); });
}

extern "C" void *gpuModuleLoad(void *queue, const void *data, size_t dataSize) {
  return catchAll([&]() -> void * { return loadModule(asQueue(queue), data, dataSize); });
}

extern "C" void *gpuKernelGet(void * /*queue*/, void *module, const char *name) {
  return catchAll([&]() -> void * { return getKernel(static_cast<hipModule_t>(module), name); });
}

extern "C" void *gpuLaunchKernel(void *queue, void *kernel, size_t gridX, size_t gridY, size_t gridZ,
                                 size_t blockX, size_t blockY, size_t blockZ, size_t sharedMemBytes,
                                 void *params, void *depEvents) {
  return catchAll([&]() -> void * {
    return launchKernel(asQueue(queue), kernel, gridX, gridY, gridZ, blockX, blockY, blockZ, sharedMemBytes,
                        static_cast<ImexParamDesc *>(params), static_cast<ImexEventDesc *>(depEvents));
  });
}

extern "C" void gpuWait(void *queue) {
  catchAll([&]() {
    if (!queue)
      throw std::runtime_error("gpuWait: null stream");
    CHECK_HIP(hipSetDevice(asQueue(queue)->device));
    CHECK_HIP(hipStreamSynchronize(asQueue(queue)->stream));
  });
}

extern "C" void gpuModuleUnload(void * /*queue*/, void * /*module*/) {
  // Modules are cached for the life of the process.
}

extern "C" void gpuMemSet32(void *queue, void *dst, unsigned int value, size_t count) {
  catchAll([&]() { fillMemory(asQueue(queue), dst, value, count, 32); });
}

extern "C" void gpuMemSet16(void *queue, void *dst, unsigned short value, size_t count) {
  catchAll([&]() { fillMemory(asQueue(queue), dst, value, count, 16); });
}

// ===========================================================================
// Upstream gpu-to-llvm ABI
// ===========================================================================

extern "C" void *mgpuStreamCreate(void) {
  return catchAll([&]() -> void * { return new GpuHipQueue(defaultDeviceOrdinal(), nullptr); });
}

extern "C" void mgpuStreamSynchronize(void *stream) {
  catchAll([&]() {
    GpuHipQueue *q = stream ? asQueue(stream) : defaultQueue();
    CHECK_HIP(hipSetDevice(q->device));
    CHECK_HIP(hipStreamSynchronize(q->stream));
  });
}

extern "C" void mgpuStreamDestroy(void *stream) {
  catchAll([&]() { destroyQueue(asQueue(stream)); });
}

extern "C" void mgpuLaunchKernel(void *kernel, size_t gridX, size_t gridY, size_t gridZ, size_t blockX,
                                 size_t blockY, size_t blockZ, size_t sharedMemBytes, void *stream,
                                 void **params, void ** /*extra*/, size_t paramsCount) {
  catchAll([&]() {
    GpuHipQueue *q = stream ? asQueue(stream) : defaultQueue();
    // params[i] already points at the i-th argument's value.
    std::vector<ImexParamDesc> descs(paramsCount + 1);
    for (size_t i = 0; i < paramsCount; ++i)
      descs[i] = {params[i], sizeof(void *)};
    descs[paramsCount] = {nullptr, 0};
    LaunchArgs la = makeLaunch(kernel, gridX, gridY, gridZ, blockX, blockY, blockZ, 0, descs.data());
    la.sharedMemBytes = static_cast<unsigned>(sharedMemBytes & 0xffffffffull);
    CHECK_HIP(hipSetDevice(q->device));
    enqueue(q, la);
  });
}

extern "C" void *mgpuMemAlloc(size_t size, void *stream, int isShared) {
  return catchAll([&]() {
    GpuHipQueue *q = stream ? asQueue(stream) : defaultQueue();
    return allocMemory(q, size, 64, (isShared & 0xff) != 0);
  });
}

extern "C" void mgpuMemFree(void *stream, void *ptr) {
  catchAll([&]() { freeMemory(stream ? asQueue(stream) : defaultQueue(), ptr); });
}

extern "C" void mgpuMemcpy(void *dst, void *src, size_t bytes, void *stream) {
  catchAll([&]() { copyMemory(stream ? asQueue(stream) : defaultQueue(), dst, src, bytes); });
}

extern "C" void mgpuMemset32(void *dst, unsigned int value, size_t count, void *stream) {
  catchAll([&]() { fillMemory(stream ? asQueue(stream) : defaultQueue(), dst, value, count, 32); });
}

extern "C" void mgpuMemset16(void *dst, unsigned short value, size_t count, void *stream) {
  catchAll([&]() { fillMemory(stream ? asQueue(stream) : defaultQueue(), dst, value, count, 16); });
}

extern "C" void *mgpuModuleLoad(const void *data, size_t dataSize) {
  return catchAll([&]() -> void * { return loadModule(defaultQueue(), data, dataSize); });
}

extern "C" void *mgpuModuleGetFunction(void *module, const char *name) {
  return catchAll([&]() -> void * { return getKernel(static_cast<hipModule_t>(module), name); });
}

extern "C" void mgpuModuleUnload(void * /*module*/) {
  // These wrappers cache the module (LevelZeroRuntimeWrappers.cpp:738-741).
}

// ===========================================================================
// Measurement helpers
// ===========================================================================

extern "C" int imexHipProfileKernel(void *queue, void *kernel, size_t gridX, size_t gridY, size_t gridZ,
                                    size_t blockX, size_t blockY, size_t blockZ, size_t sharedMemBytes,
                                    void *params, int warmups, int rounds, size_t flushBytes, int mode,
                                    float *times_ms) {
  return catchAll([&]() {
    if (!queue)
      throw std::runtime_error("imexHipProfileKernel: null stream");
    if (!times_ms)
      throw std::runtime_error("imexHipProfileKernel: null output");
    LaunchArgs la = makeLaunch(kernel, gridX, gridY, gridZ, blockX, blockY, blockZ, sharedMemBytes,
                               static_cast<ImexParamDesc *>(params));
    profile(asQueue(queue), la, warmups, rounds, flushBytes, mode, times_ms);
    return 0;
  });
}

extern "C" void *imexHipRecordTimestamp(void *queue) {
  return catchAll([&]() -> void * {
    if (!queue)
      throw std::runtime_error("imexHipRecordTimestamp: null stream");
    GpuHipQueue *q = asQueue(queue);
    if (q->timestamps.empty())
      q->timestamps.assign(kTimestampSlots, LaunchEvent{q, 0, nullptr, 0, true});
    LaunchEvent *le = &q->timestamps[q->timestampCount % kTimestampSlots];
    le->sequence = ++q->timestampCount; // differs from what the slot was last recorded for: recorded anew, now
    materialise(le);
    return le;
  });
}

extern "C" float imexHipEventElapsedMs(void *startEvent, void *stopEvent) {
  return catchAll([&]() {
    if (!startEvent || !stopEvent)
      throw std::runtime_error("imexHipEventElapsedMs: null event");
    LaunchEvent *first = static_cast<LaunchEvent *>(startEvent), *second = static_cast<LaunchEvent *>(stopEvent);
    // An event returned by gpuLaunchKernel is an ordering point whose HIP event is only recorded when
    // somebody first waits on it: it carries no time of its own.
    if (!first->isTimestamp || !second->isTimestamp)
      throw std::runtime_error("imexHipEventElapsedMs: both events must come from imexHipRecordTimestamp");
    hipEvent_t a = materialise(first);
    hipEvent_t b = materialise(second);
    float ms = 0.0f;
    CHECK_HIP(hipEventSynchronize(b));
    CHECK_HIP(hipEventElapsedTime(&ms, a, b));
    return ms;
  });
}

extern "C" void imexHipComputeStats(const float *values, size_t n, float *out) {
  std::vector<float> v(values, values + n);
  imexhip::KernelTimeStats s = imexhip::computeStats(v);
  out[0] = s.avg;
  out[1] = s.min;
  out[2] = s.max;
  out[3] = s.median;
  out[4] = s.stddev;
  out[5] = s.variance;
  out[6] = s.p95;
  out[7] = s.p5;
  out[8] = s.middleThirdAvg;
}

extern "C" int imexHipQueueDevice(void *queue) { return queue ? asQueue(queue)->device : -1; }

extern "C" int imexHipDeviceInfo(void *queue, int *cuCount, int *clockKHz, size_t *l2Bytes,
                                 size_t *globalBytes, char *name, size_t nameLen) {
  int device = queue ? asQueue(queue)->device : defaultDeviceOrdinal();
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess)
    return -1;
  if (cuCount)
    *cuCount = prop.multiProcessorCount;
  if (clockKHz)
    *clockKHz = prop.clockRate;
  if (l2Bytes)
    *l2Bytes = static_cast<size_t>(prop.l2CacheSize);
  if (globalBytes)
    *globalBytes = prop.totalGlobalMem;
  if (name && nameLen) {
    snprintf(name, nameLen, "%s (%s)", prop.name, prop.gcnArchName);
  }
  return 0;
}
