// The runtime library's own device code: 32-bit and 16-bit pattern fills.
//
// mgpuMemset32 / mgpuMemset16 (callee names of upstream MLIR's gpu.memset lowering; the reference's
// wrapper has no counterpart) and gpuMemSet32 / gpuMemSet16 run these kernels instead of recording a memset on the stream, so that a caller
// who captures the stream into a HIP graph gets an ordinary kernel node.
//
// imex_runtime_read_sweep is the second half of the profiler's cache flush: it reads a region that
// nothing else uses, so that every cache level ends up holding clean lines of that region -- neither
// the timed kernel's data nor dirty lines of the fill, which would otherwise be written back to HBM
// while the timed kernel runs.
//
// Launch: block (256,1,1), any grid (workgroups stride over the buffer).

#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" __global__ __launch_bounds__(256) void imex_runtime_fill_b32(uint32_t *dst, uint32_t value, int64_t n) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const int64_t tid = int64_t(blockIdx.x) * 256 + threadIdx.x;
  const int64_t threads = int64_t(gridDim.x) * 256;
  // words before the first 16-byte boundary, then whole vectors, then the tail
  const int64_t head = min(n, int64_t((16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15) / 4);
  const int64_t vecs = (n - head) / 4;
  for (int64_t i = tid; i < head; i += threads)
    dst[i] = value;
  u32x4 *body = reinterpret_cast<u32x4 *>(dst + head);
  const u32x4 v = {value, value, value, value};
  for (int64_t i = tid; i < vecs; i += threads)
    body[i] = v;
  for (int64_t i = head + vecs * 4 + tid; i < n; i += threads)
    dst[i] = value;
}

// 16-bit pattern: single elements up to the first 16-byte boundary, whole vectors, then the tail.
extern "C" __global__ __launch_bounds__(256) void imex_runtime_fill_b16(uint16_t *dst, uint32_t value, int64_t n) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const int64_t tid = int64_t(blockIdx.x) * 256 + threadIdx.x;
  const int64_t threads = int64_t(gridDim.x) * 256;
  const uint16_t v16 = static_cast<uint16_t>(value);
  const int64_t head = min(n, int64_t((16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15) / 2);
  const int64_t vecs = (n - head) / 8;
  for (int64_t i = tid; i < head; i += threads)
    dst[i] = v16;
  u32x4 *body = reinterpret_cast<u32x4 *>(dst + head);
  const uint32_t w = uint32_t(v16) | (uint32_t(v16) << 16);
  const u32x4 v = {w, w, w, w};
  for (int64_t i = tid; i < vecs; i += threads)
    body[i] = v;
  for (int64_t i = head + vecs * 8 + tid; i < n; i += threads)
    dst[i] = v16;
}

// Reads `vecs` 16-byte vectors.  The store can never happen on a zero-filled region; it only keeps the loads.
extern "C" __global__ __launch_bounds__(256) void imex_runtime_read_sweep(const uint32_t *src, int64_t vecs,
                                                                          uint32_t *sink) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const u32x4 *body = reinterpret_cast<const u32x4 *>(src);
  const int64_t tid = int64_t(blockIdx.x) * 256 + threadIdx.x;
  const int64_t threads = int64_t(gridDim.x) * 256;
  uint32_t seen = 0;
  for (int64_t i = tid; i < vecs; i += threads) {
    const u32x4 v = body[i];
    seen |= v.x | v.y | v.z | v.w;
  }
  if (seen == 0x9e3779b9u)
    *sink = seen;
}
