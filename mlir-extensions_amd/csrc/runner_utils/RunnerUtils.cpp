//===- RunnerUtils.cpp - host-side helpers called from JIT'd test mains ----===//
//
// The `_mlir_ciface_*` utility set of IMEX's libimex_runner_utils
// (lib/ExecutionEngine/ImexRunnerUtils.cpp, include/imex/ExecutionEngine/
// ImexRunnerUtils.h:66-134): fills, printing of 16-bit float memrefs, allclose,
// max-error report and the CPU reference GEMM.  No dependency on MLIR's runner
// headers: the unranked-memref descriptor layout is restated in
// imex_runner_utils.h and walked with a small strided iterator.
//
//===----------------------------------------------------------------------===//

#include "imex_runner_utils.h"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <limits>
#include <random>
#include <vector>

namespace {

enum class Ty { F32, F16, BF16 };

float bitsToFloat(uint32_t u) {
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}
uint32_t floatToBits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}

// f16 / bf16 <-> f32.  Widening is exact; narrowing rounds to nearest even.
float halfToFloat(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1fu;
  const uint32_t man = h & 0x3ffu;
  if (exp == 0x1fu)
    return bitsToFloat(sign | 0x7f800000u | (man << 13));
  if (exp == 0) {
    // zero or subnormal: man * 2^-24
    float v = static_cast<float>(man) * 5.9604644775390625e-08f;
    return (h & 0x8000u) ? -v : v;
  }
  return bitsToFloat(sign | ((exp + 112u) << 23) | (man << 13));
}
float bfloatToFloat(uint16_t b) { return bitsToFloat(static_cast<uint32_t>(b) << 16); }

uint16_t floatToHalf(float f) {
  const uint32_t u = floatToBits(f);
  const uint16_t sign = static_cast<uint16_t>((u >> 16) & 0x8000u);
  const uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u)
    return static_cast<uint16_t>(sign | 0x7e00u);
  if (a >= 0x47800000u)
    return static_cast<uint16_t>(sign | 0x7c00u);
  if (a < 0x38800000u) {
    // Below the smallest normal half: scale so the integer part is the
    // subnormal mantissa and let the FPU round to nearest even.
    const float scaled = bitsToFloat(a) * 16777216.0f; // * 2^24
    const float rounded = std::nearbyint(scaled);
    return static_cast<uint16_t>(sign | static_cast<uint16_t>(rounded));
  }
  uint32_t r = a - 0x38000000u; // rebias exponent 127 -> 15
  r += 0xfffu + ((r >> 13) & 1u);
  return static_cast<uint16_t>(sign | static_cast<uint16_t>(r >> 13));
}
uint16_t floatToBfloat(float f) {
  uint32_t u = floatToBits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u)
    return (u & 0x80000000u) ? 0xffc0u : 0x7fc0u;
  u += ((u >> 16) & 1u) + 0x7fffu;
  return static_cast<uint16_t>(u >> 16);
}

// Strided view over an unranked memref.
struct View {
  Ty ty;
  char *base = nullptr;
  int64_t offset = 0;
  int64_t rank = 0;
  const int64_t *sizes = nullptr;
  const int64_t *strides = nullptr;

  View(ImexUnrankedMemRef *m, Ty t) : ty(t) {
    rank = m->rank;
    char *d = static_cast<char *>(m->descriptor);
    std::memcpy(&base, d + sizeof(void *), sizeof(void *)); // aligned pointer
    std::memcpy(&offset, d + 2 * sizeof(void *), sizeof(int64_t));
    sizes = reinterpret_cast<const int64_t *>(d + 2 * sizeof(void *) + sizeof(int64_t));
    strides = sizes + rank;
  }
  int elemBytes() const { return ty == Ty::F32 ? 4 : 2; }
  int64_t count() const {
    int64_t n = 1;
    for (int64_t i = 0; i < rank; ++i)
      n *= sizes[i];
    return n;
  }
  // Linear (row-major) element number -> address.
  char *at(int64_t linear) const {
    int64_t off = offset;
    for (int64_t d = rank - 1; d >= 0; --d) {
      const int64_t idx = sizes[d] ? linear % sizes[d] : 0;
      linear = sizes[d] ? linear / sizes[d] : 0;
      off += idx * strides[d];
    }
    return base + off * elemBytes();
  }
  float get(int64_t linear) const {
    const char *p = at(linear);
    if (ty == Ty::F32) {
      float f;
      std::memcpy(&f, p, 4);
      return f;
    }
    uint16_t h;
    std::memcpy(&h, p, 2);
    return ty == Ty::F16 ? halfToFloat(h) : bfloatToFloat(h);
  }
  void set(int64_t linear, float v) const {
    char *p = at(linear);
    if (ty == Ty::F32) {
      std::memcpy(p, &v, 4);
    } else {
      const uint16_t h = ty == Ty::F16 ? floatToHalf(v) : floatToBfloat(v);
      std::memcpy(p, &h, 2);
    }
  }
};

void fill(ImexUnrankedMemRef *m, Ty ty, float value) {
  View v(m, ty);
  const int64_t n = v.count();
  for (int64_t i = 0; i < n; ++i)
    v.set(i, value);
}

void fillRandom(ImexUnrankedMemRef *m, Ty ty, float lower, float upper, bool genInt) {
  std::mt19937 gen;
  if (const char *seed = getenv("IMEX_RANDOM_SEED")) {
    gen.seed(static_cast<uint32_t>(strtoul(seed, nullptr, 10)));
  } else {
    std::random_device rd;
    gen.seed(rd());
  }
  std::uniform_real_distribution<> dist(lower, upper);
  View v(m, ty);
  const int64_t n = v.count();
  for (int64_t i = 0; i < n; ++i) {
    const double d = dist(gen);
    v.set(i, genInt ? static_cast<float>(static_cast<int>(d)) : static_cast<float>(d));
  }
}

void printRec(const View &v, int64_t dim, int64_t &linear, int indent) {
  if (v.rank == 0) {
    std::cout << "[" << v.get(0) << "]";
    return;
  }
  std::cout << "[";
  for (int64_t i = 0; i < v.sizes[dim]; ++i) {
    if (dim + 1 == v.rank) {
      std::cout << v.get(linear++);
      if (i + 1 < v.sizes[dim])
        std::cout << ",   ";
    } else {
      printRec(v, dim + 1, linear, indent + 1);
      if (i + 1 < v.sizes[dim]) {
        std::cout << ", \n";
        for (int s = 0; s <= indent; ++s)
          std::cout << " ";
      }
    }
  }
  std::cout << "]";
}

void printMemref(ImexUnrankedMemRef *m, Ty ty) {
  View v(m, ty);
  std::cout << "Unranked Memref base@ = " << static_cast<void *>(v.base) << " rank = " << v.rank
            << " offset = " << v.offset << " sizes = [";
  for (int64_t i = 0; i < v.rank; ++i)
    std::cout << v.sizes[i] << (i + 1 < v.rank ? ", " : "");
  std::cout << "] strides = [";
  for (int64_t i = 0; i < v.rank; ++i)
    std::cout << v.strides[i] << (i + 1 < v.rank ? ", " : "");
  std::cout << "] data = \n";
  int64_t linear = 0;
  printRec(v, 0, linear, 0);
  std::cout << "\n";
}

// |lhs - rhs| > atol + rtol |rhs| anywhere -> false; all in f32, like the
// reference (a NaN difference therefore does not fail).
bool allclose(ImexUnrankedMemRef *m, Ty ty, ImexUnrankedMemRef *n) {
  const float atol = 1e-04f, rtol = 1e-03f;
  View a(m, ty), b(n, Ty::F32);
  const int64_t count = std::min(a.count(), b.count());
  for (int64_t i = 0; i < count; ++i) {
    const float lhs = a.get(i), rhs = b.get(i);
    if (std::fabs(lhs - rhs) > atol + rtol * std::fabs(rhs))
      return false;
  }
  return true;
}

void printAllclose(ImexUnrankedMemRef *m, Ty ty, ImexUnrankedMemRef *n) {
  std::cout << (allclose(m, ty, n) ? "[ALLCLOSE: TRUE]\n" : "[ALLCLOSE: FALSE]\n");
}

void printMaxError(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n, Ty ty) {
  View a(m, ty), b(n, ty);
  const int64_t count = std::min(a.count(), b.count());
  double maxAbs = 0.0, maxRel = 0.0;
  int64_t absIdx = 0, relIdx = 0;
  const double inf = std::numeric_limits<double>::infinity();
  double absI = inf, absJ = inf, relI = inf, relJ = inf;
  for (int64_t i = 0; i < count; ++i) {
    const double x = a.get(i), y = b.get(i);
    const double delta = std::fabs(x - y);
    const double rel = delta / std::fmax(std::fabs(x), std::fabs(y));
    if (delta > maxAbs) {
      maxAbs = delta; absIdx = i; absI = x; absJ = y;
    }
    if (rel > maxRel) {
      maxRel = rel; relIdx = i; relI = x; relJ = y;
    }
  }
  std::cout << "Max absolute error " << maxAbs << " at idx=" << absIdx << " (i=" << absI << ", j=" << absJ << ")\n";
  std::cout << "Max relative error " << maxRel << " at idx=" << relIdx << " (i=" << relI << ", j=" << relJ << ")\n";
}

// C += A.B with f32 accumulation in i-k-j order, operands widened to f32 first.
void gemm(ImexUnrankedMemRef *A, ImexUnrankedMemRef *B, ImexUnrankedMemRef *C, Ty abTy, Ty roundTo) {
  View a(A, abTy), b(B, abTy), c(C, Ty::F32);
  if (a.rank != 2 || b.rank != 2 || c.rank != 2) {
    std::cout << "Expecting 2D memrefs, got A rank: " << a.rank << ", B rank: " << b.rank << ", C rank: " << c.rank
              << '\n';
    return;
  }
  if (a.sizes[1] != b.sizes[0] || a.sizes[0] != c.sizes[0] || b.sizes[1] != c.sizes[1]) {
    std::cout << "Incompatible matrix dimensions: A: [" << a.sizes[0] << ", " << a.sizes[1] << "], B: ["
              << b.sizes[0] << ", " << b.sizes[1] << "], C: [" << c.sizes[0] << ", " << c.sizes[1] << "]\n";
    return;
  }
  auto contiguous = [](const View &v) { return v.strides[0] == v.sizes[1] && v.strides[1] == 1; };
  if (!contiguous(a) || !contiguous(b) || !contiguous(c)) {
    std::cout << "Expecting A strides to be [M, 1], B strides to be [K, 1], C strides to be [M, 1]\n";
    return;
  }
  const int64_t M = a.sizes[0], N = b.sizes[1], K = a.sizes[1];
  std::vector<float> fa(static_cast<size_t>(M * K)), fb(static_cast<size_t>(K * N)), fc(static_cast<size_t>(M * N));
  for (int64_t i = 0; i < M * K; ++i) fa[i] = a.get(i);
  for (int64_t i = 0; i < K * N; ++i) fb[i] = b.get(i);
  for (int64_t i = 0; i < M * N; ++i) fc[i] = c.get(i);
  for (int64_t i = 0; i < M; ++i)
    for (int64_t k = 0; k < K; ++k) {
      const float av = fa[i * K + k];
      const float *brow = &fb[k * N];
      float *crow = &fc[i * N];
      for (int64_t j = 0; j < N; ++j)
        crow[j] += av * brow[j];
    }
  for (int64_t i = 0; i < M * N; ++i) {
    float r = fc[i];
    if (roundTo == Ty::F16)
      r = halfToFloat(floatToHalf(r));
    else if (roundTo == Ty::BF16)
      r = bfloatToFloat(floatToBfloat(r));
    c.set(i, r);
  }
}

} // namespace

extern "C" {

void _mlir_ciface_fillResource1DBF16(ImexUnrankedMemRef *p, float v) { fill(p, Ty::BF16, v); }
void _mlir_ciface_fillResource1DF16(ImexUnrankedMemRef *p, float v) { fill(p, Ty::F16, v); }
void _mlir_ciface_fillResource1DF32(ImexUnrankedMemRef *p, float v) { fill(p, Ty::F32, v); }

void _mlir_ciface_fillResource1DRandomBF16(ImexUnrankedMemRef *p, float lo, float hi, bool genInt) {
  fillRandom(p, Ty::BF16, lo, hi, genInt);
}
void _mlir_ciface_fillResource1DRandomF16(ImexUnrankedMemRef *p, float lo, float hi, bool genInt) {
  fillRandom(p, Ty::F16, lo, hi, genInt);
}
void _mlir_ciface_fillResource1DRandomF32(ImexUnrankedMemRef *p, float lo, float hi, bool genInt) {
  fillRandom(p, Ty::F32, lo, hi, genInt);
}

void _mlir_ciface_printMemrefBF16(ImexUnrankedMemRef *m) { printMemref(m, Ty::BF16); }
void _mlir_ciface_printMemrefF16(ImexUnrankedMemRef *m) { printMemref(m, Ty::F16); }
void printMemrefBF16(int64_t rank, void *descriptor) {
  ImexUnrankedMemRef m = {rank, descriptor};
  printMemref(&m, Ty::BF16);
}
void printMemrefF16(int64_t rank, void *descriptor) {
  ImexUnrankedMemRef m = {rank, descriptor};
  printMemref(&m, Ty::F16);
}

bool _mlir_ciface_allcloseBF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n) { return allclose(m, Ty::BF16, n); }
bool _mlir_ciface_allcloseF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n) { return allclose(m, Ty::F16, n); }
bool _mlir_ciface_allcloseF32(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n) { return allclose(m, Ty::F32, n); }

void _mlir_ciface_printAllcloseBF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n) { printAllclose(m, Ty::BF16, n); }
void _mlir_ciface_printAllcloseF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n) { printAllclose(m, Ty::F16, n); }
void _mlir_ciface_printAllcloseF32(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n) { printAllclose(m, Ty::F32, n); }

void _mlir_ciface_printMaxErrorF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n) { printMaxError(m, n, Ty::F16); }
void _mlir_ciface_printMaxErrorBF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n) { printMaxError(m, n, Ty::BF16); }
void _mlir_ciface_printMaxErrorF32(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n) { printMaxError(m, n, Ty::F32); }

void _mlir_ciface_gemmF16F16F16(ImexUnrankedMemRef *A, ImexUnrankedMemRef *B, ImexUnrankedMemRef *C) {
  gemm(A, B, C, Ty::F16, Ty::F16);
}
void _mlir_ciface_gemmF16F16F32(ImexUnrankedMemRef *A, ImexUnrankedMemRef *B, ImexUnrankedMemRef *C) {
  gemm(A, B, C, Ty::F16, Ty::F32);
}
void _mlir_ciface_gemmBF16BF16F32(ImexUnrankedMemRef *A, ImexUnrankedMemRef *B, ImexUnrankedMemRef *C) {
  gemm(A, B, C, Ty::BF16, Ty::F32);
}

} // extern "C"
