/*
 * imex_runner_utils.h -- C ABI of libimex_runner_utils.so, the host-side test
 * helpers IMEX's integration tests call from JIT'd `main` functions
 * (include/imex/ExecutionEngine/ImexRunnerUtils.h:66-134,
 *  lib/ExecutionEngine/ImexRunnerUtils.cpp).
 *
 * Calling convention: with `llvm.emit_c_interface`, a `memref<*xT>` argument
 * arrives as a pointer to {int64 rank; void *descriptor}; the descriptor is
 * {T *allocated; T *aligned; int64 offset; int64 sizes[rank]; int64 strides[rank]}
 * (ImexRunnerUtils.h:36-42).  16-bit float elements are raw uint16 bit patterns.
 */
#ifndef IMEX_RUNNER_UTILS_H
#define IMEX_RUNNER_UTILS_H

#include <stdbool.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ImexUnrankedMemRef {
  int64_t rank;
  void *descriptor;
} ImexUnrankedMemRef;

/* Rank-2 instance of the ranked descriptor, for C callers that build one by hand. */
typedef struct ImexMemRef2D {
  void *allocated;
  void *aligned;
  int64_t offset;
  int64_t sizes[2];
  int64_t strides[2];
} ImexMemRef2D;

/* ImexRunnerUtils.cpp:53-73 */
void _mlir_ciface_fillResource1DBF16(ImexUnrankedMemRef *ptr, float value);
void _mlir_ciface_fillResource1DF16(ImexUnrankedMemRef *ptr, float value);
void _mlir_ciface_fillResource1DF32(ImexUnrankedMemRef *ptr, float value);

/* ImexRunnerUtils.cpp:38-50,76-99.  Uniform in [lower, upper); genInt truncates
 * each draw to an integer first.  Seeded from std::random_device like the
 * reference unless env IMEX_RANDOM_SEED gives a seed. */
void _mlir_ciface_fillResource1DRandomBF16(ImexUnrankedMemRef *ptr, float lower, float upper, bool genInt);
void _mlir_ciface_fillResource1DRandomF16(ImexUnrankedMemRef *ptr, float lower, float upper, bool genInt);
void _mlir_ciface_fillResource1DRandomF32(ImexUnrankedMemRef *ptr, float lower, float upper, bool genInt);

/* ImexRunnerUtils.cpp:101-117 */
void _mlir_ciface_printMemrefBF16(ImexUnrankedMemRef *m);
void _mlir_ciface_printMemrefF16(ImexUnrankedMemRef *m);
void printMemrefBF16(int64_t rank, void *descriptor);
void printMemrefF16(int64_t rank, void *descriptor);

/* ImexRunnerUtils.cpp:185-205,347-360: |m - n| <= 1e-4 + 1e-3 |n| everywhere. */
bool _mlir_ciface_allcloseBF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n_f32);
bool _mlir_ciface_allcloseF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n_f32);
bool _mlir_ciface_allcloseF32(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n_f32);

/* ImexRunnerUtils.cpp:207-215,362-375: prints "[ALLCLOSE: TRUE]" or "[ALLCLOSE: FALSE]". */
void _mlir_ciface_printAllcloseBF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n_f32);
void _mlir_ciface_printAllcloseF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n_f32);
void _mlir_ciface_printAllcloseF32(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n_f32);

/* ImexRunnerUtils.cpp:217-255,340-345 */
void _mlir_ciface_printMaxErrorF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n);
void _mlir_ciface_printMaxErrorBF16(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n);
void _mlir_ciface_printMaxErrorF32(ImexUnrankedMemRef *m, ImexUnrankedMemRef *n);

/* ImexRunnerUtils.cpp:257-338,385-401: C += A.B on the host, f32 accumulate in
 * i-k-j order; C is f32 storage (the F16F16F16 variant rounds the result to f16
 * and widens it back).  Contiguous row-major operands only. */
void _mlir_ciface_gemmF16F16F16(ImexUnrankedMemRef *A, ImexUnrankedMemRef *B, ImexUnrankedMemRef *C);
void _mlir_ciface_gemmF16F16F32(ImexUnrankedMemRef *A, ImexUnrankedMemRef *B, ImexUnrankedMemRef *C);
void _mlir_ciface_gemmBF16BF16F32(ImexUnrankedMemRef *A, ImexUnrankedMemRef *B, ImexUnrankedMemRef *C);

#ifdef __cplusplus
}
#endif
#endif
