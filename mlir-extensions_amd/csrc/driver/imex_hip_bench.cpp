//===- imex_hip_bench.cpp - C++ host driver over the gpu* runtime ABI ------===//
//
// Does, in plain C++ through the C ABI only, what IMEX's JIT'd `main` plus the
// `bench_imex` script do for one benchmark workload
// (benchmarks/bench_imex.in:23-92, lib/Conversion/GPUXToLLVM/GPUXToLLVMPass.cpp:
// 373-383,508-518,691-710):
//
//   gpuCreateStream -> gpuMemAlloc -> fill on the host -> gpuMemCopy (H2D) ->
//   gpuModuleLoad + gpuKernelGet + gpuLaunchKernel(ParamDesc[]) -> gpuWait ->
//   gpuMemCopy (D2H) -> gpuMemFree -> gpuStreamDestroy
//
// and prints one "<workload>: the kernel execution time is (ms, on HIP
// runtime):avg: ..." line per workload, the line bench_imex greps into
// report.txt (bench_imex.in:87-91).
//
//   imex-hip-bench [-l] [--runs N] [--warmups W] [--flush] [--zeros] [--rotate S] [--grid G] [--launch-only N] <workload>...
//   imex-hip-bench --list
//   imex-hip-bench --lds-service       (LDS lane-grouping / bank-period probe, for a bank-conflict counter run)
//   imex-hip-bench [-l] --report report.txt <workload>...|all|operators
//
//   --report FILE  bench_imex's outer loop (bench_imex.in:72-91): one child process per workload,
//                  their output echoed, every "execution time" line collected in FILE under an
//                  "Imex Perf (HIP) @ <date>" header.  The parent never touches the GPU.
//   -c             bench_imex's CPU mode is not offered: the CPU lowering stays IMEX's own pipeline
//   -l             accepted for bench_imex compatibility (the HIP runtime is the only backend here)
//   --zeros        all-zero inputs instead of random ones: MFMA power, and with it the clock the
//                  part sustains, depends on operand values; this shows the kernel at full clock
//   --rotate S     S separate copies of the workload's tensors, launches walking round them: with S x footprint
//                  beyond the 256 MiB Infinity Cache every launch streams from HBM (back-to-back figure and
//                  --launch-only runs; the per-launch statistics stay on the first set)
//   --grid G       launch G x 1 x 1 workgroups instead of the catalogue's grid (the kernels stride over their work)
//   --launch-only  skip the timing loop and just launch the kernel N times (for
//                  rocprofv3 counter runs, which time and count every dispatch themselves)
//
//===----------------------------------------------------------------------===//

#include "imex_hip_kernels.h"
#include "imex_hip_runtime.h"
#include "imex_runner_utils.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <string>
#include <vector>

#include <unistd.h>

namespace {

enum class Elem { F32, F16, BF16 };
size_t elemBytes(Elem e) { return e == Elem::F32 ? 4 : 2; }

struct Tensor {
  Elem elem;
  std::vector<int64_t> shape;
  bool isInput;
  float lo, hi; // uniform fill range for inputs
};

struct Workload {
  const char *name;
  const char *kernel;
  std::vector<int64_t> dims;    // what imexHipKernelLaunchShape takes
  std::vector<Tensor> tensors;  // kernel pointer arguments, in order
  std::vector<int64_t> indexArgs; // i64 arguments after the pointers
  int floatArg;                 // 0 none; 1 trailing f32 `init` (reductions); 2 f32 between pointers and indices (sm_scale)
  double work;                  // algorithmic bytes or flops per launch
  bool mfma;                    // roofline: MFMA (TFLOP/s) or HBM (GB/s)
  bool probe = false;           // a measurement kernel: loaded from imex_probe.hsaco beside this program
  int probeGrid = 0;            // its grid (workgroups of probeBlock lanes); 0: one lane per dims[0]
  int probeBlock = 512;
};

std::vector<Workload> workloads() {
  const int64_t K4 = 4096, K8 = 8192;
  return {
      {"relu_f32_4096x4096", "imex_relu_f32", {K4 * K4},
       {{Elem::F32, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}}, {K4 * K4}, 0,
       2.0 * K4 * K4 * 4, false},
      {"silu_f32_512x640x20x15", "imex_silu_f32", {98304000},
       {{Elem::F32, {98304000}, true, -8, 8}, {Elem::F32, {98304000}, 0, 0, 0}}, {98304000}, 0,
       2.0 * 98304000 * 4, false},
      {"silu_f16_512x640x20x15", "imex_silu_f16", {98304000},
       {{Elem::F16, {98304000}, true, -8, 8}, {Elem::F16, {98304000}, 0, 0, 0}}, {98304000}, 0,
       2.0 * 98304000 * 2, false},
      {"silu_bf16_512x640x20x15", "imex_silu_bf16", {98304000},
       {{Elem::BF16, {98304000}, true, -8, 8}, {Elem::BF16, {98304000}, 0, 0, 0}}, {98304000}, 0,
       2.0 * 98304000 * 2, false},
      {"relu_f16_512x640x20x15", "imex_relu_f16", {98304000},
       {{Elem::F16, {98304000}, true, -8, 8}, {Elem::F16, {98304000}, 0, 0, 0}}, {98304000}, 0,
       2.0 * 98304000 * 2, false},
      {"softmax_f16_16384x1024", "imex_softmax_f16", {16384, 1024},
       {{Elem::F16, {16384, 1024}, true, -4, 4}, {Elem::F16, {16384, 1024}, 0, 0, 0}}, {16384, 1024}, 0,
       2.0 * 16384 * 1024 * 2, false},
      {"rowsum_f32_8192x8192", "imex_rowsum_f32", {K8, K8},
       {{Elem::F32, {K8, K8}, 1, 0, 1}, {Elem::F32, {K8}, false, 0, 0}}, {K8, K8}, 1,
       K8 * K8 * 4.0 + K8 * 4.0, false},
      {"transpose_bf16_8192x8192", "imex_transpose2d_b16", {K8, K8},
       {{Elem::BF16, {K8, K8}, 1, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8}, 0,
       2.0 * K8 * K8 * 2, false},
      {"transpose_f32_4096x4096", "imex_transpose2d_b32", {K4, K4},
       {{Elem::F32, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}}, {K4, K4}, 0,
       2.0 * K4 * K4 * 4, false},
      {"gemm_f16_4096", "imex_gemm_f16_f16_f32", {K4, K4, K4},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true},
      // the reference's bias kernel with its own argument order (bias, C, A, B): C = bias[n] + (C + A.B)
      // (WG/gemm_4kx4kx4k_f16_f16_f32_bias.mlir:77-116); C is input and output
      {"gemm_f16_4096_bias", "imex_gemm_4kx4kx4k_f16_f16_f32_bias", {},
       {{Elem::F32, {K4}, true, -1, 1}, {Elem::F32, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -0.5f, 0.5f},
        {Elem::F16, {K4, K4}, true, -0.5f, 0.5f}},
       {}, 0, 2.0 * K4 * K4 * K4, true},
      {"gemm_f16_4096_f16_out", "imex_gemm_f16_f16_f16", {K4, K4, K4},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true},
      {"gemm_bf16_4096", "imex_gemm_bf16_bf16_f32", {K4, K4, K4},
       {{Elem::BF16, {K4, K4}, true, -1, 1}, {Elem::BF16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true},
      {"gemm_f16_4096_transpose_b", "imex_gemm_f16_f16_f32_tb", {K4, K4, K4},
       {{Elem::F16, {K4, K4}, true, -0.5f, 0.5f}, {Elem::F16, {K4, K4}, true, -0.5f, 0.5f}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true},
      {"gemm_f16_4096_transpose_a", "imex_gemm_f16_f16_f32_ta", {K4, K4, K4},
       {{Elem::F16, {K4, K4}, true, -0.5f, 0.5f}, {Elem::F16, {K4, K4}, true, -0.5f, 0.5f}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true},
      {"gemm_mlp_bf16_4096x11008x4096", "imex_gemm_bf16_bias_silu_bf16", {K4, 11008, K4},
       {{Elem::BF16, {K4, K4}, true, -1.7f, 1.7f}, {Elem::BF16, {K4, 11008}, true, -0.035f, 0.035f},
        {Elem::F32, {11008}, true, -0.17f, 0.17f}, {Elem::BF16, {K4, 11008}, false, 0, 0}},
       {K4, 11008, K4}, 0, 2.0 * K4 * 11008 * K4, true},
      // flash attention forward, the reference's shape: Z = 2, H = 2, N_CTX = 4096, D = 64, scale 0.5;
      // 4 Z H N^2 D FLOP (two products)
      {"flash_attention_f16_2x2x4096x64", "imex_flash_attention_fwd_f16", {4, K4},
       {{Elem::F16, {4 * K4, 64}, true, -1, 1}, {Elem::F16, {4 * K4, 64}, true, -1, 1},
        {Elem::F16, {4 * K4, 64}, true, -1, 1}, {Elem::F16, {4 * K4, 64}, false, 0, 0}},
       {4, K4}, 2, 4.0 * 4 * K4 * K4 * 64, true},
      // the reference's second attention shape (flash_attention_fwd_ov_with_arrray_len_4k.mlir:23): 16 heads
      {"flash_attention_f16_16x4096x64", "imex_flash_attention_fwd_f16", {16, K4},
       {{Elem::F16, {16 * K4, 64}, true, -1, 1}, {Elem::F16, {16 * K4, 64}, true, -1, 1},
        {Elem::F16, {16 * K4, 64}, true, -1, 1}, {Elem::F16, {16 * K4, 64}, false, 0, 0}},
       {16, K4}, 2, 4.0 * 16 * K4 * K4 * 64, true},
      // shapes of the reference's benchmark suite (README.md:330-335) beyond the ones above
      {"relu_f32_512x640x20x15", "imex_relu_f32", {98304000},
       {{Elem::F32, {98304000}, true, -1, 1}, {Elem::F32, {98304000}, false, 0, 0}}, {98304000}, 0,
       2.0 * 98304000 * 4, false},
      {"reduce_outer_f32_32x16x512x512", "imex_reduce_outer_f32", {32, 16 * 512 * 512},
       {{Elem::F32, {32, 16 * 512 * 512}, true, 0, 1}, {Elem::F32, {16 * 512 * 512}, false, 0, 0}},
       {32, 16 * 512 * 512}, 1, 33.0 * 16 * 512 * 512 * 4, false},
      {"softmax_f32_1024x2000", "imex_softmax_f32", {1024, 2000},
       {{Elem::F32, {1024, 2000}, true, -4, 4}, {Elem::F32, {1024, 2000}, false, 0, 0}}, {1024, 2000}, 0,
       2.0 * 1024 * 2000 * 4, false},
      {"transpose_f32_1024x1024", "imex_transpose2d_b32", {1024, 1024},
       {{Elem::F32, {1024, 1024}, true, -1, 1}, {Elem::F32, {1024, 1024}, false, 0, 0}}, {1024, 1024}, 0,
       2.0 * 1024 * 1024 * 4, false},
      {"transpose3d_f32_16x96x96", "imex_transpose3d_b32", {16, 96, 96},
       {{Elem::F32, {16, 96, 96}, true, -1, 1}, {Elem::F32, {96, 96, 16}, false, 0, 0}}, {16, 96, 96}, 0,
       2.0 * 16 * 96 * 96 * 4, false},
      // the fused chains at the benchmark's own size (launch-bound) and at one that streams from HBM
      {"exp_f32_256x256", "imex_exp_f32", {256 * 256},
       {{Elem::F32, {256 * 256}, true, -0.5f, 0.5f}, {Elem::F32, {256 * 256}, false, 0, 0}}, {256 * 256}, 0,
       2.0 * 256 * 256 * 4, false},
      {"maximum_f32_256x256", "imex_maximum_f32", {256 * 256},
       {{Elem::F32, {256 * 256}, true, -0.5f, 0.5f}, {Elem::F32, {256 * 256}, true, -0.5f, 0.5f},
        {Elem::F32, {256 * 256}, false, 0, 0}}, {256 * 256}, 0, 3.0 * 256 * 256 * 4, false},
      {"loop_fusion_f32_512x1024", "imex_loop_fusion_f32", {512 * 1024},
       {{Elem::F32, {512 * 1024}, true, 0.5f, 3}, {Elem::F32, {512 * 1024}, true, -3, 3},
        {Elem::F32, {512 * 1024}, false, 0, 0}}, {512 * 1024}, 0, 3.0 * 512 * 1024 * 4, false},
      {"loop_fusion_f32_4096x4096", "imex_loop_fusion_f32", {K4 * K4},
       {{Elem::F32, {K4 * K4}, true, 0.5f, 3}, {Elem::F32, {K4 * K4}, true, -3, 3}, {Elem::F32, {K4 * K4}, false, 0, 0}},
       {K4 * K4}, 0, 3.0 * K4 * K4 * 4, false},
      {"input_fusion_f32_512x1024", "imex_input_fusion_f32", {512, 1024},
       {{Elem::F32, {512, 1024}, true, -3, 3}, {Elem::F32, {512, 1024}, true, 0.5f, 3}, {Elem::F32, {1024}, false, 0, 0}},
       {512, 1024}, 0, 2.0 * 512 * 1024 * 4 + 1024 * 4, false},
      {"input_fusion_f32_8192x8192", "imex_input_fusion_f32", {K8, K8},
       {{Elem::F32, {K8, K8}, true, -3, 3}, {Elem::F32, {K8, K8}, true, 0.5f, 3}, {Elem::F32, {K8}, false, 0, 0}},
       {K8, K8}, 0, 2.0 * K8 * K8 * 4 + K8 * 4, false},
      // not operators (and not in the catalogue): the MFMA pipe fed from LDS with nothing else going on, one
      // workgroup per CU, on f16 operands uniform in (-1,1) like the GEMM benchmark's, on zeros, and on f16 with
      // every exponent equally likely -- the rate the operand values allow
      {"mfma_lds_ceiling_f16_uniform", "imex_mfma_lds_ceiling_f16", {256 * 512},
       {{Elem::F32, {256 * 512}, false, 0, 0}}, {256 * 512, 2048, 0}, 0, 256.0 * 8 * 2048 * 32 * 16384, true, true},
      {"mfma_lds_ceiling_f16_zeros", "imex_mfma_lds_ceiling_f16", {256 * 512},
       {{Elem::F32, {256 * 512}, false, 0, 0}}, {256 * 512, 2048, 1}, 0, 256.0 * 8 * 2048 * 32 * 16384, true, true},
      // the GEMM's tile code with one part switched off (timing only: the results are meaningless)
      {"gemm_f16_4096_probe_no_loop_copies", "imex_gemm_probe_no_loop_copies", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      {"gemm_f16_4096_probe_no_epilogue", "imex_gemm_probe_no_epilogue", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      {"gemm_f16_4096_probe_multiply_only", "imex_gemm_probe_multiply_only", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      {"gemm_f16_4096_probe_store_nontemporal", "imex_gemm_probe_store_nontemporal", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      {"gemm_mlp_bf16_probe_store_nontemporal", "imex_gemm_probe_mlp_store_nontemporal", {},
       {{Elem::BF16, {K4, K4}, true, -1.7f, 1.7f}, {Elem::BF16, {K4, 11008}, true, -0.035f, 0.035f},
        {Elem::F32, {11008}, true, -0.17f, 0.17f}, {Elem::BF16, {K4, 11008}, false, 0, 0}},
       {K4, 11008, K4}, 0, 2.0 * K4 * 11008 * K4, true, true, 688},
      {"gemm_f16_4096_probe_store_lines", "imex_gemm_probe_store_lines", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      {"gemm_f16_4096_probe_copies_only", "imex_gemm_probe_copies_only", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      {"gemm_f16_4096_probe_copies_only_a", "imex_gemm_probe_copies_only_a", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      {"gemm_f16_4096_probe_copies_only_b", "imex_gemm_probe_copies_only_b", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      {"gemm_f16_4096_probe_narrow_a", "imex_gemm_probe_narrow_a", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      {"gemm_f16_4096_probe_narrow_a_copies_only", "imex_gemm_probe_narrow_a_copies_only", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      {"gemm_f16_4096_probe_narrow_a_copies_only_a", "imex_gemm_probe_narrow_a_copies_only_a", {},
       {{Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F16, {K4, K4}, true, -1, 1}, {Elem::F32, {K4, K4}, false, 0, 0}},
       {K4, K4, K4}, 0, 2.0 * K4 * K4 * K4, true, true, 256},
      // the 16-bit transpose's traffic without the transposition: 256 x 256 tiles copied to their own / to the
      // transposed tile position, at the benchmark's 16 KiB row pitch and at 32 KiB; and the transpose itself at 32 KiB
      {"tile_copy_b16_8192x8192_own", "imex_probe_tile_copy_b16", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8, 0}, 0,
       2.0 * K8 * K8 * 2, false, true, 32 * 32, 256},
      {"tile_copy_b16_8192x8192_transposed", "imex_probe_tile_copy_b16", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8, 1}, 0,
       2.0 * K8 * K8 * 2, false, true, 32 * 32, 256},
      {"tile_copy_b16_16384x16384_own", "imex_probe_tile_copy_b16", {2 * K8, 2 * K8},
       {{Elem::BF16, {2 * K8, 2 * K8}, true, -1, 1}, {Elem::BF16, {2 * K8, 2 * K8}, false, 0, 0}}, {2 * K8, 2 * K8, 0}, 0,
       2.0 * 4 * K8 * K8 * 2, false, true, 64 * 64, 256},
      {"tile_copy_b16_16384x16384_transposed", "imex_probe_tile_copy_b16", {2 * K8, 2 * K8},
       {{Elem::BF16, {2 * K8, 2 * K8}, true, -1, 1}, {Elem::BF16, {2 * K8, 2 * K8}, false, 0, 0}}, {2 * K8, 2 * K8, 1}, 0,
       2.0 * 4 * K8 * K8 * 2, false, true, 64 * 64, 256},
      // the traffic of a tile-wise 16-bit transpose for other tile shapes (R x C: 2 C-byte read, 2 R-byte write segments)
      {"tile_traffic_b16_8192x8192_256x256", "imex_probe_tile_traffic_b16_256x256", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8}, 0,
       2.0 * K8 * K8 * 2, false, true, int(K8 / 256 * K8 / 256), 256},
      {"tile_traffic_b16_8192x8192_128x128", "imex_probe_tile_traffic_b16_128x128", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8}, 0,
       2.0 * K8 * K8 * 2, false, true, int(K8 / 128 * K8 / 128), 256},
      {"tile_traffic_b16_8192x8192_512x128", "imex_probe_tile_traffic_b16_512x128", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8}, 0,
       2.0 * K8 * K8 * 2, false, true, int(K8 / 512 * K8 / 128), 256},
      {"tile_traffic_b16_8192x8192_128x512", "imex_probe_tile_traffic_b16_128x512", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8}, 0,
       2.0 * K8 * K8 * 2, false, true, int(K8 / 128 * K8 / 512), 256},
      {"tile_traffic_b16_8192x8192_512x256", "imex_probe_tile_traffic_b16_512x256", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8}, 0,
       2.0 * K8 * K8 * 2, false, true, int(K8 / 512 * K8 / 256), 512},
      {"tile_traffic_b16_8192x8192_256x512", "imex_probe_tile_traffic_b16_256x512", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8}, 0,
       2.0 * K8 * K8 * 2, false, true, int(K8 / 256 * K8 / 512), 512},
      {"tile_traffic_b16_8192x8192_1024x128", "imex_probe_tile_traffic_b16_1024x128", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8}, 0,
       2.0 * K8 * K8 * 2, false, true, int(K8 / 1024 * K8 / 128), 512},
      {"tile_traffic_b16_8192x8192_512x512", "imex_probe_tile_traffic_b16_512x512", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8}, 0,
       2.0 * K8 * K8 * 2, false, true, int(K8 / 512 * K8 / 512), 1024},
      // reads alone and writes alone at the two pitches (half the bytes of a copy each), and the copy with a pass's rows spread out
      {"tile_read_b16_8192x16384", "imex_probe_tile_copy_b16", {K8, 2 * K8},
       {{Elem::BF16, {K8, 2 * K8}, true, -1, 1}, {Elem::BF16, {K8, 2 * K8}, false, 0, 0}}, {K8, 2 * K8, 2}, 0,
       2.0 * K8 * K8 * 2, false, true, 32 * 64, 256},
      {"tile_read_b16_16384x8192", "imex_probe_tile_copy_b16", {2 * K8, K8},
       {{Elem::BF16, {2 * K8, K8}, true, -1, 1}, {Elem::BF16, {2 * K8, K8}, false, 0, 0}}, {2 * K8, K8, 2}, 0,
       2.0 * K8 * K8 * 2, false, true, 64 * 32, 256},
      {"tile_write_b16_8192x16384", "imex_probe_tile_copy_b16", {K8, 2 * K8},
       {{Elem::BF16, {K8, 2 * K8}, true, -1, 1}, {Elem::BF16, {K8, 2 * K8}, false, 0, 0}}, {K8, 2 * K8, 3}, 0,
       2.0 * K8 * K8 * 2, false, true, 32 * 64, 256},
      {"tile_write_b16_16384x8192", "imex_probe_tile_copy_b16", {2 * K8, K8},
       {{Elem::BF16, {2 * K8, K8}, true, -1, 1}, {Elem::BF16, {2 * K8, K8}, false, 0, 0}}, {2 * K8, K8, 3}, 0,
       2.0 * K8 * K8 * 2, false, true, 64 * 32, 256},
      {"tile_copy_b16_16384x8192_own_rows_apart", "imex_probe_tile_copy_b16", {2 * K8, K8},
       {{Elem::BF16, {2 * K8, K8}, true, -1, 1}, {Elem::BF16, {2 * K8, K8}, false, 0, 0}}, {2 * K8, K8, 4}, 0,
       2.0 * 2 * K8 * K8 * 2, false, true, 64 * 32, 256},
      {"tile_copy_b16_8192x8192_transposed_rows_apart", "imex_probe_tile_copy_b16", {K8, K8},
       {{Elem::BF16, {K8, K8}, true, -1, 1}, {Elem::BF16, {K8, K8}, false, 0, 0}}, {K8, K8, 5}, 0,
       2.0 * K8 * K8 * 2, false, true, 32 * 32, 256},
      // equal bytes at the two pitches: 8192 rows of 32 KiB against 16384 rows of 16 KiB
      {"tile_copy_b16_8192x16384_own", "imex_probe_tile_copy_b16", {K8, 2 * K8},
       {{Elem::BF16, {K8, 2 * K8}, true, -1, 1}, {Elem::BF16, {K8, 2 * K8}, false, 0, 0}}, {K8, 2 * K8, 0}, 0,
       2.0 * 2 * K8 * K8 * 2, false, true, 32 * 64, 256},
      {"tile_copy_b16_16384x8192_own", "imex_probe_tile_copy_b16", {2 * K8, K8},
       {{Elem::BF16, {2 * K8, K8}, true, -1, 1}, {Elem::BF16, {2 * K8, K8}, false, 0, 0}}, {2 * K8, K8, 0}, 0,
       2.0 * 2 * K8 * K8 * 2, false, true, 64 * 32, 256},
      {"transpose_bf16_16384x16384", "imex_transpose2d_b16", {2 * K8, 2 * K8},
       {{Elem::BF16, {2 * K8, 2 * K8}, 1, -1, 1}, {Elem::BF16, {2 * K8, 2 * K8}, false, 0, 0}}, {2 * K8, 2 * K8}, 0,
       2.0 * 4 * K8 * K8 * 2, false},
      {"mfma_lds_ceiling_f16_every_exponent", "imex_mfma_lds_ceiling_f16", {256 * 512},
       {{Elem::F32, {256 * 512}, false, 0, 0}}, {256 * 512, 2048, 2}, 0, 256.0 * 8 * 2048 * 32 * 16384, true, true},
      // the same loop with the operands held in registers (no LDS reads inside it)
      {"mfma_reg_ceiling_f16_uniform", "imex_mfma_lds_ceiling_f16", {256 * 512},
       {{Elem::F32, {256 * 512}, false, 0, 0}}, {256 * 512, 2048, 4}, 0, 256.0 * 8 * 2048 * 32 * 16384, true, true},
      {"mfma_reg_ceiling_f16_zeros", "imex_mfma_lds_ceiling_f16", {256 * 512},
       {{Elem::F32, {256 * 512}, false, 0, 0}}, {256 * 512, 2048, 5}, 0, 256.0 * 8 * 2048 * 32 * 16384, true, true},
      {"mfma_reg_ceiling_f16_every_exponent", "imex_mfma_lds_ceiling_f16", {256 * 512},
       {{Elem::F32, {256 * 512}, false, 0, 0}}, {256 * 512, 2048, 6}, 0, 256.0 * 8 * 2048 * 32 * 16384, true, true},
  };
}

int64_t count(const Tensor &t) {
  int64_t n = 1;
  for (int64_t d : t.shape)
    n *= d;
  return n;
}

// Host fill through the runner utilities, on a rank-1 view of the buffer.
void fillHost(void *host, const Tensor &t) {
  struct Desc1D {
    void *allocated, *aligned;
    int64_t offset, size, stride;
  } d = {host, host, 0, count(t), 1};
  ImexUnrankedMemRef m = {1, &d};
  switch (t.elem) {
  case Elem::F32: _mlir_ciface_fillResource1DRandomF32(&m, t.lo, t.hi, false); break;
  case Elem::F16: _mlir_ciface_fillResource1DRandomF16(&m, t.lo, t.hi, false); break;
  case Elem::BF16: _mlir_ciface_fillResource1DRandomBF16(&m, t.lo, t.hi, false); break;
  }
}

// Directory of this executable (the code objects that are not in the catalogue sit beside it).
std::string programDir() {
  char buf[4096];
  const ssize_t n = readlink("/proc/self/exe", buf, sizeof buf - 1);
  if (n <= 0)
    return ".";
  buf[n] = 0;
  std::string p(buf);
  const size_t slash = p.rfind('/');
  return slash == std::string::npos ? "." : p.substr(0, slash);
}

struct Options {
  int runs = 100, warmups = 10, launchOnly = 0, rotate = 1, grid = 0;
  bool flush = false, zeros = false;
};

// The measurement kernels' code object, read once and kept for the life of the process (the runtime caches
// modules by address); empty if the file is not beside this program.
const std::vector<char> &probeImage() {
  static std::vector<char> image;
  if (image.empty()) {
    const std::string path = programDir() + "/imex_probe.hsaco";
    if (FILE *f = fopen(path.c_str(), "rb")) {
      char buf[65536];
      for (size_t n; (n = fread(buf, 1, sizeof buf, f)) > 0;)
        image.insert(image.end(), buf, buf + n);
      fclose(f);
    }
  }
  return image;
}

// --lds-service: which lanes of a wavefront the LDS serves together, and over how many bytes its banks repeat,
// for each kind of access.  One dispatch of imex_probe_lds_pair per question, a single wavefront with two active
// lanes that access different addresses a given distance apart, 64 times: the dispatch counts bank-conflict
// cycles (rocprofv3 --pmc SQ_LDS_BANK_CONFLICT) exactly when the two lanes are served in the same pass AND the
// distance is a multiple of the bank period.  Per kind: lane 0 against every other lane, 1024 bytes apart
// (a multiple of every candidate period), then lanes 0 and 1 at 16 .. 1024 bytes.  Prints the question of every
// dispatch in launch order, which is the order of the counter file's Dispatch_Id.
int runLdsServiceProbe() {
  static const char *kinds[6] = {"ds_read_b128", "ds_write_b128", "ds_read_b64", "ds_write_b64", "ds_read_b32", "ds_write_b32"};
  const std::vector<char> &image = probeImage();
  if (image.empty()) {
    fprintf(stderr, "--lds-service: cannot read %s/imex_probe.hsaco\n", programDir().c_str());
    return 1;
  }
  void *stream = gpuCreateStream(nullptr, nullptr);
  void *module = gpuModuleLoad(stream, image.data(), image.size());
  void *kernel = gpuKernelGet(stream, module, "imex_probe_lds_pair");
  void *out = gpuMemAlloc(stream, 256, 64, /*isShared=*/0);
  ImexEventDesc noDeps[1] = {{nullptr}};
  int n = 0;
  auto ask = [&](int64_t kind, int64_t lane, int64_t bytesApart) {
    ImexParamDesc ps[5] = {{&out, sizeof(void *)}, {&kind, 8}, {&lane, 8}, {&bytesApart, 8}, {nullptr, 0}};
    gpuLaunchKernel(stream, kernel, 1, 1, 1, 64, 1, 1, 0, ps, noDeps);
    gpuWait(stream);
    printf("dispatch %d: %s lanes 0 and %d, %d bytes apart\n", ++n, kinds[kind], static_cast<int>(lane),
           static_cast<int>(bytesApart));
  };
  for (int kind = 0; kind < 6; ++kind) {
    for (int lane = 1; lane < 64; ++lane)
      ask(kind, lane, 1024);
    for (int bytes = 16; bytes <= 1024; bytes *= 2)
      ask(kind, 1, bytes);
  }
  gpuMemFree(stream, out);
  gpuStreamDestroy(stream);
  return 0;
}

int runWorkload(const Workload &w, const Options &opt) {
  void *stream = gpuCreateStream(nullptr, nullptr);
  std::vector<void *> dev;
  std::vector<std::vector<char>> host;
  for (const Tensor &t : w.tensors) {
    const size_t bytes = static_cast<size_t>(count(t)) * elemBytes(t.elem);
    dev.push_back(gpuMemAlloc(stream, bytes, 64, /*isShared=*/0));
    if (t.isInput) {
      host.emplace_back(bytes);
      if (!opt.zeros)
        fillHost(host.back().data(), t);
      gpuMemCopy(stream, dev.back(), host.back().data(), bytes);
    }
  }

  size_t grid[3] = {1, 1, 1}, block[3] = {static_cast<size_t>(w.probeBlock), 1, 1}, smem = 0;
  size_t blobSize = 0;
  const void *blob = nullptr;
  if (w.probe) {
    grid[0] = w.probeGrid ? static_cast<size_t>(w.probeGrid)
                          : static_cast<size_t>((w.dims[0] + w.probeBlock - 1) / w.probeBlock);
    const std::vector<char> &probeBlob = probeImage();
    if (probeBlob.empty()) {
      fprintf(stderr, "%s: cannot read %s/imex_probe.hsaco\n", w.name, programDir().c_str());
      return 1;
    }
    blob = probeBlob.data();
    blobSize = probeBlob.size();
  } else {
    if (imexHipKernelLaunchShape(w.kernel, w.dims.data(), static_cast<int>(w.dims.size()), grid, block, &smem) != 0) {
      fprintf(stderr, "%s: no launch shape for %s\n", w.name, w.kernel);
      return 1;
    }
    blob = imexHipKernelModule(w.kernel, &blobSize);
  }
  if (opt.grid > 0) { // every kernel strides over its work, so any grid computes the same thing
    grid[0] = static_cast<size_t>(opt.grid);
    grid[1] = grid[2] = 1;
  }
  void *module = gpuModuleLoad(stream, blob, blobSize);
  void *kernel = gpuKernelGet(stream, module, w.kernel);

  // Further copies of the tensors for --rotate: set s holds its own buffers, inputs copied from set 0.
  std::vector<std::vector<void *>> sets(1, dev);
  for (int s = 1; s < opt.rotate; ++s) {
    std::vector<void *> more;
    for (size_t t = 0; t < w.tensors.size(); ++t) {
      const size_t bytes = static_cast<size_t>(count(w.tensors[t])) * elemBytes(w.tensors[t].elem);
      more.push_back(gpuMemAlloc(stream, bytes, 64, /*isShared=*/0));
      if (w.tensors[t].isInput)
        gpuMemCopy(stream, more.back(), dev[t], bytes);
    }
    sets.push_back(more);
  }

  // ParamDesc list per set: pointers, then i64 scalars, then the optional f32 init; {NULL,0} ends it.
  std::vector<int64_t> idx(w.indexArgs);
  float init = 0.0f, scale = 0.5f;
  std::vector<std::vector<ImexParamDesc>> paramSets;
  for (std::vector<void *> &set : sets) {
    std::vector<ImexParamDesc> ps;
    for (void *&p : set)
      ps.push_back({&p, sizeof(void *)});
    if (w.floatArg == 2)
      ps.push_back({&scale, sizeof(float)});
    for (int64_t &v : idx)
      ps.push_back({&v, sizeof(int64_t)});
    if (w.floatArg == 1)
      ps.push_back({&init, sizeof(float)});
    ps.push_back({nullptr, 0});
    paramSets.push_back(ps);
  }
  std::vector<ImexParamDesc> &params = paramSets[0];
  ImexEventDesc noDeps[1] = {{nullptr}};
  auto launch = [&](int i) {
    gpuLaunchKernel(stream, kernel, grid[0], grid[1], grid[2], block[0], block[1], block[2], smem,
                    paramSets[static_cast<size_t>(i) % paramSets.size()].data(), noDeps);
  };

  if (opt.launchOnly > 0) {
    for (int i = 0; i < opt.launchOnly; ++i)
      launch(i);
    gpuWait(stream);
    printf("%s: launched %s %d times over %d buffer set(s), grid (%zu,%zu,%zu) block (%zu,%zu,%zu)\n", w.name, w.kernel,
           opt.launchOnly, opt.rotate, grid[0], grid[1], grid[2], block[0], block[1], block[2]);
  } else {
    std::vector<float> times(opt.runs);
    imexHipProfileKernel(stream, kernel, grid[0], grid[1], grid[2], block[0], block[1], block[2], smem, params.data(),
                         opt.warmups, opt.runs, opt.flush ? (size_t(512) << 20) : 0, 0, times.data());
    float s[9];
    imexHipComputeStats(times.data(), times.size(), s);
    float total = 0.0f;
    if (opt.rotate > 1) {
      for (int i = 0; i < opt.warmups; ++i)
        launch(i);
      void *t0 = imexHipRecordTimestamp(stream);
      for (int i = 0; i < opt.runs; ++i)
        launch(opt.warmups + i);
      void *t1 = imexHipRecordTimestamp(stream);
      gpuWait(stream);
      total = imexHipEventElapsedMs(t0, t1);
    } else {
      imexHipProfileKernel(stream, kernel, grid[0], grid[1], grid[2], block[0], block[1], block[2], smem, params.data(),
                           opt.warmups, opt.runs, 0, 1, &total);
    }
    const double backToBackMs = total / opt.runs;
    printf("%s: the kernel execution time is (ms, on HIP runtime):avg: %.4f, min: %.4f, max: %.4f, median: %4f, "
           "std_deviation: %4f, variance: %4f, P95: %4f, P5: %4f, median_one_third_avg: %4f (over %d runs)\n",
           w.name, s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7], s[8], opt.runs);
    const double rate = w.work / (backToBackMs * (w.mfma ? 1e9 : 1e6));
    printf("%s: back-to-back %.4f ms/launch = %.1f %s (%.1f%% of the %s roofline)%s%s\n", w.name, backToBackMs, rate,
           w.mfma ? "TFLOP/s" : "GB/s", 100.0 * rate / (w.mfma ? 2500.0 : 8000.0), w.mfma ? "2.5 PFLOP/s MFMA" : "8 TB/s HBM",
           opt.flush ? " [per-launch times above measured after a cache flush]" : (opt.zeros ? " [all-zero inputs]" : ""),
           opt.rotate > 1 ? (" [rotating over " + std::to_string(opt.rotate) + " buffer sets]").c_str() : "");
  }
  fflush(stdout);

  for (std::vector<void *> &set : sets)
    for (void *p : set)
      gpuMemFree(stream, p);
  gpuStreamDestroy(stream);
  return 0;
}

} // namespace

// One child process per workload, as bench_imex runs one mlir-runner per .mlir file.
int runReport(const char *self, const std::string &reportPath, const std::string &options,
              const std::vector<std::string> &names) {
  FILE *report = fopen(reportPath.c_str(), "w");
  if (!report) {
    fprintf(stderr, "cannot write %s\n", reportPath.c_str());
    return 1;
  }
  const time_t now = time(nullptr);
  char date[64];
  strftime(date, sizeof date, "%a %b %e %H:%M:%S %Z %Y", localtime(&now));
  fprintf(report, "\n================ Imex Perf (HIP) @ %s ================\n\n", date);
  int rc = 0;
  for (const std::string &n : names) {
    fprintf(stderr, "%s: ", n.c_str());
    const std::string cmd = std::string("\"") + self + "\"" + options + " " + n;
    FILE *child = popen(cmd.c_str(), "r");
    if (!child) {
      fprintf(stderr, "cannot start %s\n", cmd.c_str());
      rc = 1;
      continue;
    }
    char line[2048];
    while (fgets(line, sizeof line, child)) {
      fputs(line, stdout);
      if (strstr(line, "execution time"))
        fputs(line, report); // the driver's lines already start with "<workload>: "
    }
    const int status = pclose(child);
    if (status != 0)
      rc = 1; // like bench_imex, keep going; the exit code reports that something failed
  }
  fclose(report);
  return rc;
}

int main(int argc, char **argv) {
  Options opt;
  std::vector<std::string> names;
  std::string reportPath, childOptions;
  const std::vector<Workload> all = workloads();
  for (int i = 1; i < argc; ++i) {
    const std::string a = argv[i];
    if (a == "--list") {
      for (const Workload &w : all)
        printf("%s  (%s)\n", w.name, w.kernel);
      return 0;
    } else if (a == "--lds-service") {
      return runLdsServiceProbe();
    } else if (a == "-l" || a == "-s") {
      // backend selectors of bench_imex (Level Zero / SYCL); HIP is the only runtime here
    } else if (a == "-c") {
      fprintf(stderr, "-c (CPU lowering) is not part of this library: it stays IMEX's linalg-to-cpu pipeline\n");
      return 1;
    } else if (a == "--report" && i + 1 < argc) {
      reportPath = argv[++i];
    } else if (a == "--flush") {
      opt.flush = true;
      childOptions += " --flush";
    } else if (a == "--zeros") {
      opt.zeros = true;
      childOptions += " --zeros";
    } else if (a == "--runs" && i + 1 < argc) {
      opt.runs = atoi(argv[++i]);
      childOptions += " --runs " + std::to_string(opt.runs);
    } else if (a == "--warmups" && i + 1 < argc) {
      opt.warmups = atoi(argv[++i]);
      childOptions += " --warmups " + std::to_string(opt.warmups);
    } else if (a == "--launch-only" && i + 1 < argc) {
      opt.launchOnly = atoi(argv[++i]);
    } else if (a == "--grid" && i + 1 < argc) {
      opt.grid = atoi(argv[++i]);
      childOptions += " --grid " + std::to_string(opt.grid);
    } else if (a == "--rotate" && i + 1 < argc) {
      opt.rotate = atoi(argv[++i]);
      childOptions += " --rotate " + std::to_string(opt.rotate);
    } else if (a == "all" || a == "operators") { // operators: everything but the measurement kernels
      for (const Workload &w : all)
        if (a == "all" || !w.probe)
          names.push_back(w.name);
    } else {
      names.push_back(a);
    }
  }
  if (names.empty() || opt.runs < 1 || opt.rotate < 1 || opt.rotate > 64) {
    fprintf(stderr, "usage: imex-hip-bench [-l] [--runs N] [--warmups W] [--flush] [--zeros] [--rotate S] [--grid G] [--launch-only N] [--report FILE] <workload>|all ...\n"
                    "       imex-hip-bench --list\n       imex-hip-bench --lds-service\n");
    return 2;
  }
  for (const std::string &n : names) {
    bool known = false;
    for (const Workload &w : all)
      known = known || n == w.name;
    if (!known) {
      fprintf(stderr, "unknown workload %s (try --list)\n", n.c_str());
      return 2;
    }
  }
  if (!reportPath.empty())
    return runReport(argv[0], reportPath, childOptions, names);
  printf("\n================ Imex Perf (HIP runtime) ================\n\n");
  for (const std::string &n : names) {
    const Workload *found = nullptr;
    for (const Workload &w : all)
      if (n == w.name)
        found = &w;
    if (!found) {
      fprintf(stderr, "unknown workload %s (try --list)\n", n.c_str());
      return 2;
    }
    if (int rc = runWorkload(*found, opt))
      return rc;
  }
  return 0;
}
