"""Build recipes for the gfx950 code objects and the host libraries.

Everything is compiled in-tree with explicit ``hipcc`` / ``gcc`` command lines
(no CMake needed, hipcc cross-compiles gfx950 without a GPU present):

  lib/imex_<group>.hsaco        one code object per kernel source file
  lib/imex_probe.hsaco          measurement kernels (bench.py and the driver load the file; not in the catalogue)
  lib/libimex-hip-kernels.so    catalogue + the code objects embedded as blobs
  lib/libimex-hip-runtime.so    the gpu* / mgpu* runtime-wrapper ABI on HIP
  lib/libimex-hip-ops.so        one-call entries of the K-splitting GEMM (allocating / not allocating)
  lib/libimex_runner_utils.so   _mlir_ciface_* host helpers

Run as a script (``python build.py``) or call :func:`build_all`.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
BUILD_DIR = os.path.join(REPO_DIR, "build")
INCLUDE_DIR = os.path.join(REPO_DIR, "include")

ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

KERNEL_GROUPS = ["eltwise", "softmax", "reduce", "transpose", "gemm", "fusion", "attention"]
# Measurement kernels: a code object of their own (lib/imex_probe.hsaco) that bench.py and the
# driver load from the file; the catalogue library holds operators only.
BENCH_ONLY_GROUPS = ["probe"]

# -ffp-contract=off: the SiLU, scalar-GEMM and reduction kernels rely on
# separately rounded multiplies and adds.  Packed-FP32 instruction selection is
# switched off for all device code.
DEVICE_FLAGS = [
    "-O3", "-std=c++17", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "--offload-arch=gfx950", "--genco",
    # kernel arguments arrive in SGPRs with the wavefront instead of being fetched by its first instructions
    # (gfx950 kernarg preload; the code object keeps the fetching prologue for firmware without it): a wavefront's
    # first global load issues a few hundred cycles earlier, 1-2 % on the 12-25 us streaming kernels
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-I" + os.path.join(CSRC, "kernels"),
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-ffp-contract=off", "-Wall", "-I" + INCLUDE_DIR]


def _run(cmd, verbose):
    if verbose:
        print("+", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError("build step failed (%d): %s\n%s" % (res.returncode, " ".join(cmd), out))
    if verbose and out:
        print(out, flush=True)


def build_kernels(verbose=False, groups=None):
    os.makedirs(LIB_DIR, exist_ok=True)
    for g in groups or KERNEL_GROUPS + BENCH_ONLY_GROUPS:
        src = os.path.join(CSRC, "kernels", g + ".hip")
        out = os.path.join(LIB_DIR, "imex_%s.hsaco" % g)
        _run([HIPCC] + DEVICE_FLAGS + [src, "-o", out], verbose)


def build_kernel_library(verbose=False):
    """Catalogue library with the code objects embedded through .incbin."""
    os.makedirs(BUILD_DIR, exist_ok=True)
    stub = os.path.join(BUILD_DIR, "imex_blobs.S")
    with open(stub, "w") as f:
        f.write('  .section .rodata\n')
        for g in KERNEL_GROUPS:
            path = os.path.join(LIB_DIR, "imex_%s.hsaco" % g)
            f.write('  .balign 4096\n  .global imex_blob_%s\nimex_blob_%s:\n  .incbin "%s"\n' % (g, g, path))
            f.write('  .global imex_blob_%s_end\nimex_blob_%s_end:\n' % (g, g))
        f.write('  .section .note.GNU-stack,"",@progbits\n')
    out = os.path.join(LIB_DIR, "libimex-hip-kernels.so")
    _run(["g++"] + HOST_FLAGS + ["-shared", "-o", out,
                                 os.path.join(CSRC, "runtime", "KernelCatalog.cpp"), stub], verbose)


def build_runtime(verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(BUILD_DIR, exist_ok=True)
    # the library's own device code (the fill kernel behind mgpuMemset32), embedded like the kernel blobs
    fill = os.path.join(LIB_DIR, "imex_runtime_fill.hsaco")
    _run([HIPCC] + DEVICE_FLAGS + [os.path.join(CSRC, "runtime", "fill.hip"), "-o", fill], verbose)
    stub = os.path.join(BUILD_DIR, "imex_runtime_blobs.S")
    with open(stub, "w") as f:
        f.write('  .section .rodata\n  .balign 4096\n  .global imex_runtime_fill_blob\nimex_runtime_fill_blob:\n')
        f.write('  .incbin "%s"\n  .global imex_runtime_fill_blob_end\nimex_runtime_fill_blob_end:\n' % fill)
        f.write('  .section .note.GNU-stack,"",@progbits\n')
    out = os.path.join(LIB_DIR, "libimex-hip-runtime.so")
    srcs = [os.path.join(CSRC, "runtime", "HipRuntimeWrappers.cpp"),
            os.path.join(CSRC, "runtime", "ProfilerStats.cpp"), stub]
    _run(["g++"] + HOST_FLAGS + ["-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROCM, "include"),
                                 "-shared", "-o", out] + srcs +
         ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(ROCM, "lib")], verbose)


def build_ops(verbose=False):
    """One-call operator entries: host code over the runtime ABI plus one device array, so hipcc builds it
    (the array lives in this library's own device image)."""
    out = os.path.join(LIB_DIR, "libimex-hip-ops.so")
    _run([HIPCC, "-O2", "-std=c++17", "-fPIC", "-shared", "--offload-arch=gfx950",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-I" + INCLUDE_DIR,
          os.path.join(CSRC, "ops", "GemmSplitK.hip"), "-o", out,
          "-L" + LIB_DIR, "-limex-hip-runtime", "-limex-hip-kernels", "-Wl,-rpath,$ORIGIN"], verbose)


def build_runner_utils(verbose=False):
    out = os.path.join(LIB_DIR, "libimex_runner_utils.so")
    _run(["g++"] + HOST_FLAGS + ["-shared", "-o", out,
                                 os.path.join(CSRC, "runner_utils", "RunnerUtils.cpp")], verbose)


def build_driver(verbose=False):
    src = os.path.join(CSRC, "driver", "imex_hip_bench.cpp")
    if not os.path.exists(src):
        return
    out = os.path.join(LIB_DIR, "imex-hip-bench")
    _run(["g++"] + HOST_FLAGS + ["-o", out, src, "-L" + LIB_DIR, "-limex-hip-runtime", "-limex-hip-kernels",
                                 "-limex_runner_utils", "-Wl,-rpath,$ORIGIN", "-ldl"], verbose)


def build_oracle(verbose=False):
    """Test infrastructure: the CPU oracle and, when the reference checkout is
    present, the reference translation unit it is validated against."""
    _run(["make", "-C", os.path.join(REPO_DIR, "oracle")], verbose)


def build_all(verbose=False):
    if not os.path.exists(HIPCC):
        raise RuntimeError("hipcc not found at %s" % HIPCC)
    build_kernels(verbose)
    build_kernel_library(verbose)
    build_runtime(verbose)
    build_ops(verbose)
    build_runner_utils(verbose)
    build_driver(verbose)
    build_oracle(verbose)


def clean():
    shutil.rmtree(LIB_DIR, ignore_errors=True)
    shutil.rmtree(BUILD_DIR, ignore_errors=True)


if __name__ == "__main__":
    if len(sys.argv) > 1 and sys.argv[1] == "clean":
        clean()
    else:
        build_all(verbose=True)
