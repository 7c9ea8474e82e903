"""ctypes mirror of the C ABI: the runtime wrappers (imex_hip_runtime.h), the
kernel catalogue (imex_hip_kernels.h) and, on top of them, one host function per
benchmark workload that does what IMEX's JIT'd ``main`` does for it: create a
stream, gpuMemAlloc, gpuMemCopy in, gpuModuleLoad + gpuKernelGet +
gpuLaunchKernel with a ParamDesc list, gpuWait, gpuMemCopy out
(lib/Conversion/GPUXToLLVM/GPUXToLLVMPass.cpp:373-383,508-518,691-710).

Nothing here computes on the CPU: if the built libraries are missing the import
of the runtime raises, and every operator goes through the HIP kernels.
"""
from __future__ import annotations

import ctypes as C
import os
import re

import numpy as np

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(PKG_DIR, "lib")


class ParamDesc(C.Structure):
    """LevelZeroRuntimeWrappers.cpp:80-89."""
    _fields_ = [("data", C.c_void_p), ("size", C.c_size_t)]


class EventDesc(C.Structure):
    """LevelZeroRuntimeWrappers.cpp:91-97."""
    _fields_ = [("event", C.c_void_p)]


class Ptr(int):
    """A device (or shared) address passed to a kernel as a memref base pointer."""


def _load(name):
    path = os.path.join(LIB_DIR, name)
    if not os.path.exists(path):
        raise ImportError(
            "%s is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or mlir-extensions_amd/build.py) first" % path)
    return C.CDLL(path, mode=C.RTLD_GLOBAL)


_RUNTIME_SYMBOLS = {
    "gpuCreateStream": (C.c_void_p, [C.c_void_p, C.c_void_p]),
    "gpuStreamDestroy": (None, [C.c_void_p]),
    "gpuMemAlloc": (C.c_void_p, [C.c_void_p, C.c_size_t, C.c_size_t, C.c_int]),
    "gpuMemFree": (None, [C.c_void_p, C.c_void_p]),
    "gpuMemCopy": (None, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
    "gpuModuleLoad": (C.c_void_p, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "gpuKernelGet": (C.c_void_p, [C.c_void_p, C.c_void_p, C.c_char_p]),
    "gpuLaunchKernel": (C.c_void_p, [C.c_void_p, C.c_void_p] + [C.c_size_t] * 7 + [C.c_void_p, C.c_void_p]),
    "gpuWait": (None, [C.c_void_p]),
    "gpuModuleUnload": (None, [C.c_void_p, C.c_void_p]),
    "mgpuStreamCreate": (C.c_void_p, []),
    "mgpuStreamSynchronize": (None, [C.c_void_p]),
    "mgpuStreamDestroy": (None, [C.c_void_p]),
    "mgpuLaunchKernel": (None, [C.c_void_p] + [C.c_size_t] * 7 + [C.c_void_p, C.POINTER(C.c_void_p),
                                                                 C.POINTER(C.c_void_p), C.c_size_t]),
    "mgpuMemAlloc": (C.c_void_p, [C.c_size_t, C.c_void_p, C.c_int]),
    "mgpuMemFree": (None, [C.c_void_p, C.c_void_p]),
    "mgpuMemcpy": (None, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "mgpuMemset32": (None, [C.c_void_p, C.c_uint, C.c_size_t, C.c_void_p]),
    "mgpuMemset16": (None, [C.c_void_p, C.c_ushort, C.c_size_t, C.c_void_p]),
    "gpuMemSet32": (None, [C.c_void_p, C.c_void_p, C.c_uint, C.c_size_t]),
    "gpuMemSet16": (None, [C.c_void_p, C.c_void_p, C.c_ushort, C.c_size_t]),
    "mgpuModuleLoad": (C.c_void_p, [C.c_void_p, C.c_size_t]),
    "mgpuModuleGetFunction": (C.c_void_p, [C.c_void_p, C.c_char_p]),
    "mgpuModuleUnload": (None, [C.c_void_p]),
    "imexHipProfileKernel": (C.c_int, [C.c_void_p, C.c_void_p] + [C.c_size_t] * 7 +
                             [C.c_void_p, C.c_int, C.c_int, C.c_size_t, C.c_int, C.POINTER(C.c_float)]),
    "imexHipRecordTimestamp": (C.c_void_p, [C.c_void_p]),
    "imexHipEventElapsedMs": (C.c_float, [C.c_void_p, C.c_void_p]),
    "imexHipComputeStats": (None, [C.POINTER(C.c_float), C.c_size_t, C.POINTER(C.c_float)]),
    "imexHipDeviceInfo": (C.c_int, [C.c_void_p, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_size_t),
                                    C.POINTER(C.c_size_t), C.c_char_p, C.c_size_t]),
    "imexHipQueueDevice": (C.c_int, [C.c_void_p]),
}

_OPS_SYMBOLS = {
    "imexHipOpsInit": (C.c_int, [C.c_void_p]),
    "imexHipGemmBiasSiluBf16SplitK": (C.c_int, [C.c_void_p] * 5 + [C.c_int64] * 3),
    "imexHipGemmBiasSiluBf16SplitKNoAlloc": (C.c_int, [C.c_void_p] * 5 + [C.c_int64] * 3),
    "imexHipOpsFixedWorkspaceBytes": (C.c_size_t, []),
    "imexHipOpsLastError": (C.c_char_p, []),
}

_KERNEL_SYMBOLS = {
    "imexHipKernelCount": (C.c_int, []),
    "imexHipKernelName": (C.c_char_p, [C.c_int]),
    "imexHipKernelSignature": (C.c_char_p, [C.c_int]),
    "imexHipKernelModule": (C.c_void_p, [C.c_char_p, C.POINTER(C.c_size_t)]),
    "imexHipKernelLaunchShape": (C.c_int, [C.c_char_p, C.POINTER(C.c_int64), C.c_int, C.POINTER(C.c_size_t),
                                           C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "imexHipStreamKWorkspaceBytes": (C.c_size_t, [C.c_size_t]),
}

_RUNNER_UTILS_SYMBOLS = [
    "_mlir_ciface_fillResource1DBF16", "_mlir_ciface_fillResource1DF16", "_mlir_ciface_fillResource1DF32",
    "_mlir_ciface_fillResource1DRandomBF16", "_mlir_ciface_fillResource1DRandomF16",
    "_mlir_ciface_fillResource1DRandomF32", "_mlir_ciface_printMemrefBF16", "_mlir_ciface_printMemrefF16",
    "printMemrefBF16", "printMemrefF16", "_mlir_ciface_allcloseBF16", "_mlir_ciface_allcloseF16",
    "_mlir_ciface_allcloseF32", "_mlir_ciface_printAllcloseBF16", "_mlir_ciface_printAllcloseF16",
    "_mlir_ciface_printAllcloseF32", "_mlir_ciface_printMaxErrorF16", "_mlir_ciface_printMaxErrorBF16",
    "_mlir_ciface_printMaxErrorF32", "_mlir_ciface_gemmF16F16F16", "_mlir_ciface_gemmF16F16F32",
    "_mlir_ciface_gemmBF16BF16F32",
]


def _bind(lib, table):
    for name, (res, args) in table.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args


_FILE_BLOBS = {}
PROBE_CODE_OBJECT = os.path.join(LIB_DIR, "imex_probe.hsaco")

_runtime = None
_kernels = None
_runner_utils = None


def runtime():
    global _runtime
    if _runtime is None:
        lib = _load("libimex-hip-runtime.so")
        _bind(lib, _RUNTIME_SYMBOLS)
        _runtime = lib
    return _runtime


def kernels():
    global _kernels
    if _kernels is None:
        lib = _load("libimex-hip-kernels.so")
        _bind(lib, _KERNEL_SYMBOLS)
        _kernels = lib
    return _kernels


_ops = None


def ops():
    """libimex-hip-ops.so: the one-call operator entries (include/imex_hip_ops.h)."""
    global _ops
    if _ops is None:
        runtime()
        kernels()
        lib = _load("libimex-hip-ops.so")
        _bind(lib, _OPS_SYMBOLS)
        _ops = lib
    return _ops


def runner_utils():
    global _runner_utils
    if _runner_utils is None:
        lib = _load("libimex_runner_utils.so")
        for name in _RUNNER_UTILS_SYMBOLS:
            getattr(lib, name)
        for name in ("_mlir_ciface_allcloseBF16", "_mlir_ciface_allcloseF16", "_mlir_ciface_allcloseF32"):
            getattr(lib, name).restype = C.c_bool
        _runner_utils = lib
    return _runner_utils


def kernel_names():
    k = kernels()
    return [k.imexHipKernelName(i).decode() for i in range(k.imexHipKernelCount())]


def launch_shape(kernel, dims):
    """(grid, block, shared_mem_bytes) for `kernel` at `dims`."""
    k = kernels()
    d = (C.c_int64 * max(len(dims), 1))(*dims)
    grid = (C.c_size_t * 3)()
    block = (C.c_size_t * 3)()
    smem = C.c_size_t(0)
    rc = k.imexHipKernelLaunchShape(kernel.encode(), d, len(dims), grid, block, C.byref(smem))
    if rc != 0:
        raise ValueError("imexHipKernelLaunchShape(%s, %s) -> %d" % (kernel, list(dims), rc))
    return tuple(grid), tuple(block), smem.value


_SIGNATURE_TYPES = {}


def signature_types(kernel):
    """Argument types of a catalogue kernel, from its signature string
    "(in: f32*, out: f32*, rows: i64, init: f32)" -> ["ptr", "ptr", "i64", "f32"]; None if unknown."""
    if kernel not in _SIGNATURE_TYPES:
        _SIGNATURE_TYPES[kernel] = _parse_signature(kernel)
    return _SIGNATURE_TYPES[kernel]


def _parse_signature(kernel):
    k = kernels()
    for i in range(k.imexHipKernelCount()):
        if k.imexHipKernelName(i).decode() == kernel:
            sig = re.sub(r"\[[^\]]*\]", "", k.imexHipKernelSignature(i).decode().strip()[1:-1])  # drop layout notes "[K,M]"
            types = []
            for part in sig.split(","):
                t = part.split(":", 1)[1].strip()
                types.append("ptr" if "*" in t else t.split()[0])
            return types
    return None


def _pack_params(args, types=None):
    """ParamDesc[n+1] terminated by {NULL, 0}; keeps the value storage alive.  With `types` (see
    signature_types) every scalar is packed as the kernel declares it -- a Python int given for an
    f32 parameter becomes a 4-byte float; without, pointers are 8 bytes, ints i64 and floats f32."""
    if types is not None and len(types) != len(args):
        raise TypeError("kernel takes %d arguments, %d given" % (len(types), len(args)))
    storage = []
    descs = (ParamDesc * (len(args) + 1))()
    for i, a in enumerate(args):
        want = types[i] if types is not None else None
        if want == "ptr" or (want is None and isinstance(a, Ptr)):
            if not isinstance(a, Ptr):
                raise TypeError("argument %d is a memref base pointer, got %r" % (i, a))
            v = C.c_void_p(int(a))
        elif want == "f32" or (want is None and isinstance(a, (float, np.floating))):
            v = C.c_float(float(a))
        elif want == "i64" or (want is None and isinstance(a, (int, np.integer))):
            if isinstance(a, (float, np.floating)) and float(a) != int(a):
                raise TypeError("argument %d is an index, got %r" % (i, a))
            v = C.c_int64(int(a))
        else:
            raise TypeError("unsupported kernel argument %r" % (a,))
        storage.append(v)
        descs[i].data = C.cast(C.pointer(v), C.c_void_p)
        descs[i].size = C.sizeof(v)
    descs[len(args)].data = None
    descs[len(args)].size = 0
    return descs, storage


class Stream:
    """gpux stream: the object every gpu* call takes first (GPUToGPUX.cpp:36-59)."""

    def __init__(self, hip_stream=None):
        """`hip_stream`: an existing hipStream_t (integer handle) for the queue to run on instead of
        creating its own; the queue does not destroy it."""
        self.rt = runtime()
        self.handle = self.rt.gpuCreateStream(None, hip_stream)
        self._events = []

    def close(self):
        if self.handle:
            self.rt.gpuStreamDestroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- memory ---------------------------------------------------------------
    def alloc(self, nbytes, shared=False, alignment=64):
        return Ptr(self.rt.gpuMemAlloc(self.handle, nbytes, alignment, 1 if shared else 0))

    def free(self, ptr):
        self.rt.gpuMemFree(self.handle, int(ptr))

    def fill32(self, ptr, value, count):
        """mgpuMemset32 on this queue: `count` 32-bit words of `value`."""
        self.rt.mgpuMemset32(int(ptr), value, count, self.handle)

    def memset(self, ptr, value, count, bits=32):
        """gpuMemSet32 / gpuMemSet16: `count` elements of `bits` width set to `value`, asynchronously."""
        (self.rt.gpuMemSet32 if bits == 32 else self.rt.gpuMemSet16)(self.handle, int(ptr), value, count)

    def copy(self, dst, src, nbytes):
        self.rt.gpuMemCopy(self.handle, int(dst), int(src), nbytes)

    def to_device(self, array):
        a = np.ascontiguousarray(array)
        p = self.alloc(a.nbytes)
        self.copy(p, a.ctypes.data, a.nbytes)
        return p

    def from_device(self, ptr, shape, dtype):
        out = np.empty(shape, dtype=dtype)
        self.copy(out.ctypes.data, ptr, out.nbytes)
        return out

    # -- kernels --------------------------------------------------------------
    def kernel(self, name):
        size = C.c_size_t(0)
        blob = kernels().imexHipKernelModule(name.encode(), C.byref(size))
        if not blob:
            raise KeyError("no kernel named %s in the catalogue" % name)
        module = self.rt.gpuModuleLoad(self.handle, blob, size.value)
        return self.rt.gpuKernelGet(self.handle, module, name.encode())

    def kernel_from_file(self, path, name):
        """A kernel of a code object that is not part of the catalogue (the measurement kernels in
        lib/imex_probe.hsaco): the file's bytes go to gpuModuleLoad like any other blob."""
        blob = _FILE_BLOBS.get(path)
        if blob is None:
            with open(path, "rb") as f:
                data = f.read()
            blob = _FILE_BLOBS[path] = C.create_string_buffer(data, len(data))  # kept: the runtime caches modules by address
        module = self.rt.gpuModuleLoad(self.handle, C.cast(blob, C.c_void_p), len(blob))
        return self.rt.gpuKernelGet(self.handle, module, name.encode())

    def profile_function(self, fn, grid, block, args, warmups, rounds):
        """ms per launch over `rounds` back-to-back launches of an already resolved kernel."""
        descs, keep = _pack_params(args)
        out = (C.c_float * 1)()
        self.rt.imexHipProfileKernel(self.handle, fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], 0,
                                     C.cast(descs, C.c_void_p), warmups, rounds, 0, 1, out)
        del keep
        return out[0] / rounds

    def launch(self, name, dims, args, deps=None, grid=None, block=None):
        """gpuModuleLoad + gpuKernelGet + gpuLaunchKernel; returns the event (or
        None when the launch shape is empty).  `grid` / `block` replace the catalogue's."""
        cat_grid, cat_block, smem = launch_shape(name, dims)
        grid = tuple(grid) if grid is not None else cat_grid
        block = tuple(block) if block is not None else cat_block
        if 0 in grid:
            return None
        fn = self.kernel(name)
        descs, keep = _pack_params(args, signature_types(name))
        evs = (EventDesc * (len(deps or []) + 1))()
        for i, e in enumerate(deps or []):
            evs[i].event = e
        ev = self.rt.gpuLaunchKernel(self.handle, fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                     smem, C.cast(descs, C.c_void_p), C.cast(evs, C.c_void_p))
        del keep
        return ev

    def prepare(self, name, dims, args):
        """Resolve the kernel, its launch shape and its ParamDesc list once and
        return a zero-argument callable that performs just the gpuLaunchKernel
        call (what JIT'd host code does inside a loop)."""
        grid, block, smem = launch_shape(name, dims)
        if 0 in grid:
            return lambda: None
        fn = self.kernel(name)
        descs, keep = _pack_params(args, signature_types(name))
        params = C.cast(descs, C.c_void_p)
        launch, handle = self.rt.gpuLaunchKernel, self.handle
        gx, gy, gz = grid
        bx, by, bz = block

        def run(_keep=(descs, keep)):
            return launch(handle, fn, gx, gy, gz, bx, by, bz, smem, params, None)
        return run

    def profile(self, name, dims, args, warmups=5, rounds=20, flush_bytes=0, mode=0):
        """Per-launch times in ms (mode 0) or [total ms] over `rounds` back-to-back launches (mode 1)."""
        grid, block, smem = launch_shape(name, dims)
        fn = self.kernel(name)
        descs, keep = _pack_params(args, signature_types(name))
        n = rounds if mode == 0 else 1
        out = (C.c_float * n)()
        self.rt.imexHipProfileKernel(self.handle, fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
                                     smem, C.cast(descs, C.c_void_p), warmups, rounds, flush_bytes, mode, out)
        del keep
        return list(out)

    def wait(self):
        self.rt.gpuWait(self.handle)

    def timestamp(self):
        return self.rt.imexHipRecordTimestamp(self.handle)

    def elapsed_ms(self, start_event, stop_event):
        return self.rt.imexHipEventElapsedMs(start_event, stop_event)

    def device_info(self):
        cu, clk = C.c_int(0), C.c_int(0)
        l2, mem = C.c_size_t(0), C.c_size_t(0)
        name = C.create_string_buffer(256)
        rc = self.rt.imexHipDeviceInfo(self.handle, C.byref(cu), C.byref(clk), C.byref(l2), C.byref(mem), name, 256)
        if rc != 0:
            raise RuntimeError("no usable GPU")
        return {"name": name.value.decode(), "cus": cu.value, "clock_khz": clk.value, "l2_bytes": l2.value,
                "global_bytes": mem.value}


def compute_stats(times_ms):
    v = (C.c_float * len(times_ms))(*times_ms)
    out = (C.c_float * 9)()
    runtime().imexHipComputeStats(v, len(times_ms), out)
    keys = ["avg", "min", "max", "median", "stddev", "variance", "p95", "p5", "middle_third_avg"]
    return dict(zip(keys, out))


# -----------------------------------------------------------------------------
# One host function per workload (the benchmarks' `forward`).  16-bit float
# tensors travel as uint16 bit patterns with an explicit dtype name.
# -----------------------------------------------------------------------------

_BYTES = {"f32": 4, "f16": 2, "bf16": 2}
_NP = {"f32": np.float32, "f16": np.uint16, "bf16": np.uint16}


def _check(x, dtype):
    if x.dtype.itemsize != _BYTES[dtype]:
        raise TypeError("array of %s does not hold %s elements" % (x.dtype, dtype))


def _unary(stream, kernel, x, dtype, dims, extra=(), out_shape=None, out_np=None):
    _check(x, dtype)
    out_shape = x.shape if out_shape is None else out_shape
    out_np = x.dtype if out_np is None else out_np
    n_out = int(np.prod(out_shape)) if len(out_shape) else 1
    d_in = stream.to_device(x)
    d_out = stream.alloc(max(n_out, 1) * np.dtype(out_np).itemsize)
    try:
        stream.launch(kernel, dims, [d_in, d_out] + list(dims) + list(extra))
        stream.wait()
        return stream.from_device(d_out, out_shape, out_np)
    finally:
        stream.free(d_in)
        stream.free(d_out)


def relu(stream, x, dtype="f32"):
    """benchmarks/relu/relu_gpu.mlir.in:3-13"""
    return _unary(stream, "imex_relu_" + dtype, x, dtype, [x.size])


def silu(stream, x, dtype="f32"):
    """benchmarks/silu/silu_gpu.mlir.in:3-19 (f16 / bf16: bit patterns in, widened to f32, rounded once)"""
    return _unary(stream, "imex_silu_" + dtype, x, dtype, [x.size])


def _binary(stream, kernel, a, b, dtype, dims, out_shape):
    _check(a, dtype)
    _check(b, dtype)
    if a.shape != b.shape:
        raise ValueError("operand shapes differ: %s vs %s" % (a.shape, b.shape))
    n_out = int(np.prod(out_shape))
    d_a, d_b = stream.to_device(a), stream.to_device(b)
    d_out = stream.alloc(max(n_out, 1) * a.dtype.itemsize)
    try:
        stream.launch(kernel, dims, [d_a, d_b, d_out] + list(dims))
        stream.wait()
        return stream.from_device(d_out, out_shape, a.dtype)
    finally:
        for p in (d_a, d_b, d_out):
            stream.free(p)


def exp(stream, x):
    """test/Integration/Dialect/XeGPU/WG/math_exp.mlir:57 (math.exp on f32: libm's expf)"""
    return _unary(stream, "imex_exp_f32", x, "f32", [x.size])


def maximum(stream, a, b):
    """test/Integration/Dialect/XeGPU/WG/arith_maximumf.mlir:61 (arith.maximumf on f32)"""
    return _binary(stream, "imex_maximum_f32", a, b, "f32", [a.size], a.shape)


def loop_fusion(stream, a, b, dtype="f32"):
    """benchmarks/kLoopFusion/kLoopFusion.mlir.in:4-30: (log a + |b|) - a"""
    return _binary(stream, "imex_loop_fusion_" + dtype, a, b, dtype, [a.size], a.shape)


def input_fusion(stream, a, b, dtype="f32"):
    """benchmarks/kInputFusion/kInputFusion.mlir.in:6-40: out[j] = sum_i (log b[i,j] + |a[i,j]|)"""
    rows, cols = a.shape
    return _binary(stream, "imex_input_fusion_" + dtype, a, b, dtype, [rows, cols], (cols,))


def flash_attention(stream, q, k, v, zh, n_ctx, sm_scale, queries_per_workgroup=None, threads=512):
    """WG/flash_attention_fwd.mlir:25-307: softmax(sm_scale * Q K^T) V per (batch, head);
    q, k, v f16 bit patterns [(zh * n_ctx), 64].  `queries_per_workgroup` (64, 128 or 256)
    picks the tiling instead of the catalogue; 256 queries also come
    with `threads` = 1024 (sixteen wavefronts, two key groups)."""
    for t in (q, k, v):
        _check(t, "f16")
        if t.shape != (zh * n_ctx, 64):
            raise ValueError("expected shape (%d, 64), got %s" % (zh * n_ctx, t.shape))
    d_q, d_k, d_v = stream.to_device(q), stream.to_device(k), stream.to_device(v)
    d_o = stream.alloc(max(q.size, 1) * 2)
    try:
        grid = block = None
        if queries_per_workgroup is not None:
            if queries_per_workgroup not in (64, 128, 256):
                raise ValueError("queries_per_workgroup must be 64, 128 or 256")
            if threads not in (512, 1024) or (threads == 1024 and queries_per_workgroup != 256):
                raise ValueError("threads is 512, or 1024 with 256 queries per workgroup")
            grid, block = (-(-n_ctx // queries_per_workgroup), zh, 1), (threads, 1, 1)
        stream.launch("imex_flash_attention_fwd_f16", [zh, n_ctx], [d_q, d_k, d_v, d_o, float(sm_scale), zh, n_ctx],
                      grid=grid, block=block)
        stream.wait()
        return stream.from_device(d_o, q.shape, np.uint16)
    finally:
        for p in (d_q, d_k, d_v, d_o):
            stream.free(p)


def mfma_lds_ceiling(stream, workgroups, iters, mode=0):
    """The measurement kernel imex_mfma_lds_ceiling_f16 (no counterpart in the reference; it lives in
    lib/imex_probe.hsaco, outside the catalogue): returns the one f32 per lane it stores, shape
    (workgroups, 512).  mode 0: operands uniform in (-1, 1) like the GEMM benchmark's; 1: zeros;
    2: every f16 exponent below 1.0 equally likely."""
    n = workgroups * 512
    if workgroups < 1:
        raise ValueError("at least one workgroup")
    d_o = stream.alloc(n * 4)
    try:
        fn = stream.kernel_from_file(PROBE_CODE_OBJECT, "imex_mfma_lds_ceiling_f16")
        descs, keep = _pack_params([d_o, n, int(iters), int(mode)])
        stream.rt.gpuLaunchKernel(stream.handle, fn, workgroups, 1, 1, 512, 1, 1, 0, C.cast(descs, C.c_void_p), None)
        stream.wait()
        return stream.from_device(d_o, (workgroups, 512), np.float32)
    finally:
        stream.free(d_o)


def softmax(stream, x, dtype="f32"):
    """benchmarks/softmax/softmax_gpu.mlir.in:4-44 (last dim of a 2-D tensor)"""
    rows, cols = x.shape
    return _unary(stream, "imex_softmax_" + dtype, x, dtype, [rows, cols])


def rowsum(stream, x, init=0.0):
    """WG/reduction_2D_1D_cross_sg_cross_lane.mlir:31-37"""
    rows, cols = x.shape
    return _unary(stream, "imex_rowsum_f32", x, "f32", [rows, cols], extra=[float(init)], out_shape=(rows,))


def rowmean(stream, x):
    """WG/reduction_4D_3D_mean_intra_sg_intra_lane.mlir:51-52: mean over the last dimension."""
    rows, cols = x.shape
    return _unary(stream, "imex_rowmean_f32", x, "f32", [rows, cols], out_shape=(rows,))


def reduce_outer(stream, x, init=0.0, dtype="f32"):
    """benchmarks/reduce/reduce_gpu.mlir.in:4-21: the outermost dim is summed away (f16 / bf16: bit
    patterns in and out, f32 accumulation)."""
    outer = x.shape[0]
    inner = int(np.prod(x.shape[1:]))
    return _unary(stream, "imex_reduce_outer_" + dtype, x, dtype, [outer, inner], extra=[float(init)],
                  out_shape=x.shape[1:])


def transpose2d(stream, x):
    """benchmarks/transpose/transpose2d_gpu.mlir.in:4-11"""
    rows, cols = x.shape
    bits = x.dtype.itemsize * 8
    return _unary(stream, "imex_transpose2d_b%d" % bits, x, "f32" if bits == 32 else "f16", [rows, cols],
                  out_shape=(cols, rows))


def transpose3d(stream, x):
    """benchmarks/transpose/transpose3d_gpu.mlir.in:4-11 (d0,d1,d2) -> (d2,d1,d0)"""
    d0, d1, d2 = x.shape
    bits = x.dtype.itemsize * 8
    return _unary(stream, "imex_transpose3d_b%d" % bits, x, "f32" if bits == 32 else "f16", [d0, d1, d2],
                  out_shape=(d2, d1, d0))


def gemm(stream, a, b, c=None, ab_dtype="f16", out_dtype="f32", trans_a=False, trans_b=False):
    """C = A.B (or C += A.B when `c` is given), WG/gemm_4kx4kx4k_f16_f16_f32.mlir:21-91.
    trans_a: `a` is stored [K,M] (WG/gemm_4kx4kx4k_transpose_a.mlir); trans_b: `b` is
    stored [N,K] (WG/gemm_4kx4kx4k_transpose_b.mlir)."""
    _check(a, ab_dtype)
    _check(b, ab_dtype)
    K, M = a.shape if trans_a else a.shape[::-1]
    K2, N = b.shape[::-1] if trans_b else b.shape
    if K != K2:
        raise ValueError("inner dimensions differ: %d vs %d" % (K, K2))
    if trans_a or trans_b:
        if (trans_a and trans_b) or c is not None or ab_dtype != "f16" or out_dtype != "f32":
            raise ValueError("the transposed-operand kernels are f16 -> f32, one operand transposed, no accumulate")
        name = "imex_gemm_f16_f16_f32_ta" if trans_a else "imex_gemm_f16_f16_f32_tb"
        out_np = np.float32
    elif out_dtype == "f16":
        name = "imex_gemm_f16_f16_f16"
        out_np = np.uint16
    else:
        name = "imex_gemm_%s_%s_f32" % (ab_dtype, ab_dtype) + ("_acc" if c is not None else "")
        out_np = np.float32
    d_a, d_b = stream.to_device(a), stream.to_device(b)
    d_c = stream.to_device(c.astype(np.float32)) if c is not None else stream.alloc(max(M * N, 1) * np.dtype(out_np).itemsize)
    try:
        stream.launch(name, [M, N, K], [d_a, d_b, d_c, M, N, K])
        stream.wait()
        return stream.from_device(d_c, (M, N), out_np)
    finally:
        for p in (d_a, d_b, d_c):
            stream.free(p)


_streamk_epoch = [0]


def gemm_bias_silu(stream, a, b, bias, streamk=False, grid=None, spin_limit=0):
    """out = bf16(silu(A.B + bias[n])) with bf16 A, B and f32 bias.  streamk: the kernel that splits the
    last, partial round of tiles along K over all workgroups (a workspace is allocated for the call)."""
    _check(a, "bf16")
    _check(b, "bf16")
    M, K = a.shape
    _, N = b.shape
    d_a, d_b, d_bias = stream.to_device(a), stream.to_device(b), stream.to_device(bias.astype(np.float32))
    d_o = stream.alloc(max(M * N, 1) * 2)
    d_ws = None
    try:
        if streamk:
            name = "imex_gemm_bf16_bias_silu_bf16_streamk"
            g = grid if grid is not None else launch_shape(name, [M, N, K])[0]
            d_ws = stream.alloc(kernels().imexHipStreamKWorkspaceBytes(g[0] * g[1] * g[2]))
            _streamk_epoch[0] += 1
            stream.launch(name, [M, N, K], [d_a, d_b, d_bias, d_o, M, N, K, d_ws, _streamk_epoch[0], spin_limit], grid=grid)
        else:
            stream.launch("imex_gemm_bf16_bias_silu_bf16", [M, N, K], [d_a, d_b, d_bias, d_o, M, N, K], grid=grid)
        stream.wait()
        return stream.from_device(d_o, (M, N), np.uint16)
    finally:
        for p in (d_a, d_b, d_bias, d_o, d_ws):
            if p is not None:
                stream.free(p)
