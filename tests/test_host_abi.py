"""CPU-only checks of the host side: the C-ABI libraries load and export every
symbol include/*.h declares, the launch-shape table, the statistics, the runner
utilities and the stdout+abort error convention (no GPU compute calls here)."""
import ctypes as C
import os
import re
import subprocess
import sys

import numpy as np
import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(REPO, "include")


def declared_functions(header):
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", text)
    return sorted({n for n in names if n.startswith(("gpu", "mgpu", "imexHip", "_mlir_ciface_", "printMemref"))})


def test_runtime_exports_every_declared_symbol(host):
    rt = host.runtime()
    names = declared_functions("imex_hip_runtime.h")
    assert {"gpuCreateStream", "gpuStreamDestroy", "gpuMemAlloc", "gpuMemFree", "gpuMemCopy", "gpuModuleLoad",
            "gpuKernelGet", "gpuLaunchKernel", "gpuWait"} <= set(names)
    for n in names:
        assert getattr(rt, n) is not None, n
    assert set(names) == set(host._RUNTIME_SYMBOLS), "python mirror and header disagree"


def test_kernel_library_exports_and_catalogue(host):
    k = host.kernels()
    for n in declared_functions("imex_hip_kernels.h"):
        assert getattr(k, n) is not None, n
    names = host.kernel_names()
    assert len(names) == len(set(names)) >= 20
    header = open(os.path.join(INCLUDE, "imex_hip_kernels.h")).read()
    for n in names:
        size = C.c_size_t(0)
        blob = k.imexHipKernelModule(n.encode(), C.byref(size))
        assert blob and size.value > 1000
        magic = C.string_at(blob, 24)
        assert magic[:4] == b"\x7fELF" or magic.startswith(b"__CLANG_OFFLOAD_BUNDLE__")
        # the kernel's name is in its code object's symbol table
        assert n.encode() in C.string_at(blob, size.value)
        stem = re.sub(r"_(f32|f16|bf16|b16|b32|acc)$", "", n)
        assert stem in header, "kernel %s is not documented in imex_hip_kernels.h" % n
    assert k.imexHipKernelModule(b"no_such_kernel", None) is None


def test_ops_library_exports_every_declared_symbol(host):
    ops = host.ops()
    names = declared_functions("imex_hip_ops.h")
    assert "imexHipGemmBiasSiluBf16SplitKNoAlloc" in names and len(names) == 5
    for n in names:
        assert getattr(ops, n) is not None, n
    assert set(names) == set(host._OPS_SYMBOLS)
    # no compute without a GPU: only what needs none
    assert ops.imexHipOpsFixedWorkspaceBytes() == host.kernels().imexHipStreamKWorkspaceBytes(256)
    assert ops.imexHipOpsLastError() == b""


def test_runner_utils_exports(host):
    ru = host.runner_utils()
    for n in declared_functions("imex_runner_utils.h"):
        assert getattr(ru, n) is not None, n


def test_launch_shapes(host):
    ls = host.launch_shape
    assert ls("imex_relu_f32", [4096 * 4096]) == ((4096, 1, 1), (256, 1, 1), 0)
    assert ls("imex_relu_f32", [1])[0] == (1, 1, 1)
    assert ls("imex_maximum_f32", [256 * 256]) == ((16, 1, 1), (256, 1, 1), 0)
    assert ls("imex_exp_f32", [256 * 256]) == ((64, 1, 1), (256, 1, 1), 0)  # one vector per lane below 4 Mi elements
    assert ls("imex_relu_f32", [0])[0][0] == 0  # nothing to launch
    assert ls("imex_relu_bf16", [8193])[0] == (2, 1, 1)
    assert ls("imex_softmax_f16", [16384, 1024])[0] == (2048, 1, 1)  # a wavefront per slot of the chip; they walk the rows
    assert ls("imex_softmax_f16", [16383, 1024])[0] == (2048, 1, 1)
    assert ls("imex_softmax_f16", [1000, 512])[0] == (250, 1, 1)
    assert ls("imex_softmax_bf16", [16384, 1024])[0] == (2048, 1, 1)  # two rows per wavefront from 16384 rows on
    assert ls("imex_softmax_bf16", [16383, 1024])[0] == (4096, 1, 1)
    assert ls("imex_softmax_f32", [16, 2000])[0] == (16, 1, 1)
    assert ls("imex_rowsum_f32", [8192, 8192])[0] == (8192, 1, 1)
    assert ls("imex_rowsum_f32", [8, 256])[0] == (2, 1, 1)
    assert ls("imex_reduce_outer_f32", [32, 16 * 512 * 512])[0] == (512, 1, 1)     # 8192 outputs per workgroup
    assert ls("imex_reduce_outer_f32", [32, 1 << 20])[0] == (512, 1, 1)            # 2048
    assert ls("imex_reduce_outer_f32", [32, 5000])[0] == (5, 1, 1)                  # 1024
    assert ls("imex_transpose2d_b16", [8192, 8192])[0] == (32, 32, 1)   # 256 x 256 tiles from 2^24 elements
    assert ls("imex_transpose2d_b16", [2048, 2048])[0] == (16, 16, 1)   # 128 x 128 below
    # 128 x 128 tiles from 2^24 elements; whole tiles: 512 workgroups walk them, the next tile's loads in flight
    assert ls("imex_transpose2d_b32", [4096, 4096])[0] == (32, 16, 1)
    assert ls("imex_transpose2d_b32", [4096, 4100])[0] == (33, 32, 1)   # ragged: one workgroup per tile
    assert ls("imex_transpose2d_b32", [128, 131072])[0] == (512, 1, 1)
    assert ls("imex_transpose3d_b32", [256, 64, 1024])[0] == (8, 2, 32)
    assert ls("imex_transpose2d_b32", [2048, 4096])[0] == (64, 32, 1)   # 64 x 64 below
    assert ls("imex_transpose2d_b32", [10, 20])[0] == (1, 1, 1)
    assert ls("imex_transpose3d_b32", [16, 96, 96])[0] == (2, 1, 96)
    assert ls("imex_gemm_f16_f16_f32", [4096, 4096, 4096]) == ((256, 1, 1), (512, 1, 1), 0)
    assert ls("imex_gemm_bf16_bias_silu_bf16", [4096, 11008, 4096])[0] == (16 * 43, 1, 1)
    assert ls("imex_gemm_f16_f16_f32", [3, 3, 3])[0] == (1, 1, 1)
    # the MFMA path takes K in steps of 32 and B rows of whole 16-byte groups (N % 8 == 0); M and N need
    # not divide the 256 x 256 tile.  The catalogue must count tiles exactly when the kernel tiles.
    assert ls("imex_gemm_f16_f16_f32", [256, 256, 32])[0] == (1, 1, 1)
    assert ls("imex_gemm_f16_f16_f32", [512, 256, 96])[0] == (2, 1, 1)
    assert ls("imex_gemm_f16_f16_f32", [255, 256, 64])[0] == (1, 1, 1)
    assert ls("imex_gemm_f16_f16_f32", [257, 520, 64])[0] == (6, 1, 1)
    assert ls("imex_gemm_f16_f16_f32", [256, 256, 48])[0] == (1, 1, 1)     # K % 32 != 0 but K % 8 == 0: still tiled
    assert ls("imex_gemm_f16_f16_f32", [256, 256, 44])[0] == (4, 1, 1)     # K % 8 != 0: 128 x 128 vector-ALU tiles
    assert ls("imex_gemm_f16_f16_f32", [256, 252, 64])[0] == (4, 1, 1)     # N % 8 != 0
    assert ls("imex_gemm_f16_f16_f32_tb", [256, 252, 64])[0] == (1, 1, 1)  # B stored [N,K]: any N
    assert ls("imex_gemm_f16_f16_f32_ta", [252, 256, 64])[0] == (4, 1, 1)    # A stored [K,M]: M % 8 != 0
    assert ls("imex_gemm_f16_f16_f32_ta", [248, 256, 64])[0] == (1, 1, 1)
    # a strided operand of 2 GiB or more cannot be addressed with 32-bit offsets: the vector-ALU tiles
    assert ls("imex_gemm_f16_f16_f32", [256, 32768, 32768])[0] == (2 * 256, 1, 1)
    assert ls("imex_gemm_f16_f16_f32", [256, 32768, 32736])[0] == (128, 1, 1)
    assert ls("imex_gemm_f16_f16_f32_tb", [256, 32768, 32768])[0] == (128, 1, 1)
    assert ls("imex_gemm_4kx4kx4k_f16_f16_f32", []) == ((16, 16, 1), (512, 1, 1), 0)
    assert ls("imex_flash_attention_fwd_f16", [4, 4096]) == ((64, 4, 1), (512, 1, 1), 0)
    assert ls("imex_flash_attention_fwd_f16", [2, 100])[0] == (2, 2, 1)    # N_CTX need not divide the tiles
    assert ls("imex_flash_attention_fwd_f16", [40, 1000])[:2] == ((8, 40, 1), (512, 1, 1))
    assert ls("imex_flash_attention_fwd_f16", [64, 1000])[:2] == ((4, 64, 1), (1024, 1, 1))
    # 64, 128 or 256 queries per workgroup: the most that still leaves 256 workgroups
    assert ls("imex_flash_attention_fwd_f16", [8, 4096])[0] == (32, 8, 1)
    assert ls("imex_flash_attention_fwd_f16", [16, 4096])[:2] == ((16, 16, 1), (1024, 1, 1))  # 256 queries: 16 wavefronts
    assert ls("imex_flash_attention_fwd_f16", [64, 1024])[:2] == ((4, 64, 1), (1024, 1, 1))
    assert ls("imex_flash_attention_fwd_f16", [3, 256])[0] == (4, 3, 1)
    assert ls("imex_input_fusion_f32", [512, 1024])[:2] == ((256, 1, 1), (320, 1, 1))  # 4 columns per workgroup
    assert ls("imex_input_fusion_bf16", [512, 1024])[:2] == ((256, 1, 1), (320, 1, 1))
    assert ls("imex_input_fusion_f32", [512, 4096])[:2] == ((512, 1, 1), (256, 1, 1))
    assert ls("imex_input_fusion_f32", [512, 65536])[0] == (1024, 1, 1)    # 64
    # tall and wide: the streaming form, 576 lanes per 128-byte row segment
    assert ls("imex_input_fusion_f32", [8192, 8192])[:2] == ((256, 1, 1), (576, 1, 1))
    assert ls("imex_input_fusion_bf16", [8192, 8192])[:2] == ((128, 1, 1), (576, 1, 1))
    assert ls("imex_input_fusion_f16", [2048, 8200])[:2] == ((129, 1, 1), (576, 1, 1))
    assert ls("imex_input_fusion_f32", [2047, 8192])[1] == (256, 1, 1)
    assert ls("imex_input_fusion_f16", [8192, 4096])[1] == (256, 1, 1)
    assert ls("imex_gemm_4kx4kx4k_transpose_a", []) == ((16, 16, 1), (512, 1, 1), 0)
    assert ls("imex_gemm_f16_f16_f32_tb", [512, 256, 96])[0] == (2, 1, 1)
    with pytest.raises(ValueError):
        ls("imex_mfma_lds_ceiling_f16", [512])  # measurement kernels are not catalogue entries
    with pytest.raises(ValueError):
        ls("imex_relu_f32", [1, 2])
    with pytest.raises(ValueError):
        ls("imex_relu_f32", [-1])
    with pytest.raises(ValueError):
        ls("nope", [1])


def test_param_desc_packing(host):
    descs, keep = host._pack_params([host.Ptr(0x1000), 7, 2.5])
    assert C.sizeof(host.ParamDesc) == 16
    assert [d.size for d in descs] == [8, 8, 4, 0]
    assert descs[3].data is None
    assert C.cast(descs[0].data, C.POINTER(C.c_void_p))[0] == 0x1000
    assert C.cast(descs[1].data, C.POINTER(C.c_int64))[0] == 7
    assert C.cast(descs[2].data, C.POINTER(C.c_float))[0] == 2.5


def test_profiler_stats_vs_oracle(host, orc):
    rng = np.random.default_rng(3)
    for n in (1, 2, 3, 4, 7, 100, 1000):
        v = (rng.random(n) * 2).astype(np.float32)
        s = host.compute_stats(list(v))
        for mine, theirs in (("avg", "avg"), ("min", "min"), ("max", "max"), ("median", "median_textbook"),
                             ("stddev", "stddev"), ("variance", "variance"), ("p95", "p95"), ("p5", "p5"),
                             ("middle_third_avg", "middle_third_avg")):
            assert s[mine] == orc.stat(theirs, v), (mine, n)


# ---- error convention: message on stdout, then abort() ------------------------------
def _run_snippet(code):
    prog = ("import sys; sys.path.insert(0, %r)\nimport __graft_entry__ as e\nhost = e.load_package().host\n"
            "rt = host.runtime()\nimport ctypes as C\n" % REPO) + code
    return subprocess.run([sys.executable, "-c", prog], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                          timeout=120)


def test_spirv_blob_is_rejected_before_any_gpu_call():
    r = _run_snippet("blob = C.create_string_buffer(b'\\x03\\x02\\x23\\x07' + b'\\0' * 60)\n"
                     "rt.gpuModuleLoad(None, blob, 64)\nprint('survived')\n")
    assert r.returncode == -6  # SIGABRT
    assert "An exception was thrown: gpuModuleLoad: blob is SPIR-V" in r.stdout
    assert "survived" not in r.stdout


def test_garbage_and_null_blobs_abort():
    r = _run_snippet("blob = C.create_string_buffer(b'garbage!' * 8)\nrt.gpuModuleLoad(None, blob, 64)\n")
    assert r.returncode == -6 and "not a code object" in r.stdout
    # an ELF for another machine (x86-64 = 62) is refused by its header, before any HIP call
    r = _run_snippet("blob = C.create_string_buffer(b'\\x7fELF' + bytes(14) + bytes([62, 0]) + bytes(44))\nrt.gpuModuleLoad(None, blob, 64)\n")
    assert r.returncode == -6 and "not an AMDGPU code object" in r.stdout
    r = _run_snippet("rt.gpuModuleLoad(None, None, 0)\n")
    assert r.returncode == -6 and "null module data" in r.stdout
    r = _run_snippet("rt.gpuKernelGet(None, None, b'k')\n")
    assert r.returncode == -6 and "gpuKernelGet: null module" in r.stdout
    r = _run_snippet("rt.gpuLaunchKernel(None, None, 1,1,1, 1,1,1, 0, None, None)\n")
    assert r.returncode == -6 and "null stream" in r.stdout


def test_null_free_is_ignored_and_unload_is_noop():
    r = _run_snippet("rt.gpuMemFree(None, None)\nrt.gpuModuleUnload(None, None)\nrt.mgpuModuleUnload(None)\nprint('ok')\n")
    assert r.returncode == 0 and "ok" in r.stdout


# ---- runner utilities ------------------------------------------------------------------
class Desc2D(C.Structure):
    _fields_ = [("allocated", C.c_void_p), ("aligned", C.c_void_p), ("offset", C.c_int64),
                ("sizes", C.c_int64 * 2), ("strides", C.c_int64 * 2)]


class Unranked(C.Structure):
    _fields_ = [("rank", C.c_int64), ("descriptor", C.c_void_p)]


def memref2d(a):
    d = Desc2D(a.ctypes.data, a.ctypes.data, 0, (C.c_int64 * 2)(*a.shape), (C.c_int64 * 2)(a.shape[1], 1))
    u = Unranked(2, C.cast(C.pointer(d), C.c_void_p))
    return u, d


def test_runner_utils_gemm_matches_oracle_and_golden(host, orc):
    ru = host.runner_utils()
    a = orc.fill_uniform(24 * 40, "f16", 1, -1, 1).reshape(24, 40)
    b = orc.fill_uniform(40 * 16, "f16", 2, -1, 1).reshape(40, 16)
    c = np.zeros((24, 16), np.float32)
    (ua, da), (ub, db), (uc, dc) = memref2d(a), memref2d(b), memref2d(c)
    ru._mlir_ciface_gemmF16F16F32(C.byref(ua), C.byref(ub), C.byref(uc))
    assert np.array_equal(c, orc.gemm(a, b, "f16"))
    ab = orc.fill_uniform(24 * 40, "bf16", 3, -1, 1).reshape(24, 40)
    bb = orc.fill_uniform(40 * 16, "bf16", 4, -1, 1).reshape(40, 16)
    c2 = np.ones((24, 16), np.float32)
    (ua, da), (ub, db), (uc, dc) = memref2d(ab), memref2d(bb), memref2d(c2)
    ru._mlir_ciface_gemmBF16BF16F32(C.byref(ua), C.byref(ub), C.byref(uc))
    assert np.array_equal(c2, orc.gemm(ab, bb, "bf16", c=np.ones((24, 16), np.float32)))
    c3 = np.zeros((24, 16), np.float32)
    (ua, da), (ub, db), (uc, dc) = memref2d(a), memref2d(b), memref2d(c3)
    ru._mlir_ciface_gemmF16F16F16(C.byref(ua), C.byref(ub), C.byref(uc))
    assert np.array_equal(c3, orc.gemm(a, b, "f16", out_round="f16"))


def test_runner_utils_allclose_and_fill(host, orc):
    ru = host.runner_utils()
    ref = orc.fill_uniform(64, "f32", 5, -2, 2).reshape(8, 8)
    near = (ref * np.float32(1.0005)).astype(np.float32)
    far = ref.copy()
    far[3, 3] += 0.01
    (ur, dr), (un, dn), (uf, df) = memref2d(ref), memref2d(near), memref2d(far)
    assert ru._mlir_ciface_allcloseF32(C.byref(un), C.byref(ur)) is True
    assert ru._mlir_ciface_allcloseF32(C.byref(uf), C.byref(ur)) is False
    assert orc.allclose_f32(near, ref) and not orc.allclose_f32(far, ref)
    h = orc.float_to_half(ref)
    (uh, dh) = memref2d(h)
    assert ru._mlir_ciface_allcloseF16(C.byref(uh), C.byref(ur)) == orc.allclose_f32(orc.half_to_float(h), ref)
    buf = np.zeros((4, 6), np.uint16)
    (ub, db) = memref2d(buf)
    ru._mlir_ciface_fillResource1DBF16.argtypes = [C.c_void_p, C.c_float]
    ru._mlir_ciface_fillResource1DBF16(C.byref(ub), 1.5)
    assert np.all(buf == 0x3fc0)
    os.environ["IMEX_RANDOM_SEED"] = "7"
    r1 = np.zeros((5, 5), np.float32)
    (u1, d1) = memref2d(r1)
    ru._mlir_ciface_fillResource1DRandomF32.argtypes = [C.c_void_p, C.c_float, C.c_float, C.c_bool]
    ru._mlir_ciface_fillResource1DRandomF32(C.byref(u1), -0.5, 0.5, False)
    assert r1.min() >= -0.5 and r1.max() < 0.5 and len(np.unique(r1)) > 20
    del os.environ["IMEX_RANDOM_SEED"]


def test_runner_utils_conversions_exhaustive(host, orc):
    """allcloseF16 / allcloseBF16 widen with the library's own converters: compare
    all 65536 patterns against the oracle by filling through the library."""
    ru = host.runner_utils()
    vals = orc.half_to_float(np.arange(0x7c00, dtype=np.uint16)).reshape(-1, 64)
    out = np.zeros(vals.shape, np.uint16)
    ref = np.ascontiguousarray(vals)
    (uo, do), (ur, dr) = memref2d(out), memref2d(ref)
    # every finite half survives f32 -> f16 through the library: allclose with itself is exact
    for i, v in enumerate(ref.ravel()[:: 997]):
        one = np.zeros((1, 1), np.uint16)
        (u1, d1) = memref2d(one)
        ru._mlir_ciface_fillResource1DF16.argtypes = [C.c_void_p, C.c_float]
        ru._mlir_ciface_fillResource1DF16(C.byref(u1), float(v))
        assert one[0, 0] == orc.float_to_half(np.array([v], np.float32))[0]


def test_print_helpers(host, orc, capfd):
    ru = host.runner_utils()
    g = np.array([[14.1, 14.8, 14.6], [11, 13, 10.5], [13.9, 19.9, 12.4]], np.float32)
    h = orc.float_to_half(g)
    (uh, dh), (ug, dg) = memref2d(h), memref2d(g)
    ru._mlir_ciface_printAllcloseF16(C.byref(uh), C.byref(ug))
    ru._mlir_ciface_printMemrefF16(C.byref(uh))
    ru._mlir_ciface_printMaxErrorF32(C.byref(ug), C.byref(ug))
    C.CDLL(None).fflush(None)  # the library prints through C++ iostreams
    out = capfd.readouterr().out
    assert "[ALLCLOSE: TRUE]" in out
    assert "sizes = [3, 3] strides = [3, 1] data =" in out
    assert "[11,   13,   10.5]" in out
    assert "Max absolute error 0" in out


def test_driver_command_line():
    """Parts of the C++ driver that need no GPU: the workload list, bench_imex's -c
    (not offered) and an unknown workload name."""
    import subprocess
    exe = os.path.join(REPO, "mlir-extensions_amd", "lib", "imex-hip-bench")
    r = subprocess.run([exe, "--list"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert r.returncode == 0
    names = [l.split()[0] for l in r.stdout.splitlines() if l.strip()]
    assert "gemm_f16_4096" in names and "flash_attention_f16_2x2x4096x64" in names and len(names) >= 11
    r = subprocess.run([exe, "-c", "all"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert r.returncode == 1 and "CPU lowering" in r.stderr
    r = subprocess.run([exe, "no_such_workload"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert r.returncode == 2 and "unknown workload" in r.stderr


def test_launch_shapes_cover_the_problem(host):
    """For the kernels that do not stride over their work (element-wise, reductions,
    fused chains, tiled GEMM) the catalogue's grid must cover every element; checked
    over random problem sizes against each kernel's work per workgroup."""
    from hypothesis import given, settings, strategies as st
    ls = host.launch_shape

    @settings(max_examples=300, deadline=None)
    @given(n=st.integers(1, 1 << 34))
    def eltwise(n):
        small = n < (1 << 22)
        for name, per in (("imex_relu_f32", 4096), ("imex_silu_f32", 1024 if small else 4096), ("imex_relu_bf16", 8192),
                          ("imex_loop_fusion_f32", 1024 if small else 4096),
                          ("imex_loop_fusion_f16", 2048 if small else 8192)):
            (gx, gy, gz), block, _ = ls(name, [n])
            assert block == (256, 1, 1) and gy == gz == 1
            assert (gx - 1) * per < n <= gx * per

    @settings(max_examples=300, deadline=None)
    @given(rows=st.integers(1, 1 << 20), cols=st.integers(1, 1 << 14))
    def rowwise(rows, cols):
        (gx, _, _), _, _ = ls("imex_rowsum_f32", [rows, cols])
        assert gx == rows if cols > 2048 else gx * 4 >= rows
        (gx, _, _), _, _ = ls("imex_reduce_outer_f32", [rows, cols])
        assert gx >= 1 and gx * 8192 >= cols  # the kernel strides over whatever the grid leaves
        (gx, _, _), _, _ = ls("imex_input_fusion_f32", [rows, cols])
        assert gx * 64 >= cols
        (gx, _, _), _, _ = ls("imex_softmax_f16", [rows, cols])
        assert gx >= 1 and (gx == min(-(-rows // 4), 2048) if cols <= 1024 else gx >= min(rows, 1048560))
        (gx, _, _), _, _ = ls("imex_softmax_bf16", [rows, cols])
        assert gx >= 1 and (gx * (8 if rows >= 16384 else 4) >= rows if cols <= 1024 else gx >= min(rows, 1048560))

    @settings(max_examples=300, deadline=None)
    @given(M=st.integers(1, 20000), N=st.integers(1, 20000), k=st.integers(1, 512), round_n=st.booleans(),
           round_k=st.booleans())
    def gemm(M, N, k, round_n, round_k):
        N = (N + 7) // 8 * 8 if round_n else N
        K = k * 8 if round_k else k * 7 + 5
        for name in ("imex_gemm_f16_f16_f32", "imex_gemm_f16_f16_f32_ta", "imex_gemm_f16_f16_f32_tb",
                     "imex_gemm_bf16_bias_silu_bf16"):
            (gx, gy, gz), block, _ = ls(name, [M, N, K])
            assert block == (512, 1, 1) and gy == gz == 1
            tileable = K % 8 == 0 and (name.endswith("_tb") or N % 8 == 0) and (not name.endswith("_ta") or M % 8 == 0)
            assert gx == (-(-M // 256) * -(-N // 256) if tileable else -(-M // 128) * -(-N // 128))

    eltwise()
    rowwise()
    gemm()
