"""GPU tests of the runtime-wrapper ABI itself: allocation kinds, copies in every
direction, module/kernel caching, event dependencies, the profiling loop and the
upstream mgpu* entry points."""
import ctypes as C
import os
import subprocess
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_shared_allocation_is_host_dereferenceable(host, orc, stream):
    n = 4096 + 5
    p_in = stream.alloc(n * 4, shared=True)
    p_out = stream.alloc(n * 4, shared=True)
    assert int(p_in) % 256 == 0
    x = orc.fill_uniform(n, "f32", 1, -1, 1)
    # host code writes straight into the shared buffer, as JIT'd memref.copy does
    C.memmove(int(p_in), x.ctypes.data, n * 4)
    stream.launch("imex_relu_f32", [n], [p_in, p_out, n])
    stream.wait()
    got = np.ctypeslib.as_array(C.cast(int(p_out), C.POINTER(C.c_float)), shape=(n,)).copy()
    assert np.array_equal(got, orc.relu_f32(x))
    stream.free(p_in)
    stream.free(p_out)


def test_copies_in_every_direction(host, stream):
    x = np.arange(100000, dtype=np.uint32)
    d1, d2 = stream.alloc(x.nbytes), stream.alloc(x.nbytes)
    stream.copy(d1, x.ctypes.data, x.nbytes)     # H2D
    stream.copy(d2, d1, x.nbytes)                # D2D
    y = np.zeros_like(x)
    stream.copy(y.ctypes.data, d2, x.nbytes)     # D2H
    z = np.zeros_like(x)
    stream.copy(z.ctypes.data, y.ctypes.data, x.nbytes)  # H2H
    assert np.array_equal(x, y) and np.array_equal(x, z)
    stream.copy(d1, x.ctypes.data, 0)            # empty copy is a no-op
    stream.free(d1)
    stream.free(d2)


def test_alignment_and_zero_size(host, stream):
    p = stream.alloc(1000, alignment=4096)
    assert int(p) % 4096 == 0
    stream.free(p)
    q = stream.alloc(0)
    assert int(q) != 0
    stream.free(q)


def test_module_and_kernel_caching(host, stream):
    rt, k = stream.rt, host.kernels()
    size = C.c_size_t(0)
    blob = k.imexHipKernelModule(b"imex_relu_f32", C.byref(size))
    m1 = rt.gpuModuleLoad(stream.handle, blob, size.value)
    m2 = rt.gpuModuleLoad(stream.handle, blob, size.value)
    assert m1 == m2 and m1
    f1 = rt.gpuKernelGet(stream.handle, m1, b"imex_relu_f32")
    f2 = rt.gpuKernelGet(stream.handle, m1, b"imex_relu_f32")
    assert f1 == f2 and f1
    assert rt.gpuKernelGet(stream.handle, m1, b"imex_silu_f32") != f1


def test_unknown_kernel_name_aborts_with_message():
    prog = ("import sys; sys.path.insert(0, %r)\nimport __graft_entry__ as e\nhost = e.load_package().host\n"
            "import ctypes as C\ns = host.Stream()\nsize = C.c_size_t(0)\n"
            "blob = host.kernels().imexHipKernelModule(b'imex_relu_f32', C.byref(size))\n"
            "m = s.rt.gpuModuleLoad(s.handle, blob, size.value)\ns.rt.gpuKernelGet(s.handle, m, b'no_such_kernel')\n" % REPO)
    r = subprocess.run([sys.executable, "-c", prog], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert r.returncode == -6
    assert "An exception was thrown: gpuKernelGet: kernel 'no_such_kernel' not found" in r.stdout


def test_event_dependencies_across_streams(host, orc):
    n = 1 << 20
    x = orc.fill_uniform(n, "f32", 3, -1, 1)
    with host.Stream() as s1, host.Stream() as s2:
        d_in, d_mid, d_out = s1.to_device(x), s1.alloc(n * 4), s1.alloc(n * 4)
        ev = s1.launch("imex_silu_f32", [n], [d_in, d_mid, n])
        assert ev
        # the second stream's launch waits on the first stream's event
        s2.launch("imex_relu_f32", [n], [d_mid, d_out, n], deps=[ev])
        s2.wait()
        got = s2.from_device(d_out, (n,), np.float32)
        assert np.array_equal(got, orc.relu_f32(orc.silu_f32(x)))
        t0 = s1.timestamp()
        s1.launch("imex_silu_f32", [n], [d_in, d_mid, n])
        t1 = s1.timestamp()
        assert 0.0 < s1.elapsed_ms(t0, t1) < 100.0
        for p in (d_in, d_mid, d_out):
            s1.free(p)


def test_launch_events_are_recycled_safely(host, orc):
    """Launch events come from a 4096-slot ring per stream: a handle older than that
    still orders a dependent launch after the work it stood for."""
    n = 4096
    x = orc.fill_uniform(n, "f32", 9, -1, 1)
    with host.Stream() as s1, host.Stream() as s2:
        d_in, d_mid, d_out = s1.to_device(x), s1.alloc(n * 4), s1.alloc(n * 4)
        step = s1.prepare("imex_relu_f32", [n], [d_in, d_mid, n])
        first = s1.launch("imex_relu_f32", [n], [d_in, d_mid, n])
        for _ in range(5000):
            step()
        last = s1.launch("imex_silu_f32", [n], [d_in, d_mid, n])
        assert first and last
        s2.launch("imex_relu_f32", [n], [d_mid, d_out, n], deps=[first, last])
        s2.wait()
        got = s2.from_device(d_out, (n,), np.float32)
        assert np.array_equal(got, orc.relu_f32(orc.silu_f32(x)))
        for p in (d_in, d_mid, d_out):
            s1.free(p)


def test_profile_helper_modes(host, orc, stream):
    n = 1 << 22
    d_in, d_out = stream.to_device(orc.fill_uniform(n, "f32", 4, -1, 1)), stream.alloc(n * 4)
    per_launch = stream.profile("imex_relu_f32", [n], [d_in, d_out, n], warmups=2, rounds=10, mode=0)
    assert len(per_launch) == 10 and all(0 < t < 50 for t in per_launch)
    flushed = stream.profile("imex_relu_f32", [n], [d_in, d_out, n], warmups=2, rounds=5, flush_bytes=64 << 20, mode=0)
    assert len(flushed) == 5 and all(t > 0 for t in flushed)
    total = stream.profile("imex_relu_f32", [n], [d_in, d_out, n], warmups=2, rounds=10, mode=1)
    assert len(total) == 1 and 0 < total[0] < 500
    stream.free(d_in)
    stream.free(d_out)


def test_profiled_launch_runs_the_whole_grid(host, orc, stream):
    """The profiler's timed launches attach their timestamps to the dispatch through a launch call that
    takes sizes in work-items, not workgroups: a launch with a two-dimensional grid must still cover the
    whole problem, flushed or not."""
    zh, n_ctx = 3, 512
    q, k, v = (orc.fill_uniform(zh * n_ctx * 64, "f16", 70 + i, -1, 1).reshape(zh * n_ctx, 64) for i in range(3))
    expected = host.flash_attention(stream, q, k, v, zh, n_ctx, 0.125)
    d_q, d_k, d_v = stream.to_device(q), stream.to_device(k), stream.to_device(v)
    d_o = stream.alloc(q.size * 2)
    for flush_bytes in (0, 16 << 20):
        stream.memset(d_o, 0x7e00, q.size, 16)
        times = stream.profile("imex_flash_attention_fwd_f16", [zh, n_ctx], [d_q, d_k, d_v, d_o, 0.125, zh, n_ctx],
                               warmups=0, rounds=2, flush_bytes=flush_bytes, mode=0)
        assert len(times) == 2 and all(0 < t < 50 for t in times)
        assert np.array_equal(stream.from_device(d_o, q.shape, np.uint16), expected)
    for p in (d_q, d_k, d_v, d_o):
        stream.free(p)


def test_profiling_env_prints_reference_line():
    prog = ("import sys; sys.path.insert(0, %r)\nimport __graft_entry__ as e\nimport numpy as np\n"
            "host = e.load_package().host\ns = host.Stream()\n"
            "y = host.relu(s, np.linspace(-1, 1, 5000).astype(np.float32))\nprint('result', float(y.sum()))\n" % REPO)
    env = dict(os.environ, IMEX_ENABLE_PROFILING="1", IMEX_PROFILING_RUNS="7", IMEX_PROFILING_WARMUPS="2",
               IMEX_ENABLE_CACHE_FLUSHING="1", IMEX_CACHE_FLUSH_BYTES=str(32 << 20))
    r = subprocess.run([sys.executable, "-c", prog], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                       timeout=300, env=env)
    assert r.returncode == 0, r.stdout + r.stderr
    line = [l for l in r.stdout.splitlines() if "execution time" in l]
    assert len(line) == 1
    assert line[0].startswith("the kernel execution time is (ms, on HIP runtime):avg: ")
    assert line[0].endswith("(over 7 runs)")
    for key in ("min:", "max:", "median:", "std_deviation:", "variance:", "P95:", "P5:", "median_one_third_avg:"):
        assert key in line[0]
    assert "result" in r.stdout  # the real launch still happens after profiling


def test_mgpu_entry_points(host, orc):
    rt, k = host.runtime(), host.kernels()
    n = 10000
    x = orc.fill_uniform(n, "f32", 5, -1, 1)
    s = rt.mgpuStreamCreate()
    d_in = rt.mgpuMemAlloc(n * 4, s, 0)
    d_out = rt.mgpuMemAlloc(n * 4, s, 0)
    rt.mgpuMemcpy(d_in, x.ctypes.data, n * 4, s)
    rt.mgpuMemset32(d_out, 0x3f800000, n, s)
    size = C.c_size_t(0)
    blob = k.imexHipKernelModule(b"imex_relu_f32", C.byref(size))
    fn = rt.mgpuModuleGetFunction(rt.mgpuModuleLoad(blob, size.value), b"imex_relu_f32")
    args = [C.c_void_p(d_in), C.c_void_p(d_out), C.c_int64(n)]
    argv = (C.c_void_p * 3)(*[C.cast(C.pointer(a), C.c_void_p) for a in args])
    grid, block, _ = host.launch_shape("imex_relu_f32", [n])
    ones = np.zeros(n, np.float32)
    rt.mgpuStreamSynchronize(s)
    rt.mgpuMemcpy(ones.ctypes.data, d_out, n * 4, s)
    assert np.all(ones == 1.0)
    rt.mgpuLaunchKernel(fn, grid[0], 1, 1, block[0], 1, 1, 0, s, argv, None, 3)
    rt.mgpuStreamSynchronize(s)
    y = np.zeros(n, np.float32)
    rt.mgpuMemcpy(y.ctypes.data, d_out, n * 4, s)
    assert np.array_equal(y, orc.relu_f32(x))
    rt.mgpuMemFree(s, d_in)
    rt.mgpuMemFree(s, d_out)
    rt.mgpuStreamDestroy(s)


@pytest.mark.parametrize("bits", [32, 16])
def test_memset_entry_points(host, bits):
    """gpuMemSet32 / gpuMemSet16 (stream first) and mgpuMemset16: fills that start and end off the
    16-byte grid, a length of zero, and what lies on either side of the filled range left alone."""
    np_t = np.uint32 if bits == 32 else np.uint16
    value = 0xdeadbeef if bits == 32 else 0xbf80  # bf16 -1.0
    with host.Stream() as s:
        for n, first in ((1, 0), (7, 3), (4096, 1), (100003, 5), ((1 << 21) + 9, 2)):
            size = n + first + 11
            back = np.arange(size, dtype=np.int64).astype(np_t)
            d = s.to_device(back)
            s.memset(int(d) + first * back.itemsize, value, n, bits=bits)
            s.memset(int(d), 0x1234, 0, bits=bits)  # nothing to do
            s.wait()
            got = s.from_device(d, (size,), np_t)
            assert np.all(got[first:first + n] == np_t(value)), (n, first)
            assert np.array_equal(got[:first], back[:first]) and np.array_equal(got[first + n:], back[first + n:]), (n, first)
            s.free(d)
        if bits == 16:
            d = s.alloc(2 * 1000)
            host.runtime().mgpuMemset16(int(d), 0x3c00, 1000, s.handle)  # f16 1.0
            s.wait()
            assert np.all(s.from_device(d, (1000,), np.uint16) == 0x3c00)
            s.free(d)


def test_timestamp_handles_recycle(host, orc):
    """Timestamps live in a 1024-slot ring per stream: recording thousands of them does not grow the
    queue, and the two most recent ones still time the launches between them."""
    n = 1 << 20
    with host.Stream() as s:
        d_in, d_out = s.to_device(orc.fill_uniform(n, "f32", 4, -1, 1)), s.alloc(n * 4)
        step = s.prepare("imex_relu_f32", [n], [d_in, d_out, n])
        seen = set()
        for _ in range(3000):
            seen.add(s.timestamp())
        assert len(seen) == 1024
        t0 = s.timestamp()
        for _ in range(20):
            step()
        t1 = s.timestamp()
        s.wait()
        assert 0.0 < s.elapsed_ms(t0, t1) < 100.0
        s.free(d_in)
        s.free(d_out)


def test_elapsed_time_refuses_launch_events():
    """A launch event is an ordering point without a time of its own: imexHipEventElapsedMs takes
    timestamps only, and says so through the ABI's error convention (message on stdout, abort)."""
    prog = ("import sys; sys.path.insert(0, %r)\nimport __graft_entry__ as e\nimport numpy as np\n"
            "host = e.load_package().host\ns = host.Stream()\nd = s.alloc(4096)\n"
            "ev = s.launch('imex_relu_f32', [1024], [d, d, 1024])\nt = s.timestamp()\ns.wait()\n"
            "print('before', flush=True)\ns.elapsed_ms(ev, t)\nprint('not reached')\n" % REPO)
    r = subprocess.run([sys.executable, "-c", prog], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert r.returncode != 0
    assert "before" in r.stdout and "not reached" not in r.stdout
    assert "An exception was thrown: imexHipEventElapsedMs: both events must come from imexHipRecordTimestamp" in r.stdout


def test_profiling_env_zero_warmups():
    """IMEX_PROFILING_WARMUPS=0 means no warm-up launches (LevelZeroRuntimeWrappers.cpp:547-551), not the default."""
    prog = ("import sys; sys.path.insert(0, %r)\nimport __graft_entry__ as e\nimport numpy as np\n"
            "host = e.load_package().host\ns = host.Stream()\n"
            "y = host.relu(s, np.linspace(-1, 1, 5000).astype(np.float32))\nprint('result', float(y.sum()))\n" % REPO)
    env = dict(os.environ, IMEX_ENABLE_PROFILING="1", IMEX_PROFILING_RUNS="4", IMEX_PROFILING_WARMUPS="0")
    r = subprocess.run([sys.executable, "-c", prog], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                       timeout=300, env=env)
    assert r.returncode == 0, r.stdout + r.stderr
    assert sum("execution time" in l and l.endswith("(over 4 runs)") for l in r.stdout.splitlines()) == 1


def test_driver_report_mode(tmp_path):
    """The C++ driver in bench_imex's role: one child process per workload, their
    "execution time" lines collected in a report file (benchmarks/bench_imex.in:72-91)."""
    exe = os.path.join(REPO, "mlir-extensions_amd", "lib", "imex-hip-bench")
    report = tmp_path / "report.txt"
    r = subprocess.run([exe, "-l", "--runs", "5", "--warmups", "2", "--report", str(report),
                        "relu_f32_4096x4096", "softmax_f16_16384x1024"],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = report.read_text().splitlines()
    assert any(l.startswith("================ Imex Perf (HIP) @ ") for l in lines)
    timed = [l for l in lines if "execution time" in l]
    assert len(timed) == 2
    assert timed[0].startswith("relu_f32_4096x4096: the kernel execution time is (ms, on HIP runtime):avg: ")
    assert timed[1].startswith("softmax_f16_16384x1024: the kernel execution time is (ms, on HIP runtime):avg: ")
    assert all(l.endswith("(over 5 runs)") for l in timed)


def test_driver_runs_every_workload():
    """Every workload the C++ driver lists goes through the whole ABI sequence once
    (allocate, fill, copy, load, launch, time, copy back, free) and reports a rate."""
    exe = os.path.join(REPO, "mlir-extensions_amd", "lib", "imex-hip-bench")
    listed = subprocess.run([exe, "--list"], stdout=subprocess.PIPE, text=True, timeout=60).stdout.split("\n")
    names = [l.split()[0] for l in listed if l.strip()]
    assert len(names) >= 20
    r = subprocess.run([exe, "--runs", "3", "--warmups", "1", "all"], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                       text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    for n in names:
        assert any(l.startswith(n + ": back-to-back") for l in r.stdout.splitlines()), n


def test_driver_lds_service_probe_mode():
    """`--lds-service` launches one two-lane LDS probe per question (6 access kinds x (63 lane pairs + 7
    distances)) and names each dispatch in launch order, which is what a bank-conflict counter run is decoded by."""
    exe = os.path.join(REPO, "mlir-extensions_amd", "lib", "imex-hip-bench")
    r = subprocess.run([exe, "--lds-service"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("dispatch ")]
    assert len(lines) == 6 * 70
    assert lines[0] == "dispatch 1: ds_read_b128 lanes 0 and 1, 1024 bytes apart"
    assert lines[-1] == "dispatch 420: ds_write_b32 lanes 0 and 1, 1024 bytes apart"


def test_adopted_stream_and_graph_replay(host, orc):
    """A queue built on a caller's hipStream_t (the `context` argument of gpuCreateStream) launches
    on that stream, so a launch-bound sequence can be captured into a HIP graph and replayed:
    here the fused chain out = (log a + |b|) - a feeding a ReLU, three replays with fresh inputs,
    each checked against the oracle and against the same two launches run eagerly."""
    import ctypes as C
    import numpy as np
    hip = C.CDLL("libamdhip64.so")
    raw = C.c_void_p()
    assert hip.hipStreamCreateWithFlags(C.byref(raw), 1) == 0  # non-blocking, default priority
    s = host.Stream(hip_stream=raw.value)
    n = 70000
    a = orc.fill_uniform(n, "f32", 201, 0.5, 3.0)
    b = orc.fill_uniform(n, "f32", 202, -3.0, 3.0)
    d_a, d_b, d_t, d_o = s.to_device(a), s.to_device(b), s.alloc(n * 4), s.alloc(n * 4)
    chain = s.prepare("imex_loop_fusion_f32", [n], [d_a, d_b, d_t, n])
    relu = s.prepare("imex_relu_f32", [n], [d_t, d_o, n])
    d_m = s.alloc(n * 4 + 4)
    marks = int(d_m) + 4, 0x3fc00000, n - 3     # a fill that starts and ends off the 16-byte grid
    chain(), relu()   # eager once: modules loaded, kernels resolved, nothing left to allocate under capture
    s.fill32(*marks)
    s.wait()
    want = orc.relu_f32(orc.loop_fusion_f32(a, b))
    assert np.array_equal(s.from_device(d_o, (n,), np.float32).view(np.uint32), want.view(np.uint32))

    graph, exe = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(raw, 2) == 0          # relaxed mode
    s.fill32(*marks)                                        # the fill is a kernel, so an ordinary graph node
    chain(), relu()
    assert hip.hipStreamEndCapture(raw, C.byref(graph)) == 0
    assert hip.hipGraphInstantiate(C.byref(exe), graph, None, None, C.c_size_t(0)) == 0
    for seed in (203, 204, 205):
        a2 = orc.fill_uniform(n, "f32", seed, 0.5, 3.0)
        s.copy(d_a, a2.ctypes.data, n * 4)                  # new input, same buffers
        zeros, stale = np.zeros(n, np.float32), np.full(n + 1, seed, np.uint32)  # named: alive until copied
        s.copy(d_o, zeros.ctypes.data, n * 4)
        s.copy(d_m, stale.ctypes.data, n * 4 + 4)
        assert hip.hipGraphLaunch(exe, raw) == 0
        s.wait()
        filled = s.from_device(d_m, (n + 1,), np.uint32)
        assert filled[0] == seed and np.all(filled[1:n - 2] == 0x3fc00000) and np.all(filled[n - 2:] == seed), seed
        got = s.from_device(d_o, (n,), np.float32)
        assert np.array_equal(got.view(np.uint32), orc.relu_f32(orc.loop_fusion_f32(a2, b)).view(np.uint32)), seed
    assert hip.hipGraphExecDestroy(exe) == 0 and hip.hipGraphDestroy(graph) == 0
    for p in (d_a, d_b, d_t, d_o, d_m):
        s.free(p)
    s.close()                                               # must leave the adopted stream alive
    assert hip.hipStreamSynchronize(raw) == 0
    assert hip.hipStreamDestroy(raw) == 0
