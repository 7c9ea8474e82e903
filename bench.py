#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME,...] [--no-cpu]

A "step" is one launch of the headline kernel -- the f16 4096^3 GEMM, the
workload the MFMA target of BASELINE.json is quoted on -- over synthetic seeded
inputs already resident in HBM.  K steps are timed between two stream
synchronisations; the same region is also timed with HIP events recorded on the
launch stream through the C ABI.  Every other configuration of BASELINE.json is
measured too and reported under "per_config" under three protocols (the same
buffers back to back, a ring of buffer sets larger than every cache, and the
reference profiler's cache flush before each launch), each with its roofline
fraction and a single-core CPU baseline.

Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

REPO = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, REPO)
import __graft_entry__ as entry  # noqa: E402

METRIC = "GEMM TFLOP/s (% MFMA peak) + softmax/reduce/transpose GB/s (% HBM peak), 1 GPU"
HBM_PEAK_GBS = 8000.0       # MI355X published HBM3E bandwidth
MFMA_PEAK_TFLOPS = 2500.0   # MI355X published dense f16 / bf16 MFMA rate
FLUSH_BYTES = 512 << 20     # > L2 (8 x 4 MiB) + 256 MiB Infinity Cache
SETTLE_LAUNCHES = 300       # untimed launches of the headline kernel before the caller's warm-up and timed steps
# the reference's CPU benchmark templates (benchmarks/relu/relu_cpu.mlir.in:22-61): warm-ups, then wall-clocked calls
# that allocate their result inside the timed call, average reported
CPU_PROTOCOL = "full tensor, %d warm-ups + %d timed calls, result allocated inside each call, one core"


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


# ---- seeded synthetic inputs -------------------------------------------------------------------
# The raw output stream of std::mt19937 (numpy's MT19937 with the classic integer seeding is the
# same generator) and the transforms of the benchmark definition: uniform u = (w >> 8) * 2^-24,
# x = lo + (hi - lo) u in f64; normal by Box-Muller in f64 on two such uniforms; raw bit patterns
# with NaN encodings redrawn.  f64 -> f32 -> f16 / bf16, each step round-to-nearest-even.
def _mt19937_raw(seed, n):
    bitgen = np.random.MT19937()
    bitgen._legacy_seeding(seed)
    return bitgen.random_raw(n).astype(np.uint32)


def _narrow(x64, dtype):
    f = x64.astype(np.float32)
    if dtype == "f32":
        return f
    if dtype == "f16":
        return f.astype(np.float16).view(np.uint16)
    u = f.view(np.uint32)
    rounded = ((u + (((u >> 16) & 1) + 0x7fff)) >> 16).astype(np.uint16)
    nan = (u & 0x7fffffff) > 0x7f800000
    return np.where(nan, np.where(u >> 31, 0xffc0, 0x7fc0).astype(np.uint16), rounded)


def gen_uniform(n, dtype, seed, lo, hi):
    u = (_mt19937_raw(seed, n) >> 8).astype(np.float64) * (1.0 / 16777216.0)
    return _narrow(lo + (hi - lo) * u, dtype)


def gen_normal(n, dtype, seed, mu, sigma):
    pairs = (n + 1) // 2
    w = _mt19937_raw(seed, 2 * pairs)
    u1 = ((w[0::2] >> 8) + 1).astype(np.float64) * (1.0 / 16777216.0)
    u2 = (w[1::2] >> 8).astype(np.float64) * (1.0 / 16777216.0)
    r, angle = np.sqrt(-2.0 * np.log(u1)), 6.283185307179586476925286766559 * u2
    out = np.empty(2 * pairs, np.float64)
    out[0::2] = mu + sigma * (r * np.cos(angle))
    out[1::2] = mu + sigma * (r * np.sin(angle))
    return _narrow(out[:n], dtype)


def gen_bits(n, dtype, seed):
    """Raw words masked to the element width, NaN encodings skipped (each element takes the next
    word of the stream that is not a NaN)."""
    out = np.empty(0, np.uint32)
    drawn = 0
    stream = _mt19937_raw(seed, n + n // 16 + 1024)   # f16 words are NaNs 3 % of the time
    while True:
        w = stream[drawn:]
        if dtype == "f32":
            keep = ~(((w & 0x7f800000) == 0x7f800000) & ((w & 0x007fffff) != 0))
            vals = w[keep]
        else:
            h = w & 0xffff
            exp, man = (0x7c00, 0x03ff) if dtype == "f16" else (0x7f80, 0x007f)
            vals = h[~(((h & exp) == exp) & ((h & man) != 0))]
        out = np.concatenate([out, vals])
        if out.size >= n:
            break
        drawn = stream.size
        stream = _mt19937_raw(seed, 2 * stream.size)   # the same stream, longer
    out = out[:n]
    return out.view(np.float32) if dtype == "f32" else out.astype(np.uint16)


class Workload:
    """One BASELINE.json configuration: device buffers, the kernel launch, its algorithmic
    work and the matching CPU-baseline call."""

    def __init__(self, name, kernel, dims, bound, work, unit, dtype, describe):
        self.name, self.kernel, self.dims = name, kernel, dims
        self.bound, self.work, self.unit, self.dtype, self.describe = bound, work, unit, dtype, describe
        self.args = None
        self.buffers = []
        self.sizes = {}  # device pointer value -> (bytes, is_input)
        self.cpu = None  # callable -> (value, sample description)


def build_workloads(host, orc, stream, only):
    wl = []

    def want(name):
        return only is None or name in only

    def dev(a):
        p = stream.to_device(a)
        cur.buffers.append(p)
        cur.sizes[int(p)] = (a.nbytes, True)
        return p

    def out(nbytes):
        p = stream.alloc(nbytes)
        cur.buffers.append(p)
        cur.sizes[int(p)] = (nbytes, False)
        return p

    if want("gemm_f16_4096"):
        M = N = K = 4096
        cur = Workload("gemm_f16_4096", "imex_gemm_f16_f16_f32", [M, N, K], "mfma", 2.0 * M * N * K, "TFLOP/s",
                       "f16", "C[4096,4096] f32 = A[4096,4096] f16 . B[4096,4096] f16, uniform(-1,1), seeds 20246/20247")
        a = gen_uniform(M * K, "f16", 20246, -1.0, 1.0).reshape(M, K)
        b = gen_uniform(K * N, "f16", 20247, -1.0, 1.0).reshape(K, N)
        cur.args = [dev(a), dev(b), out(M * N * 4), M, N, K]
        rows = 4096

        def cpu(a=a, b=b, rows=rows, N=N, K=K):  # (N and K bound here: later workloads reuse the names)
            t = time.perf_counter()
            ms = orc.time_gemm_rows(a, b, rows, "f16")
            wall_s = time.perf_counter() - t
            log("cpu baseline gemm_f16_4096: %.0f GFLOP in %.2f s inside the oracle's own bracket, %.2f s around the call" % (
                2.0 * rows * N * K / 1e9, ms / 1e3, wall_s))
            return 2.0 * rows * N * K / (ms * 1e9), "all %d rows of C (the whole workload), one un-warmed call of the i-k-j loop" % rows
        cur.cpu = cpu
        wl.append(cur)

    if want("gemm_mlp_bf16"):
        M, K, N = 4096, 4096, 11008
        cur = Workload("gemm_mlp_bf16", "imex_gemm_bf16_bias_silu_bf16", [M, N, K], "mfma", 2.0 * M * N * K, "TFLOP/s",
                       "bf16", "out[4096,11008] bf16 = silu(A[4096,4096] bf16 . B[4096,11008] bf16 + bias f32), seeds 20248-20250")
        a = gen_normal(M * K, "bf16", 20248, 0.0, 1.0).reshape(M, K)
        b = gen_normal(K * N, "bf16", 20249, 0.0, 0.02).reshape(K, N)
        bias = gen_normal(N, "f32", 20250, 0.0, 0.1)
        cur.args = [dev(a), dev(b), dev(bias), out(M * N * 2), M, N, K]
        rows = 512

        def cpu(a=a, b=b, bias=bias, rows=rows, N=N, K=K):
            ms = orc.time_mlp_rows(a, b, bias, rows)
            return 2.0 * rows * N * K / (ms * 1e9), ("first %d of 4096 rows: the i-k-j GEMM loop, then bias + SiLU + rounding "
                                                     "to bf16; one un-warmed call" % rows)
        cur.cpu = cpu
        wl.append(cur)

    if want("relu_f32"):
        n = 4096 * 4096
        cur = Workload("relu_f32", "imex_relu_f32", [n], "hbm", 2.0 * n * 4, "GB/s", "f32",
                       "relu f32 [4096,4096] uniform(-1,1) seed 20241, out of place")
        x = gen_uniform(n, "f32", 20241, -1.0, 1.0)
        cur.args = [dev(x), out(n * 4), n]
        cur.cpu = lambda x=x: (2.0 * x.size * 4 / (orc.time_relu_f32(x, 5, 200) * 1e6), CPU_PROTOCOL % (5, 200))
        wl.append(cur)

    if want("softmax_f16"):
        rows, cols = 16384, 1024
        cur = Workload("softmax_f16", "imex_softmax_f16", [rows, cols], "hbm", 2.0 * rows * cols * 2, "GB/s", "f16",
                       "softmax f16 [16384,1024] normal(0,2) seed 20242, f32 internals")
        x = gen_normal(rows * cols, "f16", 20242, 0.0, 2.0).reshape(rows, cols)
        cur.args = [dev(x), out(rows * cols * 2), rows, cols]
        cur.cpu = lambda x=x: (2.0 * x.size * 2 / (orc.time_softmax_f16(x, 5, 100) * 1e6), CPU_PROTOCOL % (5, 100))
        wl.append(cur)

    if want("rowsum_f32"):
        rows = cols = 8192
        cur = Workload("rowsum_f32", "imex_rowsum_f32", [rows, cols], "hbm", rows * cols * 4.0 + rows * 4.0, "GB/s",
                       "f32", "row-sum f32 [8192,8192] uniform(0,1) seed 20243 -> [8192]")
        x = gen_uniform(rows * cols, "f32", 20243, 0.0, 1.0).reshape(rows, cols)
        cur.args = [dev(x), out(rows * 4), rows, cols, 0.0]
        cur.cpu = lambda x=x: ((x.size * 4.0 + x.shape[0] * 4.0) / (orc.time_rowsum_f32(x, 5, 200) * 1e6), CPU_PROTOCOL % (5, 200))
        wl.append(cur)

    if want("transpose_f32"):
        rows = cols = 4096
        cur = Workload("transpose_f32", "imex_transpose2d_b32", [rows, cols], "hbm", 2.0 * rows * cols * 4, "GB/s",
                       "f32", "transpose f32 [4096,4096] random non-NaN bits seed 20245")
        x = gen_bits(rows * cols, "f32", 20245).reshape(rows, cols)
        cur.args = [dev(x), out(rows * cols * 4), rows, cols]
        cur.cpu = lambda x=x: (2.0 * x.size * 4 / (orc.time_transpose2d(x, 5, 100) * 1e6), CPU_PROTOCOL % (5, 100))
        wl.append(cur)

    if want("transpose_bf16"):
        rows = cols = 8192
        cur = Workload("transpose_bf16", "imex_transpose2d_b16", [rows, cols], "hbm", 2.0 * rows * cols * 2, "GB/s",
                       "bf16", "transpose bf16 [8192,8192] random non-NaN bits seed 20244")
        x = gen_bits(rows * cols, "bf16", 20244).reshape(rows, cols)
        cur.args = [dev(x), out(rows * cols * 2), rows, cols]
        cur.cpu = lambda x=x: (2.0 * x.size * 2 / (orc.time_transpose2d(x, 5, 20) * 1e6),
                             CPU_PROTOCOL % (5, 20) + " (20 instead of the template's 100: a call takes ~0.8 s)")
        wl.append(cur)

    if want("silu_f32"):
        n = 512 * 640 * 20 * 15
        cur = Workload("silu_f32", "imex_silu_f32", [n], "hbm", 2.0 * n * 4, "GB/s", "f32",
                       "silu f32 512x640x20x15 uniform(-8,8) seed 20251")
        x = gen_uniform(n, "f32", 20251, -8.0, 8.0)
        cur.args = [dev(x), out(n * 4), n]
        cur.cpu = lambda x=x: (2.0 * x.size * 4 / (orc.time_silu_f32(x, 5, 20) * 1e6),
                             CPU_PROTOCOL % (5, 20) + " (20 instead of the template's 100: a call takes ~0.9 s)")
        wl.append(cur)
    return wl


def measured_traffic():
    """HBM-side bytes per launch from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE
    summary (profiles/hbm_traffic_fetch_write_pmc.txt); {} if it is absent."""
    path = os.path.join(REPO, "profiles", "hbm_traffic_fetch_write_pmc.txt")
    out = {}
    try:
        with open(path) as f:
            for line in f:
                parts = line.split()
                if line.startswith("#") or len(parts) != 8:
                    continue
                out[parts[0]] = int(parts[7])
    except OSError:
        pass
    return out


TRAFFIC = measured_traffic()


def roofline(w, ms):
    if w.bound == "mfma":
        achieved, peak, unit = w.work / (ms * 1e9), MFMA_PEAK_TFLOPS, "TFLOP/s"
    else:
        achieved, peak, unit = w.work / (ms * 1e6), HBM_PEAK_GBS, "GB/s"
    return {"bound": w.bound, "achieved": round(achieved, 3), "peak": peak, "unit": unit,
            "frac": round(achieved / peak, 4), "traffic": TRAFFIC.get(w.name),
            "traffic_source": "profiles/hbm_traffic_fetch_write_pmc.txt (rocprofv3 FETCH_SIZE / WRITE_SIZE, not measured in this run)"
            if w.name in TRAFFIC else None}


def measure_secondary(stream, w, rounds):
    """Back-to-back launches (one event pair around all of them) and the
    IMEX-profiler protocol with a cache flush before each timed launch."""
    # MFMA-bound kernels get a long warm-up: coming from lighter work the part needs
    # ~100 launches before its clock settles under the new load
    warm = 150 if w.bound == "mfma" else 20
    hot_total = stream.profile(w.kernel, w.dims, w.args, warmups=warm, rounds=rounds, mode=1)[0]
    hot_ms = hot_total / rounds
    cold = stream.profile(w.kernel, w.dims, w.args, warmups=2, rounds=min(rounds, 20), flush_bytes=FLUSH_BYTES, mode=0)
    cold_ms = float(np.median(cold))
    return hot_ms, cold_ms


def measure_rotating(host, stream, w, passes):
    """Back-to-back launches that walk a ring of separate copies of the workload's
    buffers, together larger than every cache level (>= 2 GiB against 32 MiB of L2
    and 256 MiB of Infinity Cache): each launch reads and writes memory that no
    cache still holds, and nothing but the kernel's own earlier outputs is being
    written back meanwhile.  The steady state of a streaming pipeline, and the
    figure to hold against the HBM roofline."""
    footprint = sum(b for b, _ in w.sizes.values())
    copies = max(2, min(24, -(-(2 << 30) // footprint)))
    sets, extra = [], []
    for _ in range(copies):
        args = []
        for a in w.args:
            if isinstance(a, host.Ptr) and int(a) in w.sizes:
                nbytes, is_input = w.sizes[int(a)]
                p = stream.alloc(nbytes)
                if is_input:
                    stream.copy(p, a, nbytes)
                extra.append(p)
                args.append(p)
            else:
                args.append(a)
        sets.append(stream.prepare(w.kernel, w.dims, args))
    # one untimed walk round the ring; MFMA-bound kernels walk it until ~150 launches have gone by, as in
    # measure_secondary: coming from the allocations and copies above the part needs that long to settle
    for _ in range(-(-150 // copies) if w.bound == "mfma" else 1):
        for step in sets:
            step()
    stream.wait()
    ev0 = stream.timestamp()
    for _ in range(passes):
        for step in sets:
            step()
    ev1 = stream.timestamp()
    stream.wait()
    ms = stream.elapsed_ms(ev0, ev1) / (passes * copies)
    for p in extra:
        stream.free(p)
    return ms, copies


def measure_split_k(stream, host):
    """out = bf16(silu(A.B + bias)) through the plain kernel and through the K-splitting operator entry
    (imexHipGemmBiasSiluBf16SplitK of libimex-hip-ops.so), same buffers back to back: ms per launch for the MLP
    shape (many tiles: the plain kernel is the faster one) and for shapes with few tiles and a deep K loop (where
    splitting K is what fills the chip).  Zero-filled operands: this compares schedules, not clocks."""
    ops = host.ops()
    if ops.imexHipOpsInit(stream.handle) != 0:
        raise RuntimeError("imexHipOpsInit: %s" % ops.imexHipOpsLastError().decode())
    out = {}
    for M, N, K in ((4096, 11008, 4096), (2048, 2048, 4096), (1024, 1024, 8192), (512, 512, 16384)):
        a, b, bias, o = stream.alloc(M * K * 2), stream.alloc(K * N * 2), stream.alloc(N * 4), stream.alloc(M * N * 2)
        for ptr, n in ((a, M * K // 2), (b, K * N // 2), (bias, N)):
            stream.memset(ptr, 0, n, bits=32)
        plain = stream.profile("imex_gemm_bf16_bias_silu_bf16", [M, N, K], [a, b, bias, o, M, N, K],
                               warmups=50, rounds=200, mode=1)[0] / 200

        def split():
            if ops.imexHipGemmBiasSiluBf16SplitK(stream.handle, int(a), int(b), int(bias), int(o), M, N, K) != 0:
                raise RuntimeError(ops.imexHipOpsLastError().decode())
        for _ in range(50):
            split()
        stream.wait()
        ev0 = stream.timestamp()
        for _ in range(200):
            split()
        ev1 = stream.timestamp()
        stream.wait()
        out["%dx%dx%d" % (M, N, K)] = {"plain_ms": round(plain, 5), "split_k_ms": round(stream.elapsed_ms(ev0, ev1) / 200, 5)}
        for ptr in (a, b, bias, o):
            stream.free(ptr)
    return out


def measure_tile_rounds(stream):
    """imex_gemm_bf16_bias_silu_bf16 with M = K = 4096 at N = 2048 .. 16384: half a round, whole rounds and the MLP
    shape's 2.69 rounds of 256 tiles on the 256 CUs, random operands (numpy generator, seed 5), same buffers back to
    back: what the last, partial round of tiles costs against whole ones."""
    rng = np.random.default_rng(5)

    def bf16(x):
        return (x.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    M = K = 4096
    a = stream.to_device(bf16(rng.standard_normal((M, K), np.float32)))
    out = {}
    for N in (2048, 4096, 8192, 11008, 12288, 16384):
        b = stream.to_device(bf16(rng.standard_normal((K, N), np.float32) * 0.02))
        bias = stream.to_device((rng.standard_normal(N) * 0.1).astype(np.float32))
        o = stream.alloc(M * N * 2)
        ms = stream.profile("imex_gemm_bf16_bias_silu_bf16", [M, N, K], [a, b, bias, o, M, N, K],
                            warmups=200, rounds=300, mode=1)[0] / 300
        out["N=%d" % N] = {"tiles": (M // 256) * -(-N // 256), "ms": round(ms, 5)}
        for ptr in (b, bias, o):
            stream.free(ptr)
    stream.free(a)
    return out


def measure_reference_suite(stream):
    """Every shape and dtype the reference's benchmark suite instantiates (README.md:330-335, benchmarks/*/
    *.shapes.in, *.dtypes.in) plus the two fused chains at their size (512x1024): microseconds per launch over 200
    back-to-back launches on zero-filled buffers.  Most of them are launch-bound (2.5-4 us)."""
    out = {}

    def run(label, kernel, dims, sizes, scalars):
        ptrs = [stream.alloc(n) for n in sizes]
        ms = stream.profile(kernel, dims, ptrs + scalars, warmups=20, rounds=200, mode=1)[0] / 200
        for p in ptrs:
            stream.free(p)
        out[label] = round(ms * 1e3, 2)

    width = {"f32": 4, "f16": 2, "bf16": 2}
    for shape in ((1, 160, 160, 120), (50, 640, 20, 15), (512, 640, 20, 15)):
        n = int(np.prod(shape))
        for dt, w in width.items():
            run("relu_%s_%s" % (dt, "x".join(map(str, shape))), "imex_relu_" + dt, [n], [n * w, n * w], [n])
    for shape in ((1, 1024, 40, 30), (50, 20, 3072), (512, 640, 20, 15)):
        n = int(np.prod(shape))
        for dt in ("f32", "f16"):
            run("silu_%s_%s" % (dt, "x".join(map(str, shape))), "imex_silu_" + dt, [n], [n * width[dt]] * 2, [n])
    for rows in (1, 16, 64, 256, 1024):
        for dt, w in width.items():
            n = rows * 2000
            run("softmax_%s_%dx2000" % (dt, rows), "imex_softmax_" + dt, [rows, 2000], [n * w, n * w], [rows, 2000])
    for r, c in ((128, 136), (1024, 1024)):
        for bits in (32, 16):
            n = r * c * bits // 8
            run("transpose_b%d_%dx%d" % (bits, r, c), "imex_transpose2d_b%d" % bits, [r, c], [n, n], [r, c])
    for d in ((16, 96, 96), (96, 7, 96)):
        for bits in (32, 16):
            n = d[0] * d[1] * d[2] * bits // 8
            run("transpose_b%d_%dx%dx%d" % ((bits,) + d), "imex_transpose3d_b%d" % bits, list(d), [n, n], list(d))
    inner = 16 * 512 * 512
    for dt, w in width.items():
        run("reduce_%s_32x16x512x512" % dt, "imex_reduce_outer_" + dt, [32, inner], [32 * inner * w, inner * w],
            [32, inner, 0.0])
    for dt, w in width.items():
        n = 512 * 1024
        run("loop_fusion_%s_512x1024" % dt, "imex_loop_fusion_" + dt, [n], [n * w] * 3, [n])
        run("input_fusion_%s_512x1024" % dt, "imex_input_fusion_" + dt, [512, 1024], [n * w, n * w, 1024 * w], [512, 1024])
    return out


def vendor_yardstick():
    """The vendor library's f16 4096^3 GEMM on the headline's operands (same seeds, same distribution), timed
    the way the headline is: settle launches, then 1000 launches between two events.  torch.mm dispatches to
    hipBLASLt / rocBLAS; nothing in the product uses either.  What the part sustains on these operand values
    under a tuned library is the scale the headline's fraction of the 2.5 PFLOP/s peak has to be read on."""
    import torch
    M = N = K = 4096
    a = torch.from_numpy(gen_uniform(M * K, "f16", 20246, -1.0, 1.0).view(np.float16).reshape(M, K)).cuda()
    b = torch.from_numpy(gen_uniform(K * N, "f16", 20247, -1.0, 1.0).view(np.float16).reshape(K, N)).cuda()
    results = {}
    for label, make in (("f16_out", lambda x, y: torch.mm(x, y)),
                        ("f32_out", lambda x, y: torch.mm(x, y, out_dtype=torch.float32))):
        for operands, (x, y) in (("uniform", (a, b)), ("zeros", (torch.zeros_like(a), torch.zeros_like(b)))):
            try:
                for _ in range(SETTLE_LAUNCHES):
                    make(x, y)
                torch.cuda.synchronize()
                start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                for _ in range(1000):
                    make(x, y)
                stop.record()
                torch.cuda.synchronize()
                ms = start.elapsed_time(stop) / 1000
                results["%s_%s" % (label, operands)] = {"ms_per_launch": round(ms, 5),
                                                        "tflops": round(2.0 * M * N * K / ms / 1e9, 1),
                                                        "frac_of_2.5_pflops": round(2.0 * M * N * K / ms / 1e9 / 2500.0, 4)}
            except (RuntimeError, TypeError) as e:  # e.g. a torch build whose mm takes no out_dtype
                results["%s_%s" % (label, operands)] = {"error": str(e).splitlines()[0][:200]}
            log("vendor GEMM %s, %s operands: %s" % (label, operands, results["%s_%s" % (label, operands)]))
    # The MLP-shaped configuration: the library's bf16 GEMM alone (bf16 output, no bias, no activation), and with
    # the bias add and SiLU as the framework's separate kernels after it.
    Mm, Km, Nm = 4096, 4096, 11008
    am = torch.from_numpy(gen_normal(Mm * Km, "bf16", 20248, 0.0, 1.0).view(np.int16).reshape(Mm, Km)).cuda().view(torch.bfloat16)
    bm = torch.from_numpy(gen_normal(Km * Nm, "bf16", 20249, 0.0, 0.02).view(np.int16).reshape(Km, Nm)).cuda().view(torch.bfloat16)
    biasm = torch.from_numpy(gen_normal(Nm, "f32", 20250, 0.0, 0.1)).cuda()
    for label, make in (("mlp_bf16_gemm_only", lambda: torch.mm(am, bm)),
                        ("mlp_bf16_gemm_bias_silu_unfused",
                         lambda: torch.nn.functional.silu(torch.mm(am, bm).float() + biasm).to(torch.bfloat16))):
        try:
            for _ in range(50):
                make()
            torch.cuda.synchronize()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(200):
                make()
            stop.record()
            torch.cuda.synchronize()
            ms = start.elapsed_time(stop) / 200
            results[label] = {"ms_per_launch": round(ms, 5), "tflops": round(2.0 * Mm * Nm * Km / ms / 1e9, 1),
                              "frac_of_2.5_pflops": round(2.0 * Mm * Nm * Km / ms / 1e9 / 2500.0, 4)}
        except (RuntimeError, TypeError) as e:
            results[label] = {"error": str(e).splitlines()[0][:200]}
        log("vendor %s: %s" % (label, results[label]))
    del am, bm

    # Flash-attention forward, head dimension 64, f16, no mask: the framework's fused attention.
    for label, (z, h, n_ctx) in (("attention_f16_2x2x4096x64", (2, 2, 4096)), ("attention_f16_16x4096x64", (1, 16, 4096))):
        try:
            q, k, v = (torch.randn((z, h, n_ctx, 64), device="cuda", dtype=torch.float32).to(torch.float16) for _ in range(3))
            for _ in range(50):
                torch.nn.functional.scaled_dot_product_attention(q, k, v)
            torch.cuda.synchronize()
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(300):
                torch.nn.functional.scaled_dot_product_attention(q, k, v)
            stop.record()
            torch.cuda.synchronize()
            ms = start.elapsed_time(stop) / 300
            flop = 4.0 * z * h * n_ctx * n_ctx * 64
            results[label] = {"ms_per_launch": round(ms, 5), "tflops": round(flop / ms / 1e9, 1),
                              "frac_of_2.5_pflops": round(flop / ms / 1e9 / 2500.0, 4)}
        except (RuntimeError, TypeError) as e:
            results[label] = {"error": str(e).splitlines()[0][:200]}
        log("vendor %s: %s" % (label, results[label]))

    # The memory-bound configurations through the same library's own kernels, on the rotating protocol (a ring
    # of separate tensor sets of at least 2 GiB, every result written into a preallocated tensor of its set).
    def rotating(make_set, op, algorithmic_bytes, set_bytes):
        sets = [make_set() for _ in range(max(2, -(-(2 << 30) // set_bytes)))]
        for st in sets:
            op(*st)
        torch.cuda.synchronize()
        passes = max(2, 200 // len(sets))
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(passes):
            for st in sets:
                op(*st)
        stop.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(stop) / (passes * len(sets))
        return {"ms_per_launch": round(ms, 5), "frac_of_8_TBps": round(algorithmic_bytes / ms / 1e6 / 8000.0, 4)}

    def randn(shape, dtype):
        return torch.randn(shape, device="cuda", dtype=torch.float32).to(dtype)

    streaming = {}
    cases = (
        ("relu_f32_4096x4096", lambda: (randn((4096, 4096), torch.float32), torch.empty((4096, 4096), device="cuda")),
         lambda x, y: torch.clamp_min(x, 0.0, out=y), 2 * 4096 * 4096 * 4, 2 * 4096 * 4096 * 4),
        ("softmax_f16_16384x1024",
         lambda: (randn((16384, 1024), torch.float16), torch.empty((16384, 1024), device="cuda", dtype=torch.float16)),
         lambda x, y: torch.softmax(x, 1, out=y), 2 * 16384 * 1024 * 2, 2 * 16384 * 1024 * 2),
        ("rowsum_f32_8192x8192", lambda: (randn((8192, 8192), torch.float32), torch.empty((8192,), device="cuda")),
         lambda x, y: torch.sum(x, 1, out=y), 8192 * 8192 * 4 + 8192 * 4, 8192 * 8192 * 4),
        ("transpose_bf16_8192x8192",
         lambda: (randn((8192, 8192), torch.bfloat16), torch.empty((8192, 8192), device="cuda", dtype=torch.bfloat16)),
         lambda x, y: y.copy_(x.t()), 2 * 8192 * 8192 * 2, 2 * 8192 * 8192 * 2),
        ("transpose_f32_4096x4096",
         lambda: (randn((4096, 4096), torch.float32), torch.empty((4096, 4096), device="cuda")),
         lambda x, y: y.copy_(x.t()), 2 * 4096 * 4096 * 4, 2 * 4096 * 4096 * 4),
        ("silu_f32_512x640x20x15",
         lambda: (randn((98304000,), torch.float32), torch.empty((98304000,), device="cuda")),
         lambda x, y: torch.ops.aten.silu.out(x, out=y), 2 * 98304000 * 4, 2 * 98304000 * 4),
    )
    for name, make_set, op, algorithmic, set_bytes in cases:
        try:
            streaming[name] = rotating(make_set, op, algorithmic, set_bytes)
        except (RuntimeError, TypeError) as e:
            streaming[name] = {"error": str(e).splitlines()[0][:200]}
        torch.cuda.empty_cache()
        log("vendor %s: %s" % (name, streaming[name]))
    print(json.dumps({"vendor_gemm_f16_4096": results, "vendor_streaming_rotating": streaming,
                      "library": "torch %s (mm, clamp_min, softmax, sum, copy_ of a transposed view, silu)" % torch.__version__,
                      "protocol": "GEMM: %d settle launches, then 1000 launches between two events; streaming: a ring of "
                                  "tensor sets of at least 2 GiB, one settle pass, then about 200 launches between two events"
                                  % SETTLE_LAUNCHES}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--only", type=str, default=None, help="comma-separated workload names")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline legs")
    ap.add_argument("--suite", action="store_true",
                    help="also time every shape of the reference's benchmark suite (us per launch, back to back)")
    ap.add_argument("--vendor-yardstick", action="store_true",
                    help="time the vendor GEMM library (through torch.mm) on the headline's operands and exit: "
                         "a yardstick printed as its own JSON line, never part of `value`")
    args = ap.parse_args()
    if args.vendor_yardstick:
        vendor_yardstick()
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: every kernel here runs on a single MI355X and this build has no "
              "multi-GPU path (--gpus %d refused)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    only = set(args.only.split(",")) if args.only else None
    if only is not None:
        only.add("gemm_f16_4096")

    pkg = entry.load_package()
    host = pkg.host
    orc = None if args.no_cpu else entry.load_oracle()  # the oracle only ever runs as the CPU baseline
    host.runtime()
    host.kernels()  # raises if the HIP libraries are not built: there is no fallback

    t_setup = time.time()
    stream = host.Stream()
    info = stream.device_info()
    log("device: %s, %d CUs @ %.0f MHz" % (info["name"], info["cus"], info["clock_khz"] / 1e3))
    workloads = build_workloads(host, orc, stream, only)
    log("inputs generated and resident in HBM after %.1f s" % (time.time() - t_setup))

    # Host -> device copy rate through gpuMemCopy (pageable host memory), for the
    # PCIe-inclusive figure quoted in the design notes; never part of `value`.
    probe = np.zeros(64 << 20, np.uint8)
    d_probe = stream.alloc(probe.nbytes)
    stream.copy(d_probe, probe.ctypes.data, probe.nbytes)
    t = time.perf_counter()
    stream.copy(d_probe, probe.ctypes.data, probe.nbytes)
    h2d_gbs = probe.nbytes / (time.perf_counter() - t) / 1e9
    stream.free(d_probe)
    log("gpuMemCopy host->device: %.1f GB/s" % h2d_gbs)

    # A streaming kernel on `host_shared` allocations (gpuMemAlloc with isShared: pinned host memory the
    # GPU reads and writes over the host link): the rate a pipeline gets when it leaves its tensors in
    # the buffers IMEX's insert-gpu-allocs pass marks host_shared instead of copying them to the device.
    n_sh = 4096 * 4096
    sh_in, sh_out = stream.alloc(n_sh * 4, shared=True), stream.alloc(n_sh * 4, shared=True)
    sh_ms = stream.profile("imex_relu_f32", [n_sh], [sh_in, sh_out, n_sh], warmups=1, rounds=3, mode=1)[0] / 3
    shared_gbs = 2.0 * n_sh * 4 / (sh_ms * 1e6)
    stream.free(sh_in)
    stream.free(sh_out)
    log("imex_relu_f32 on host_shared buffers: %.1f GB/s" % shared_gbs)

    # The secondary workloads run first.  Coming from idle or from lighter work, the first ~100 GEMM
    # launches run ~10% slower while the power controller settles, which a short timed region would
    # mostly measure: the headline loop below therefore starts with SETTLE_LAUNCHES untimed launches,
    # whatever --warmup says.
    per = []
    secondary = sorted(workloads[1:], key=lambda w: w.bound == "mfma")  # the other GEMM goes last
    for w in secondary:
        hot_ms, cold_ms = measure_secondary(stream, w, rounds=50 if w.bound == "mfma" else 200)
        rot_ms, copies = measure_rotating(host, stream, w, passes=max(2, 200 // 24))
        if w is not secondary[-1]:
            # A hot loop started right after the ring's ~2 GiB are freed measures 6-10 % low, whichever
            # workload it belongs to; a pause removes most of that.  Not after the last one: the headline
            # kernel follows with its own settle phase and must not find the device idle.
            time.sleep(1.5)
        # `roofline` is the rotating figure: every launch streams its tensors from HBM.  Back-to-back launches
        # on one buffer pair are served in part by the 256 MiB Infinity Cache (`roofline_cache_resident`, not an
        # HBM fraction); `roofline_cache_flushed` is the reference profiler's protocol, which also times an
        # event pair per launch and the write-back of the flush's dirty lines.
        rf = roofline(w, rot_ms)
        entry_ = {"name": w.name, "workload": w.describe, "kernel": w.kernel, "dtype": w.dtype,
                  "ms_per_launch": round(rot_ms, 5), "rotating_buffer_sets": copies,
                  "ms_per_launch_cache_resident": round(hot_ms, 5), "ms_per_launch_cache_flushed": round(cold_ms, 5),
                  "roofline": rf, "roofline_protocol": "rotating: back-to-back launches over %d separate buffer sets (>= 2 GiB)" % copies,
                  "roofline_cache_flushed": roofline(w, cold_ms),
                  "roofline_cache_resident": roofline(w, hot_ms),
                  # the protocol the reference's own profiler defines (IMEX_ENABLE_CACHE_FLUSHING): one
                  # isolated launch per sample after a cache flush
                  "contract_protocol": "cache_flushed", "contract_frac": roofline(w, cold_ms)["frac"]}
        log("%s: rotating over %d buffer sets %.4f ms (%.1f %s, %.1f%% of peak); cache-flushed %.4f ms (%.1f%%); "
            "same buffers back to back %.4f ms (%.1f%%)" % (
                w.name, copies, rot_ms, rf["achieved"], rf["unit"], 100 * rf["frac"], cold_ms,
                100 * entry_["roofline_cache_flushed"]["frac"], hot_ms, 100 * entry_["roofline_cache_resident"]["frac"]))
        per.append(entry_)

    head = workloads[0]
    K, W = args.steps, args.warmup
    step = stream.prepare(head.kernel, head.dims, head.args)
    # First the caller's protocol to the letter -- W warm-ups, K timed steps, straight from whatever the
    # device was doing before -- reported as `value_without_settle`; then the settle phase and the same
    # again, which is `value`.
    for _ in range(W):
        step()
    stream.wait()
    t0 = time.perf_counter()
    for _ in range(K):
        step()
    stream.wait()
    unsettled_ms = (time.perf_counter() - t0) * 1e3 / K
    for _ in range(SETTLE_LAUNCHES):
        step()
    for _ in range(W):
        step()
    stream.wait()
    t0 = time.perf_counter()
    ev0 = stream.timestamp()  # HIP events on the launch stream bracket exactly the K timed launches
    for _ in range(K):
        step()
    ev1 = stream.timestamp()
    stream.wait()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3 / K
    event_ms = stream.elapsed_ms(ev0, ev1) / K
    # device-side duration of a launch: back-to-back launches from C, no Python in the loop
    b2b = max(K, 200)
    kernel_ms = stream.profile(head.kernel, head.dims, head.args, warmups=20, rounds=b2b, mode=1)[0] / b2b
    log("%s: wall %.4f ms/step, events %.4f ms/step, back-to-back %.4f ms/launch" % (head.name, wall_ms, event_ms, kernel_ms))
    value = head.work / (wall_ms * 1e9)

    # What the matrix pipe sustains on this kind of operand data with nothing else going on
    # (imex_mfma_lds_ceiling_f16 in lib/imex_probe.hsaco: MFMA 16x16x32 fed from LDS, no global traffic),
    # measured right after the headline loop so the part is in the same thermal / power state.
    ceiling = {}
    groups, iters = info["cus"], 2048
    d_sink = stream.alloc(groups * 512 * 4)
    probe_fn = stream.kernel_from_file(host.PROBE_CODE_OBJECT, "imex_mfma_lds_ceiling_f16")
    reg_ceiling = {}
    for label, mode in (("f16_uniform_pm1", 0), ("zeros", 1), ("f16_every_exponent", 2)):
        for into, m in ((ceiling, mode), (reg_ceiling, mode + 4)):  # + 4: operands held in registers, no LDS reads
            ms = stream.profile_function(probe_fn, (groups, 1, 1), (512, 1, 1), [d_sink, groups * 512, iters, m],
                                         warmups=100, rounds=200)
            into[label] = round(groups * 8.0 * iters * 32 * 16384 / (ms * 1e9), 1)
    stream.free(d_sink)
    log("MFMA-from-LDS loop: %.0f TFLOP/s on f16 uniform in (-1,1), %.0f on zeros, %.0f with every exponent equally likely; "
        "operands held in registers: %.0f / %.0f / %.0f" % (
            ceiling["f16_uniform_pm1"], ceiling["zeros"], ceiling["f16_every_exponent"],
            reg_ceiling["f16_uniform_pm1"], reg_ceiling["zeros"], reg_ceiling["f16_every_exponent"]))

    result = {
        "metric": METRIC, "value": round(value, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": K,
        # untimed launches of the headline kernel in front of the timed steps: the settle phase and the caller's W
        "warmup": SETTLE_LAUNCHES + W, "warmup_requested": W,
        "value_without_settle": round(head.work / (unsettled_ms * 1e9), 3),
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic (seeded std::mt19937 stream, inputs resident in HBM)",
        "config": {"workload": "BASELINE.json configs[3]: " + head.describe, "kernel": head.kernel,
                   "launch": "grid (256,1,1) x block (512,1,1)", "device": info["name"],
                   "cus": info["cus"], "clock_mhz": info["clock_khz"] / 1e3,
                   "gpuMemCopy_h2d_GBps": round(h2d_gbs, 1),
                   "relu_f32_on_host_shared_buffers_GBps": round(shared_gbs, 1)},
        # `achieved` prices the launch at its HIP-event duration over the timed region
        "roofline": dict(roofline(head, event_ms), event_ms_per_step=round(event_ms, 5),
                         back_to_back_ms=round(kernel_ms, 5)),
        "settle_launches": SETTLE_LAUNCHES,
        # context for `roofline`, not a replacement for its published peak: TFLOP/s of a loop of
        # nothing but MFMA 16x16x32 + LDS operand reads on f16 uniform in (-1,1), on zeros, and on
        # f16 with random mantissas and every exponent below 1.0 equally likely
        "mfma_lds_ceiling_tflops": ceiling,
        # the same loop with its twelve operand fragments held in registers: what the matrix pipe sustains on
        # these values with no LDS traffic at all
        "mfma_register_fed_tflops": reg_ceiling,
    }

    if not args.no_cpu and head.cpu:
        t = time.time()
        v, sample = head.cpu()
        result["cpu_baseline"] = {"value": round(v, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                                  "sample": sample, "host_cores": os.cpu_count()}
        log("cpu baseline %s: %.4f GFLOP/s (%.1f s)" % (head.name, v * 1e3, time.time() - t))

    for w, entry_ in zip(secondary, per):
        if not args.no_cpu and w.cpu:
            t = time.time()
            v, sample = w.cpu()
            entry_["cpu_baseline"] = {"value": round(v, 6), "unit": w.unit, "cores": 1, "kind": "port", "sample": sample}
            log("cpu baseline %s: %.4f %s (%.1f s)" % (w.name, v, w.unit, time.time() - t))
    result["per_config"] = per
    if args.suite:
        result["reference_suite_us_per_launch"] = measure_reference_suite(stream)
        log("reference benchmark suite: %d shapes timed" % len(result["reference_suite_us_per_launch"]))
        result["gemm_bias_silu_split_k_ms_per_launch_MxNxK"] = measure_split_k(stream, host)
        log("split-K operator entry against the plain kernel: %s" % result["gemm_bias_silu_split_k_ms_per_launch_MxNxK"])
        result["gemm_bias_silu_ms_by_rounds_of_tiles"] = measure_tile_rounds(stream)
        log("MLP kernel by rounds of tiles: %s" % result["gemm_bias_silu_ms_by_rounds_of_tiles"])

    for w in workloads:
        for p in w.buffers:
            stream.free(p)
    stream.close()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
