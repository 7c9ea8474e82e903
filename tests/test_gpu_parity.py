"""GPU parity tests: every kernel, called through the gpu* C ABI, against the CPU
oracle on the same seeded inputs; reference golden vectors; size-independent
properties at the full benchmark shapes.

Bars: bit-exact for relu / transpose / reduce_outer / integer GEMM; <= 1 ulp for
SiLU (f32); |d| <= 1e-3 |ref| + 2^-24 for f16 softmax (2^-24 = one f16 subnormal
step, the output type's absolute resolution) and 1e-3 relative for row sums;
max|d| <= 5e-3 max|ref| for the GEMMs.
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_vectors.json")) as f:
    GOLD = json.load(f)


def arr(v, shape=None):
    a = np.asarray(v, np.float32)
    return a.reshape(shape) if shape else a


def say(msg):
    print("[case] " + msg, flush=True)


# =============================== ReLU =====================================
def test_relu_golden_and_specials(host, orc, stream):
    g = GOLD["relu_f32_4x5_spirv"]
    assert np.array_equal(host.relu(stream, arr(g["input"], g["shape"])), arr(g["expected"], g["shape"]))
    x = np.array([0x7fc00001, 0xffc12345, 0x80000000, 0, 1, 0x80000001, 0x7f800000, 0xff800000, 0x7f800001],
                 np.uint32).view(np.float32)
    assert np.array_equal(host.relu(stream, x).view(np.uint32), orc.relu_f32(x).view(np.uint32))


@pytest.mark.parametrize("n", [1, 3, 4095, 4096, 4097, 100003, 1 << 20])
def test_relu_ragged_sizes(host, orc, stream, n):
    say("relu n=%d" % n)
    x = orc.fill_uniform(n, "f32", 20241 + n % 7, -1.0, 1.0)
    assert np.array_equal(host.relu(stream, x).view(np.uint32), orc.relu_f32(x).view(np.uint32))


def test_relu_config_4096x4096(host, orc, stream):
    x = orc.fill_uniform(4096 * 4096, "f32", 20241, -1.0, 1.0).reshape(4096, 4096)
    assert np.array_equal(host.relu(stream, x).view(np.uint32), orc.relu_f32(x).view(np.uint32))


def test_relu_every_f32_pattern(host, stream):
    """All 2^32 bit patterns against the closed form (x if x > 0 or NaN else +0)."""
    chunk = 1 << 27
    for base in range(0, 1 << 32, chunk):
        if base % (1 << 30) == 0:
            say("relu sweep base=0x%08x" % base)
        u = np.arange(base, base + chunk, dtype=np.uint32)
        got = host.relu(stream, u.view(np.float32)).view(np.uint32)
        keep = (u.view(np.int32) > 0) | (u > np.uint32(0xff800000))
        assert np.array_equal(got, np.where(keep, u, np.uint32(0)))


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_relu_every_16bit_pattern(host, orc, stream, dtype):
    x = np.tile(np.arange(65536, dtype=np.uint16), 3)[:-5]  # unaligned tail
    assert np.array_equal(host.relu(stream, x, dtype), orc.relu_16(x, dtype))


# =============================== SiLU =====================================
def test_silu_within_one_ulp(host, orc, stream):
    x = np.concatenate([
        orc.fill_uniform(1 << 20, "f32", 20251, -8.0, 8.0),
        orc.fill_uniform(1 << 18, "f32", 1, -110.0, 110.0),
        orc.fill_bits(1 << 18, "f32", 2).view(np.float32),
        np.array([0.0, -0.0, 1.3, np.inf, -np.inf, 88.0, -88.0, 88.72, 88.73, -103.9, -104.0, 1e-45, -1e-45, 1e38,
                  -1e38], np.float32),
        np.array([0x7fc00000], np.uint32).view(np.float32)])
    got, ref = host.silu(stream, x), orc.silu_f32(x)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan)
    d = orc.ulp_distance_f32(got[~nan], ref[~nan])
    say("silu max ulp distance %d, exact %d of %d" % (d.max(), int((d == 0).sum()), d.size))
    assert d.max() <= 1
    assert host.silu(stream, np.array([0.0], np.float32))[0] == 0.0


def test_silu_same_bits_as_the_oracle_on_ordinary_inputs(host, orc, stream):
    """|x| < 64 takes the kernel's straight-line form (exp without its special cases, the reciprocal
    as an explicit refinement sequence): the same bits as libm's expf and an IEEE division, on every
    f32 in [1, 2) (2^23 consecutive values) and on 8 Mi values spread over (-64, 64)."""
    sweep = np.arange(0x3f800000, 0x40000000, dtype=np.uint32).view(np.float32)
    spread = orc.fill_uniform(1 << 23, "f32", 77, -63.99, 63.99)
    for name, x in (("every f32 in [1,2)", sweep), ("-every f32 in [1,2)", -sweep), ("uniform(-64,64)", spread)):
        say("silu bit-exact: " + name)
        assert np.array_equal(host.silu(stream, x).view(np.uint32), orc.silu_f32(x).view(np.uint32)), name


def test_silu_benchmark_shape(host, orc, stream):
    x = orc.fill_uniform(512 * 640 * 20 * 15, "f32", 20251, -8.0, 8.0)
    got, ref = host.silu(stream, x), orc.silu_f32(x)
    assert orc.ulp_distance_f32(got, ref).max() <= 1


# ============================ exp, maximum ================================
def test_exp_same_bits_as_libm(host, orc, stream):
    """WG/math_exp.mlir: math.exp against the CPU loop's libm call -- the test's own input range
    (-0.5, 0.5), the whole finite range, and the special values."""
    for name, x in (("reference range", orc.fill_uniform(256 * 256, "f32", 31, -0.5, 0.5)),
                    ("(-110, 110)", orc.fill_uniform(1 << 21, "f32", 32, -110.0, 110.0)),
                    ("(-64, 64) ragged", orc.fill_uniform((1 << 20) + 13, "f32", 33, -63.9, 63.9))):
        say("exp: " + name)
        assert np.array_equal(host.exp(stream, x).view(np.uint32), orc.expf_n(x).view(np.uint32)), name
    special = np.array([0.0, -0.0, np.inf, -np.inf, 88.72, 88.73, -103.9, -104.0, 1e-45, -1e-45, 1e38, -1e38, 64.0, -64.0],
                       np.float32)
    assert np.array_equal(host.exp(stream, special).view(np.uint32), orc.expf_n(special).view(np.uint32))
    assert np.isnan(host.exp(stream, np.array([np.nan], np.float32))[0])


def test_maximum_matches_the_oracle(host, orc, stream):
    """WG/arith_maximumf.mlir: bit for bit where no operand is NaN, NaN where one is."""
    a, b = orc.fill_uniform(256 * 256, "f32", 41, -0.5, 0.5), orc.fill_uniform(256 * 256, "f32", 42, -0.5, 0.5)
    assert np.array_equal(host.maximum(stream, a, b), np.maximum(a, b))
    n = (1 << 20) + 7
    a, b = orc.fill_bits(n, "f32", 43).view(np.float32).copy(), orc.fill_bits(n, "f32", 44).view(np.float32).copy()
    a[:8] = [0.0, -0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, np.nan]
    b[:8] = [-0.0, 0.0, -0.0, 1.0, -1.0, 1.0, np.nan, np.nan]
    got, ref = host.maximum(stream, a, b), orc.maximum_f32(a, b)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(got), nan) and nan[5] and nan[6] and nan[7]
    assert np.array_equal(got[~nan].view(np.uint32), ref[~nan].view(np.uint32))


# =============================== Softmax ==================================
def close_16(orc, got_bits, ref_bits, dtype):
    got, ref = orc.to_float(got_bits, dtype), orc.to_float(ref_bits, dtype)
    quantum = 2.0 ** -24 if dtype == "f16" else 0.0
    rtol = 1e-3 if dtype == "f16" else 2.0 ** -7  # bf16: one unit in the last place
    return np.all(np.abs(got - ref) <= rtol * np.abs(ref) + quantum)


@pytest.mark.parametrize("key", ["softmax_f32_10x20", "softmax_f32_10x20_spirv"])
def test_softmax_golden(host, orc, stream, key):
    g = GOLD[key]
    got = host.softmax(stream, arr(g["input"], g["shape"]), "f32")
    want = arr(g["expected"], g["shape"])
    assert np.max(np.abs(got - want) / want) < 2e-5
    assert orc.allclose_f32(got, want)


def test_softmax_config_f16_16384x1024(host, orc, stream):
    x = orc.fill_normal(16384 * 1024, "f16", 20242, 0.0, 2.0).reshape(16384, 1024)
    got, ref = host.softmax(stream, x, "f16"), orc.softmax_16(x, "f16")
    assert close_16(orc, got, ref, "f16")
    assert orc.allclose_f32(orc.half_to_float(got), orc.softmax_f32(orc.half_to_float(x)))
    sums = orc.half_to_float(got).sum(axis=1, dtype=np.float64)
    assert np.max(np.abs(sums - 1.0)) < 2e-3  # 1024 outputs each rounded to f16


@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 7), (5, 8), (16, 2000), (64, 2000), (7, 1000), (9, 512), (4, 4096),
                                       (3, 5000), (2, 65536 + 8), (1025, 64), (6, 1016),
                                       (16385, 24), (20001, 8)])  # two rows per wavefront, odd row counts
@pytest.mark.parametrize("dtype", ["f16", "f32"])
def test_softmax_shapes(host, orc, stream, rows, cols, dtype):
    say("softmax %s %dx%d" % (dtype, rows, cols))
    x = orc.fill_normal(rows * cols, dtype, rows * 131 + cols, 0.0, 2.0).reshape(rows, cols)
    got = host.softmax(stream, x, dtype)
    if dtype == "f32":
        ref = orc.softmax_f32(x)
        assert np.all(np.abs(got - ref) <= 1e-3 * np.abs(ref))
        assert np.max(np.abs(got - ref) / np.maximum(ref, 1e-30)) < 5e-5
    else:
        assert close_16(orc, got, orc.softmax_16(x, "f16"), "f16")


def test_softmax_bf16_and_exact_rows(host, orc, stream):
    x = orc.fill_normal(64 * 1024, "bf16", 9, 0.0, 2.0).reshape(64, 1024)
    assert close_16(orc, host.softmax(stream, x, "bf16"), orc.softmax_16(x, "bf16"), "bf16")
    eq = orc.float_to_half(np.full((8, 1024), 3.3, np.float32))
    assert np.all(host.softmax(stream, eq, "f16") == 0x1400)  # exactly 2^-10
    # a row of -inf-free extremes: one dominant element
    x = np.full((4, 1024), -20.0, np.float32)
    x[:, 5] = 20.0
    got = host.softmax(stream, x, "f32")
    assert np.all(got[:, 5] == 1.0) and got.sum() == 4.0


@pytest.mark.parametrize("rows,cols", [(3, 5000), (2, 65536 + 8), (5, 4097), (2, 300001)])
def test_softmax_long_rows_streaming_form(host, orc, stream, rows, cols):
    """Rows beyond 4096 columns take the running (max, sum) form of WG/softmax_intra_sg_cross_lane.mlir:135-175;
    checked against the reference's scalar three-pass loop (:85-117) and the benchmark form, on random
    rows, on a ramp whose maximum moves with every vector (every partial sum is rescaled again and
    again), on its mirror image, and on one huge element at the very end."""
    say("softmax streaming %dx%d" % (rows, cols))
    x = orc.fill_normal(rows * cols, "f32", 81 + cols % 7, 0.0, 2.0).reshape(rows, cols).copy()
    x[0] = np.linspace(-40.0, 30.0, cols, dtype=np.float32)  # outputs stay normal f32 numbers (the hardware exp flushes subnormal results)
    x[1] = x[0][::-1]
    if rows > 2:
        x[2, -1] = 60.0
    got = host.softmax(stream, x, "f32")
    for ref in (orc.softmax_f32(x, three_pass=True), orc.softmax_f32(x)):
        assert np.all(np.abs(got - ref) <= 1e-3 * np.abs(ref))  # the stated bar
    # the sequential f32 sum of the reference loop carries up to ~2e-4 of rounding over 300 001 addends (it
    # differs by that much between a row and its mirror image); against the exact row sum the kernel is tighter
    assert np.max(np.abs(got.sum(axis=1, dtype=np.float64) - 1.0)) < 2e-5
    xh = orc.from_float(x, "f16")
    assert close_16(orc, host.softmax(stream, xh, "f16"), orc.softmax_16(xh, "f16"), "f16")


@pytest.mark.parametrize("cols,path", [(1024, "registers"), (2000, "lds"), (5000, "streamed")])
def test_softmax_reciprocal_deviation_is_one_rounding(host, orc, stream, cols, path):
    """The kernel multiplies by one reciprocal per row where the reference divides per element.  What that may
    cost, pinned on each of the kernel's three paths: an f16 output is the oracle's divided result or its
    neighbour (one unit in the last place), and all but a small fraction are the same bits."""
    say("softmax reciprocal deviation, %s path, cols=%d" % (path, cols))
    x = orc.fill_normal(64 * cols, "f16", 4242 + cols, 0.0, 2.0).reshape(64, cols)
    got, ref = host.softmax(stream, x, "f16"), orc.softmax_16(x, "f16")
    steps = np.abs(got.astype(np.int32) - ref.astype(np.int32))  # positive f16 bit patterns are ordered like their values
    assert steps.max() <= 1
    assert np.mean(steps == 0) > 0.98


@pytest.mark.parametrize("dtype,cols", [("f32", 20), ("f32", 512), ("f16", 1024), ("f32", 3000), ("f16", 4096),
                                        ("f32", 5000), ("f16", 70000)])
def test_softmax_nan_and_infinite_rows(host, orc, stream, dtype, cols):
    """Rows the benchmark's inputs never hold, on every path of the kernel (registers, LDS, streamed):
    a NaN anywhere makes its whole row NaN (arith.maximumf and the sum both carry it), a row of
    nothing but -inf is 0/0 = NaN because the running maximum starts at -3.40282347e38 rather than
    -inf, +inf in a row gives inf - inf = NaN, and a -inf among finite values is an exact zero."""
    say("softmax special rows %s cols=%d" % (dtype, cols))
    x = orc.to_float(orc.fill_normal(6 * cols, dtype, 71, 0.0, 2.0), dtype).reshape(6, cols).copy()
    x[1, cols // 3] = np.nan
    x[2, :] = -np.inf
    x[3, cols - 1] = np.inf
    x[4, 0] = -np.inf
    x[5, :] = -3.0e38 if dtype == "f32" else -65504.0
    xin = x if dtype == "f32" else orc.from_float(x, dtype)
    got = orc.to_float(host.softmax(stream, xin, dtype), dtype)
    ref = orc.softmax_f32(x) if dtype == "f32" else orc.to_float(orc.softmax_16(xin, dtype), dtype)
    assert np.array_equal(np.isnan(got), np.isnan(ref))
    assert np.isnan(ref[1]).all() and np.isnan(ref[2]).all() and np.isnan(ref[3]).all() and not np.isnan(ref[[0, 4, 5]]).any()
    assert got[4, 0] == 0.0
    ok = ~np.isnan(ref)
    assert np.all(np.abs(got[ok] - ref[ok]) <= 1e-3 * np.abs(ref[ok]) + (2.0 ** -24 if dtype == "f16" else 0.0))


@pytest.mark.parametrize("rows,cols", [(1000, 1024), (1000, 1016), (37, 1024), (4097, 1024), (5, 8)])
def test_softmax_f16_rows_in_registers_any_grid(host, orc, stream, rows, cols):
    """The f16 register path walks its rows with the next row's loads in flight: a wavefront that takes one
    row, two, three (odd and even trip counts of the two-row loop) or a few hundred gives the same bits as
    the catalogue's grid, for whole 1024-column rows and for rows that leave lanes without a vector."""
    say("softmax f16 walk %dx%d" % (rows, cols))
    x = orc.fill_normal(rows * cols, "f16", 7 * rows + cols, 0.0, 2.0).reshape(rows, cols)
    x[rows // 2, cols // 2] = 0x7E00  # a NaN row in the middle of a walk
    ref = orc.softmax_16(x, "f16")
    want = host.softmax(stream, x, "f16")
    nan = np.isnan(orc.half_to_float(ref))
    assert np.array_equal(np.isnan(orc.half_to_float(want)), nan) and nan[rows // 2].all() and nan.sum() == cols
    ok = ~nan
    assert close_16(orc, want[ok], ref[ok], "f16")
    for grid in (1, 2, -(-rows // 12), -(-rows // 8), -(-rows // 4) + 3):
        d_in, d_out = stream.to_device(x), stream.alloc(rows * cols * 2)
        stream.launch("imex_softmax_f16", [rows, cols], [d_in, d_out, rows, cols], grid=(grid, 1, 1))
        stream.wait()
        got = stream.from_device(d_out, (rows, cols), np.uint16)
        stream.free(d_in), stream.free(d_out)
        assert np.array_equal(got[ok], want[ok]) and np.isnan(orc.half_to_float(got[~ok])).all(), grid


# =============================== Reductions ================================
def test_rowsum_golden_and_exact(host, orc, stream):
    g = GOLD["sum_f32_10x20"]
    x = arr(g["input"], g["shape"])
    assert np.array_equal(host.rowsum(stream, x), np.full(10, 210.0, np.float32))
    assert host.rowsum(stream, x.reshape(1, 200))[0] == 2100.0
    g = GOLD["wg_reduction_rows"]
    x = np.repeat(np.arange(8, dtype=np.float32)[:, None], 256, axis=1)
    assert list(host.rowsum(stream, x)) == g["expected"]
    assert host.rowsum(stream, np.ones((1, 65536), np.float32))[0] == 65536.0
    # integer-valued inputs: any summation order is exact
    for rows, cols in [(37, 1000), (5, 8192), (3, 4099), (130, 2048), (2, 2052), (9, 1)]:
        xi = orc.fill_int(rows * cols, "f32", rows + cols, -8, 8).reshape(rows, cols)
        assert np.array_equal(host.rowsum(stream, xi, init=3.0), orc.rowsum_f32(xi, init=3.0)), (rows, cols)


def test_rowsum_config_8192x8192(host, orc, stream):
    x = orc.fill_uniform(8192 * 8192, "f32", 20243, 0.0, 1.0).reshape(8192, 8192)
    got, ref = host.rowsum(stream, x), orc.rowsum_f32(x)
    assert np.max(np.abs(got - ref) / np.abs(ref)) <= 1e-3
    exact = x.sum(axis=1, dtype=np.float64)
    say("rowsum rel err vs f64: kernel %.2e, sequential oracle %.2e" %
        (np.max(np.abs(got - exact) / exact), np.max(np.abs(ref - exact) / exact)))
    assert np.max(np.abs(got - exact) / exact) < 1e-5


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_silu_sixteen_bit(host, orc, stream, dtype):
    """benchmarks/silu/silu.dtypes.in lists f16: widen, the f32 chain, one rounding -- same bits as the oracle.
    Every 16-bit pattern once (NaNs compared as NaNs), then the benchmark's 1x1024x40x30 and a large ragged size."""
    every = np.arange(65536, dtype=np.uint16)
    got, ref = host.silu(stream, every, dtype), orc.silu_16(every, dtype)
    gf, rf = orc.to_float(got, dtype), orc.to_float(ref, dtype)
    nan = np.isnan(rf)
    assert np.array_equal(np.isnan(gf), nan) and np.array_equal(got[~nan], ref[~nan])
    for n in (1024 * 40 * 30, (1 << 22) + 4099):
        x = orc.fill_uniform(n, dtype, 304, -8.0, 8.0)
        assert np.array_equal(host.silu(stream, x, dtype), orc.silu_16(x, dtype)), n


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(32, 16, 64, 64), (10, 24), (7, 1023), (3, 512 * 4096 + 16), (5, 512 * 2048 + 3)])
def test_reduce_outer_sixteen_bit(host, orc, stream, dtype, shape):
    """benchmarks/reduce/reduce.dtypes.in lists f16 and bf16: f32 accumulation in slice order, one rounding."""
    x = orc.fill_uniform(int(np.prod(shape)), dtype, 305, -1.0, 1.0).reshape(shape)
    got = host.reduce_outer(stream, x, init=0.25, dtype=dtype)
    assert np.array_equal(got, orc.reduce_outer_16(x, dtype, init=0.25))


def test_rowmean(host, orc, stream):
    """Mean over the last dimension (WG/reduction_4D_3D_mean_intra_sg_intra_lane.mlir: 1x24x1024x64,
    uniform(-1,1) inputs, checked there against the sequential CPU loop with allclose)."""
    x = orc.fill_uniform(24 * 1024 * 64, "f32", 79, -1.0, 1.0).reshape(24 * 1024, 64)
    got, ref = host.rowmean(stream, x), orc.rowmean_f32(x)
    assert np.all(np.abs(got - ref) <= 1e-4 + 1e-3 * np.abs(ref))   # the reference's allclose
    assert np.max(np.abs(got - ref)) <= 2e-7                          # and far inside it
    # integer-valued rows: the sum is exact in any order, so the mean is the oracle's bits
    for rows, cols in ((7, 64), (5, 3000), (1000, 96), (3, 1)):
        m = orc.fill_int(rows * cols, "f32", 80, -8, 8).reshape(rows, cols)
        assert np.array_equal(host.rowmean(stream, m), orc.rowmean_f32(m)), (rows, cols)


@pytest.mark.parametrize("shape", [(32, 16, 64, 64), (10, 20), (7, 1023), (33, 4100), (1, 5), (3, 1, 9),
                                   (5, 512 * 2048 + 4), (3, 512 * 4096 + 1028), (2, 512 * 8192 + 8), (6, 512 * 2048 + 3)])
def test_reduce_outer_bit_exact(host, orc, stream, shape):
    """The last four shapes reach the 8, 16 and 32 KiB-per-slice variants with a ragged last
    workgroup, and the one-lane-per-output path at a size where it strides."""
    x = orc.fill_uniform(int(np.prod(shape)), "f32", 77, -1.0, 1.0).reshape(shape)
    got, ref = host.reduce_outer(stream, x, init=0.25), orc.reduce_outer_f32(x, init=0.25)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_reduce_outer_benchmark_shape_and_any_grid(host, orc, stream):
    """32x16x512x512 (the reference suite's reduce shape, README.md:335): integer-valued inputs
    make the sum exact; then the same kernel on a grid of 7 workgroups, which must stride."""
    import ctypes as C
    outer, inner = 32, 16 * 512 * 512
    x = orc.fill_int(outer * inner, "f32", 78, -8, 8).reshape(outer, inner)
    got = host.reduce_outer(stream, x, init=1.0)
    assert np.array_equal(got, 1.0 + x.sum(axis=0, dtype=np.float64).astype(np.float32))
    small = x[:, :300000]
    small = np.ascontiguousarray(small)
    d_in, d_out = stream.to_device(small), stream.alloc(small.shape[1] * 4)
    fn = stream.kernel("imex_reduce_outer_f32")
    descs, keep = host._pack_params([d_in, d_out, outer, small.shape[1], 1.0])
    stream.rt.gpuLaunchKernel(stream.handle, fn, 7, 1, 1, 256, 1, 1, 0, C.cast(descs, C.c_void_p), None)
    stream.wait()
    out = stream.from_device(d_out, (small.shape[1],), np.float32)
    stream.free(d_in)
    stream.free(d_out)
    assert np.array_equal(out, 1.0 + small.sum(axis=0, dtype=np.float64).astype(np.float32))


@pytest.mark.parametrize("grid", [(3, 1, 1), (100000, 1, 1)])
def test_streaming_kernels_any_grid(host, orc, stream, grid):
    """relu, silu, softmax, row sum and the fused chain stride over their work: a grid much
    smaller or much larger than the catalogue's gives the same bits."""
    n = 3 * 4096 * 5 + 77
    x = orc.fill_uniform(n, "f32", 91, -3, 3)
    for kernel, ref in (("imex_relu_f32", orc.relu_f32(x)), ("imex_silu_f32", orc.silu_f32(x))):
        d_in, d_out = stream.to_device(x), stream.alloc(n * 4)
        stream.launch(kernel, [n], [d_in, d_out, n], grid=grid)
        stream.wait()
        got = stream.from_device(d_out, (n,), np.float32)
        stream.free(d_in), stream.free(d_out)
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), kernel
    for rows, cols in ((37, 3000), (1000, 300)):
        m = orc.fill_int(rows * cols, "f32", 92, -8, 8).reshape(rows, cols)
        d_in, d_out = stream.to_device(m), stream.alloc(rows * 4)
        stream.launch("imex_rowsum_f32", [rows, cols], [d_in, d_out, rows, cols, 2.0], grid=grid)
        stream.wait()
        got = stream.from_device(d_out, (rows,), np.float32)
        stream.free(d_in), stream.free(d_out)
        assert np.array_equal(got, 2.0 + m.sum(axis=1, dtype=np.float64).astype(np.float32)), (rows, cols)
    a = np.abs(orc.fill_uniform(n, "f32", 93, -3, 3)) + 0.5
    d_a, d_b, d_out = stream.to_device(x), stream.to_device(a), stream.alloc(n * 4)
    stream.launch("imex_loop_fusion_f32", [n], [d_a, d_b, d_out, n], grid=grid)
    stream.wait()
    got = stream.from_device(d_out, (n,), np.float32)
    for p in (d_a, d_b, d_out):
        stream.free(p)
    assert np.array_equal(got.view(np.uint32), orc.loop_fusion_f32(x, a).view(np.uint32))


# =============================== Transpose =================================
def test_transpose_golden(host, orc, stream):
    g = GOLD["transpose_f32_10x20"]
    assert np.array_equal(host.transpose2d(stream, arr(g["input"], g["shape"])), arr(g["expected"], [20, 10]))
    g = GOLD["transpose_bf16_10x20"]
    xb = orc.float_to_bfloat(arr(g["input"], g["shape"]))
    assert np.array_equal(orc.bfloat_to_float(host.transpose2d(stream, xb)), arr(g["expected"], [20, 10]))


@pytest.mark.parametrize("rows,cols", [(1, 1), (64, 64), (128, 136), (1024, 1024), (63, 65), (8, 2000), (200, 8),
                                       (72, 520), (1000, 3), (257, 129)])
@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_transpose_shapes_bit_exact(host, orc, stream, rows, cols, dtype):
    say("transpose %s %dx%d" % (dtype, rows, cols))
    x = orc.fill_bits(rows * cols, dtype, 20244 + rows).reshape(rows, cols)
    got = host.transpose2d(stream, x)
    assert np.array_equal(got, orc.transpose2d(x))
    assert np.array_equal(host.transpose2d(stream, got), x)  # involution


def test_transpose_config_sizes(host, orc, stream):
    x = orc.fill_bits(8192 * 8192, "bf16", 20244).reshape(8192, 8192)
    got = host.transpose2d(stream, x)
    assert np.array_equal(got, x.T)
    # index-encoded input: every element lands where its index says
    idx = np.arange(4096 * 4096, dtype=np.uint32).reshape(4096, 4096)
    assert np.array_equal(host.transpose2d(stream, idx), idx.T)
    y = orc.fill_bits(4096 * 4096, "f32", 20245).reshape(4096, 4096)
    assert np.array_equal(host.transpose2d(stream, y), orc.transpose2d(y))


@pytest.mark.parametrize("rows,cols", [(4104, 4120), (8200, 2056), (300, 65544)])
@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_transpose_large_tiles_ragged(host, orc, stream, rows, cols, dtype):
    """From 2^24 elements the kernels use 128 x 128 (32-bit) / 256 x 128 (16-bit)
    tiles; these shapes end in partial tiles on both sides."""
    x = orc.fill_bits(rows * cols, dtype, 20244 + cols).reshape(rows, cols)
    got = host.transpose2d(stream, x)
    assert np.array_equal(got, x.T)


@pytest.mark.parametrize("rows,cols", [(4096, 4224), (128, 131072), (8192, 4096)])
def test_transpose_b32_whole_tiles_pipelined(host, orc, stream, rows, cols):
    """32-bit problems made of whole 128 x 128 tiles: at most 512 workgroups, each walking two or more tiles
    with the next tile's loads issued before the current tile is written (an odd and an even number of tiles
    per workgroup, a single tile row)."""
    x = np.arange(rows * cols, dtype=np.uint32).reshape(rows, cols)
    assert np.array_equal(host.transpose2d(stream, x), x.T)


def test_transpose3d_b32_whole_tiles_pipelined(host, orc, stream):
    shape = (256, 64, 1024)
    x = np.arange(int(np.prod(shape)), dtype=np.uint32).reshape(shape)
    assert np.array_equal(host.transpose3d(stream, x), x.transpose(2, 1, 0))


def test_transpose_any_grid(host, orc, stream):
    """Workgroups stride over the tiles: a grid smaller or larger than one workgroup
    per tile gives the same result."""
    import ctypes as C
    for name, np_t, rows, cols in [("imex_transpose2d_b32", np.uint32, 4096, 4104), ("imex_transpose2d_b16", np.uint16, 520, 264),
                                   ("imex_transpose2d_b32", np.uint32, 4096, 4096)]:
        x = np.arange(rows * cols, dtype=np.uint64).astype(np_t).reshape(rows, cols)
        for grid in [(3, 1, 1), (7, 5, 2), (40, 30, 1)]:
            d_in, d_out = stream.to_device(x), stream.alloc(x.nbytes)
            fn = stream.kernel(name)
            descs, keep = host._pack_params([d_in, d_out, rows, cols])
            stream.rt.gpuLaunchKernel(stream.handle, fn, grid[0], grid[1], grid[2], 256, 1, 1, 0,
                                      C.cast(descs, C.c_void_p), None)
            stream.wait()
            got = stream.from_device(d_out, (cols, rows), np_t)
            stream.free(d_in)
            stream.free(d_out)
            assert np.array_equal(got, x.T), (name, grid)


@pytest.mark.parametrize("shape", [(16, 96, 96), (96, 7, 96), (5, 3, 9), (64, 2, 72), (520, 64, 512)])
def test_transpose3d(host, orc, stream, shape):
    n = int(np.prod(shape))
    x32 = orc.fill_bits(n, "f32", 5).reshape(shape)
    assert np.array_equal(host.transpose3d(stream, x32), orc.transpose3d(x32))
    x16 = orc.fill_bits(n, "f16", 6).reshape(shape)
    assert np.array_equal(host.transpose3d(stream, x16), x16.transpose(2, 1, 0))


# ========================= fused element-wise chains ========================
@pytest.mark.parametrize("shape", [(512, 1024), (7, 13), (1, 4097), (300, 1000)])
def test_loop_fusion_f32_bit_exact(host, orc, stream, shape):
    """kLoopFusion: the device logf is the host libm's algorithm, every op is a
    separately rounded f32 one, so the result is the oracle's bit for bit."""
    n = int(np.prod(shape))
    a = orc.fill_uniform(n, "f32", 41, 0.01, 40.0).reshape(shape)
    b = orc.fill_uniform(n, "f32", 42, -5.0, 5.0).reshape(shape)
    a.flat[:6] = [3.3, 1.0, 1e-40, 0.0, np.inf, 0.99999994]
    got = host.loop_fusion(stream, a, b)
    want = orc.loop_fusion_f32(a, b)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_loop_fusion_logf_sweep(host, orc, stream):
    """b = 0 and exact cancellation aside, out + a = log a: sweep log over 16M bit
    patterns of the whole positive range through the fused kernel."""
    bits = (np.arange(1 << 24, dtype=np.uint64) * 127 + 1).astype(np.uint32) % np.uint32(0x7f800000)
    a = bits.view(np.float32)
    b = np.zeros_like(a)
    got = host.loop_fusion(stream, a, b)
    want = orc.loop_fusion_f32(a, b)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_empty_inputs_every_operator(host, stream):
    """Tensors with a zero extent: nothing is launched (a grid of zero workgroups is not a launch), results have
    the right shape, a row sum over no columns is the initial value and a product over K = 0 is all zeros."""
    f = np.float32
    assert host.relu(stream, np.zeros((0,), f)).shape == (0,)
    assert host.silu(stream, np.zeros((0,), f)).shape == (0,)
    assert host.softmax(stream, np.zeros((0, 16), f), "f32").shape == (0, 16)
    assert host.softmax(stream, np.zeros((4, 0), f), "f32").shape == (4, 0)
    assert host.rowsum(stream, np.zeros((0, 16), f)).shape == (0,)
    assert np.array_equal(host.rowsum(stream, np.zeros((5, 0), f)), np.zeros(5, f))
    assert host.transpose2d(stream, np.zeros((0, 7), f)).shape == (7, 0)
    assert host.transpose2d(stream, np.zeros((7, 0), f)).shape == (0, 7)
    assert host.gemm(stream, np.zeros((0, 8), np.uint16), np.zeros((8, 16), np.uint16)).shape == (0, 16)
    assert np.array_equal(host.gemm(stream, np.zeros((4, 0), np.uint16), np.zeros((0, 16), np.uint16)), np.zeros((4, 16), f))


def test_fused_chains_empty_and_single(host, orc, stream):
    empty = np.zeros((0,), np.float32)
    assert host.loop_fusion(stream, empty, empty).shape == (0,)
    one = host.loop_fusion(stream, np.float32([2.5]), np.float32([-1.5]))
    assert np.array_equal(one, orc.loop_fusion_f32(np.float32([2.5]), np.float32([-1.5])))
    no_rows = host.input_fusion(stream, np.zeros((0, 12), np.float32), np.zeros((0, 12), np.float32))
    assert np.array_equal(no_rows.view(np.uint32), np.zeros(12, np.uint32))  # a sum over nothing: +0.0
    col = host.input_fusion(stream, np.float32([[1.0], [-2.0], [3.0]]), np.float32([[0.5], [2.0], [8.0]]))
    assert np.array_equal(col, orc.input_fusion_f32(np.float32([[1.0], [-2.0], [3.0]]), np.float32([[0.5], [2.0], [8.0]])))


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_loop_fusion_16bit(host, orc, stream, dtype):
    n = 512 * 1024 + 77
    a = orc.fill_uniform(n, dtype, 43, 0.05, 30.0)
    b = orc.fill_uniform(n, dtype, 44, -5.0, 5.0)
    got = orc.to_float(host.loop_fusion(stream, a, b, dtype), dtype)
    # widen, f32 chain, one rounding at the end
    want = orc.to_float(orc.from_float(orc.loop_fusion_f32(orc.to_float(a, dtype), orc.to_float(b, dtype)), dtype), dtype)
    assert np.array_equal(got, want)


# from 2048 x 4096 on the launch asks for the streaming form (576 lanes): whole tiles, ragged rows and a partial
# last block of columns, and a column count that is not made of whole vectors (the kernel falls back by itself)
# below 4096 columns: four columns per workgroup, 64-row tiles, eight tiles' loads together (one group, several
# groups, a partial last tile, a partial last block of columns)
@pytest.mark.parametrize("shape", [(512, 1024), (9, 5), (1000, 300), (3, 2049), (1500, 36), (513, 4), (2048, 4096),
                                   (2500, 4100), (2049, 4098)])
def test_input_fusion_f32_bit_exact(host, orc, stream, shape):
    """kInputFusion: column sums in row order from +0.0, as the reference adds them."""
    n = int(np.prod(shape))
    a = orc.fill_uniform(n, "f32", 45, -5.0, 5.0).reshape(shape)
    b = orc.fill_uniform(n, "f32", 46, 0.01, 40.0).reshape(shape)
    got = host.input_fusion(stream, a, b)
    want = orc.input_fusion_f32(a, b)
    assert got.shape == (shape[1],)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("shape", [(512, 1024), (700, 41), (2048, 8192), (2100, 8200)])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_input_fusion_16bit(host, orc, stream, dtype, shape):
    rows, cols = shape
    a = orc.fill_uniform(rows * cols, dtype, 47, -2.0, 2.0).reshape(rows, cols)
    b = orc.fill_uniform(rows * cols, dtype, 48, 0.5, 4.0).reshape(rows, cols)
    got = orc.to_float(host.input_fusion(stream, a, b, dtype), dtype)
    want = orc.to_float(orc.from_float(orc.input_fusion_f32(orc.to_float(a, dtype), orc.to_float(b, dtype)), dtype), dtype)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shape,block", [((600, 520), 320), ((2048, 4160), 576), ((2048, 4160), 256), ((600, 520), 256)])
def test_input_fusion_any_grid(host, orc, stream, shape, block):
    """Workgroups stride over the blocks of columns in every form of the kernel (the narrow and the wide
    streaming form, and the 256-lane form a launch with 256 lanes always gets): a grid of a few
    workgroups gives the same bits as the catalogue's."""
    import ctypes as C
    rows, cols = shape
    a = orc.fill_uniform(rows * cols, "f32", 51, -5.0, 5.0).reshape(shape)
    b = orc.fill_uniform(rows * cols, "f32", 52, 0.01, 40.0).reshape(shape)
    want = orc.input_fusion_f32(a, b)
    d_a, d_b, d_out = stream.to_device(a), stream.to_device(b), stream.alloc(cols * 4)
    fn = stream.kernel("imex_input_fusion_f32")
    descs, keep = host._pack_params([d_a, d_b, d_out, rows, cols])
    for grid in (1, 7):
        stream.memset(d_out, 0x7fc00000, cols, 32)
        stream.rt.gpuLaunchKernel(stream.handle, fn, grid, 1, 1, block, 1, 1, 0, C.cast(descs, C.c_void_p), None)
        stream.wait()
        got = stream.from_device(d_out, (cols,), np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (shape, block, grid)
    for p in (d_a, d_b, d_out):
        stream.free(p)


# ============================ flash attention ===============================
def attention_close(got_bits, ref_bits, orc):
    """The reference checks its kernel with allclose (atol 1e-4, rtol 1e-3) on a constant
    input.  On random inputs the kernel (P truncated to f16 before normalisation, keys
    in blocks) and the CPU loop (P truncated after normalisation, keys in order) differ
    by f16 roundings of P, each <= 2^-11 relative: |d| <= 2^-10 * max|V| plus one f16
    output rounding."""
    got, ref = orc.half_to_float(got_bits), orc.half_to_float(ref_bits)
    return np.max(np.abs(got - ref)) <= 2.0 ** -10 + 2.0 ** -11 * np.max(np.abs(ref))


@pytest.mark.parametrize("zh,n_ctx", [(1, 128), (3, 256), (2, 1024), (2, 100), (1, 64)])
def test_flash_attention_vs_oracle(host, orc, stream, zh, n_ctx):
    n = zh * n_ctx
    q = orc.fill_uniform(n * 64, "f16", 51, -1, 1).reshape(n, 64)
    k = orc.fill_uniform(n * 64, "f16", 52, -1, 1).reshape(n, 64)
    v = orc.fill_uniform(n * 64, "f16", 53, -1, 1).reshape(n, 64)
    got = host.flash_attention(stream, q, k, v, zh, n_ctx, 0.5)
    rows = np.arange(n) if n <= 512 else np.unique(np.concatenate([np.arange(0, n, 37), [n_ctx - 1, n_ctx, n - 1]]))
    ref = orc.flash_attention_rows(q, k, v, n_ctx, 0.5, rows)
    assert attention_close(got[rows], ref, orc)


def test_flash_attention_sixteen_heads(host, orc, stream):
    """16 x 1024 x 64 with the scale 0.350097656 of the reference's second attention
    test (WG/flash_attention_fwd_ov_with_arrray_len_1k.mlir:22,40; inputs there are
    uniform(-1,1), checked against a natural-exp softmax)."""
    zh, n_ctx, scale = 16, 1024, 0.350097656
    n = zh * n_ctx
    q = orc.fill_uniform(n * 64, "f16", 61, -1, 1).reshape(n, 64)
    k = orc.fill_uniform(n * 64, "f16", 62, -1, 1).reshape(n, 64)
    v = orc.fill_uniform(n * 64, "f16", 63, -1, 1).reshape(n, 64)
    got = host.flash_attention(stream, q, k, v, zh, n_ctx, scale)
    rows = np.unique(np.concatenate([np.arange(0, n, 211), [1023, 1024, n - 1]]))
    assert attention_close(got[rows], orc.flash_attention_rows(q, k, v, n_ctx, scale, rows), orc)


@pytest.mark.parametrize("zh,n_ctx,scale", [(3, 512, 0.5), (2, 256, 4.0), (1, 2048, 0.125)])
def test_flash_attention_every_tiling(host, orc, stream, zh, n_ctx, scale):
    """64, 128 and 256 queries per workgroup (2, 4, 8 query blocks x 4, 2, 1 key groups; ring of
    2, 4, 8 stages) and 256 queries as sixteen wavefronts (8 x 2, ring of 4): each against the
    oracle, on the same inputs."""
    n = zh * n_ctx
    q = orc.fill_uniform(n * 64, "f16", 71, -2, 2).reshape(n, 64)
    k = orc.fill_uniform(n * 64, "f16", 72, -2, 2).reshape(n, 64)
    v = orc.fill_uniform(n * 64, "f16", 73, -1, 1).reshape(n, 64)
    rows = np.unique(np.concatenate([np.arange(0, n, 7), [n_ctx - 1, n - 1]]))
    ref = orc.flash_attention_rows(q, k, v, n_ctx, scale, rows)
    for queries, threads in ((64, 512), (128, 512), (256, 512), (256, 1024)):
        say("attention %dx%d, %d queries per workgroup of %d threads" % (zh, n_ctx, queries, threads))
        got = host.flash_attention(stream, q, k, v, zh, n_ctx, scale, queries_per_workgroup=queries, threads=threads)
        assert attention_close(got[rows], ref, orc), (queries, threads)


@pytest.mark.parametrize("zh,n_ctx,scale", [(2, 100, 0.5), (3, 1000, 0.125), (2, 257, 1.0), (1, 5, 0.5), (5, 333, 2.0),
                                             (1, 193, 0.5), (2, 64, 0.5)])
def test_flash_attention_ragged_context(host, orc, stream, zh, n_ctx, scale):
    """N_CTX that divides none of the tiles: padded queries are not stored, padded keys get a
    score of -inf; key groups that see no key at all (short heads) merge as empty.  Every
    tiling, every row, against the oracle; the rows behind Out stay untouched."""
    n = zh * n_ctx
    q = orc.fill_uniform(n * 64, "f16", 81, -2, 2).reshape(n, 64)
    k = orc.fill_uniform(n * 64, "f16", 82, -2, 2).reshape(n, 64)
    v = orc.fill_uniform(n * 64, "f16", 83, -1, 1).reshape(n, 64)
    rows = np.arange(n) if n <= 1200 else np.unique(np.concatenate([np.arange(0, n, 3), [n_ctx - 1, n_ctx, n - 1]]))
    ref = orc.flash_attention_rows(q, k, v, n_ctx, scale, rows)
    got = host.flash_attention(stream, q, k, v, zh, n_ctx, scale)
    assert attention_close(got[rows], ref, orc), "catalogue launch"
    for queries, threads in ((64, 512), (128, 512), (256, 512), (256, 1024)):
        say("attention %dx%d ragged, %d queries per workgroup of %d threads" % (zh, n_ctx, queries, threads))
        guard = np.full((n + 256, 64), 0x7e01, np.uint16)
        d_q, d_k, d_v, d_o = (stream.to_device(t) for t in (q, k, v, guard))
        grid = (-(-n_ctx // queries), zh, 1)
        stream.launch("imex_flash_attention_fwd_f16", [zh, n_ctx], [d_q, d_k, d_v, d_o, float(scale), zh, n_ctx],
                      grid=grid, block=(threads, 1, 1))
        stream.wait()
        out = stream.from_device(d_o, (n + 256, 64), np.uint16)
        for p in (d_q, d_k, d_v, d_o):
            stream.free(p)
        assert np.all(out[n:] == 0x7e01), (queries, threads, "wrote behind Out")
        assert attention_close(out[rows], ref, orc), (queries, threads)


def test_flash_attention_negative_scale_takes_the_reference_loop(host, orc, stream):
    """The tiled path takes the row maximum before scaling, which needs a positive scale; any
    other scale runs the one-lane-per-query loop of the same kernel."""
    zh, n_ctx = 2, 256
    n = zh * n_ctx
    q = orc.fill_uniform(n * 64, "f16", 84, -1, 1).reshape(n, 64)
    k = orc.fill_uniform(n * 64, "f16", 85, -1, 1).reshape(n, 64)
    v = orc.fill_uniform(n * 64, "f16", 86, -1, 1).reshape(n, 64)
    rows = np.arange(0, n, 3)
    got = host.flash_attention(stream, q, k, v, zh, n_ctx, -0.5)
    assert attention_close(got[rows], orc.flash_attention_rows(q, k, v, n_ctx, -0.5, rows), orc)


@pytest.mark.parametrize("zh", [8, 16])
def test_flash_attention_catalogue_picks_wide_tilings(host, orc, stream, zh):
    """N_CTX = 4096 with 8 and 16 heads: the catalogue launches 128- and 256-query workgroups
    (16 heads is the reference's flash_attention_fwd_ov_with_arrray_len_4k.mlir shape)."""
    n_ctx = 4096
    grid, block, _ = host.launch_shape("imex_flash_attention_fwd_f16", [zh, n_ctx])
    assert grid == (n_ctx // (16 * zh), zh, 1) and block == ((1024 if zh == 16 else 512), 1, 1)
    n = zh * n_ctx
    q = orc.fill_uniform(n * 64, "f16", 74, -1, 1).reshape(n, 64)
    k = orc.fill_uniform(n * 64, "f16", 75, -1, 1).reshape(n, 64)
    v = orc.fill_uniform(n * 64, "f16", 76, -1, 1).reshape(n, 64)
    got = host.flash_attention(stream, q, k, v, zh, n_ctx, 0.5)
    rows = np.unique(np.concatenate([np.arange(0, n, 2999), [255, 256, n_ctx - 1, n_ctx, n - 1]]))
    assert attention_close(got[rows], orc.flash_attention_rows(q, k, v, n_ctx, 0.5, rows), orc)


def test_flash_attention_sharp_scores(host, orc, stream):
    """Large score range (scale 4, |q.k| up to ~20): the running max changes from block
    to block and the rescaling of the accumulator is exercised."""
    zh, n_ctx = 2, 512
    n = zh * n_ctx
    q = orc.fill_uniform(n * 64, "f16", 54, -2, 2).reshape(n, 64)
    k = orc.fill_uniform(n * 64, "f16", 55, -2, 2).reshape(n, 64)
    v = orc.fill_uniform(n * 64, "f16", 56, -1, 1).reshape(n, 64)
    got = host.flash_attention(stream, q, k, v, zh, n_ctx, 4.0)
    rows = np.arange(0, n, 5)
    assert attention_close(got[rows], orc.flash_attention_rows(q, k, v, n_ctx, 4.0, rows), orc)


def test_flash_attention_reference_config(host, orc, stream):
    """Z = 2, H = 2, N_CTX = 4096, D = 64, scale 0.5 (flash_attention_fwd.mlir:449-454):
    the reference's own constant input exactly, then random inputs on sampled rows."""
    zh, n_ctx = 4, 4096
    n = zh * n_ctx
    const = orc.from_float(np.full((n, 64), 0.625, np.float32), "f16")
    out = host.flash_attention(stream, const, const, const, zh, n_ctx, 0.5)
    assert np.all(orc.half_to_float(out) == 0.625)
    q = orc.fill_uniform(n * 64, "f16", 57, -1, 1).reshape(n, 64)
    k = orc.fill_uniform(n * 64, "f16", 58, -1, 1).reshape(n, 64)
    v = orc.fill_uniform(n * 64, "f16", 59, -1, 1).reshape(n, 64)
    got = host.flash_attention(stream, q, k, v, zh, n_ctx, 0.5)
    rows = np.array([0, 1, 63, 64, 4095, 4096, 5000, 8191, 8192, 12287, 12288, 16383])
    ref = orc.flash_attention_rows(q, k, v, n_ctx, 0.5, rows)
    assert attention_close(got[rows], ref, orc)
    # permuting the keys (and values with them) of one head leaves its outputs unchanged up to rounding
    perm = np.random.default_rng(3).permutation(n_ctx)
    k2, v2 = k.copy(), v.copy()
    k2[:n_ctx], v2[:n_ctx] = k[:n_ctx][perm], v[:n_ctx][perm]
    got2 = host.flash_attention(stream, q, k2, v2, zh, n_ctx, 0.5)
    assert attention_close(got2[:n_ctx], got[:n_ctx], orc)
    assert np.array_equal(got2[n_ctx:], got[n_ctx:])


# =============================== GEMM ======================================
def gemm_close(got, ref):
    return np.max(np.abs(got - ref)) <= 5e-3 * np.max(np.abs(ref))


def test_gemm_golden_3x3(host, orc, stream):
    g = GOLD["gemm_f16_acc_f32_3x3"]
    a, b = orc.float_to_half(arr(g["A"], [3, 3])), orc.float_to_half(arr(g["B"], [3, 3]))
    c = host.gemm(stream, a, b, c=arr(g["C0"], [3, 3]), ab_dtype="f16")
    assert orc.allclose_f32(c, arr(g["expected"], [3, 3]))
    assert np.array_equal(c, orc.gemm(a, b, "f16", c=arr(g["C0"], [3, 3])))  # scalar path: same order, bit-exact
    g = GOLD["gemm_bf16_acc_f32_3x3"]
    a, b = orc.float_to_bfloat(arr(g["A"], [3, 3])), orc.float_to_bfloat(arr(g["B"], [3, 3]))
    c = host.gemm(stream, a, b, c=arr(g["C0"], [3, 3]), ab_dtype="bf16")
    assert np.max(np.abs(c.ravel() - arr(g["expected"]))) < 6e-5
    g = GOLD["dot_f16_acc_f32_8x16x32"]
    a = orc.float_to_half(np.full((8, 16), 1.0, np.float32))
    b = orc.float_to_half(np.full((16, 32), 2.0, np.float32))
    out = host.gemm(stream, a, b, ab_dtype="f16", out_dtype="f16")
    assert np.all(orc.half_to_float(out) == g["expected_fill"])


@pytest.mark.parametrize("M,N,K", [(5, 7, 9), (100, 36, 130), (256, 256, 20), (256, 256, 44), (255, 252, 64), (17, 300, 64),
                                   (300, 260, 50), (129, 129, 17)])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_untileable_shapes_bit_exact(host, orc, stream, M, N, K, dtype):
    """K not a multiple of 8 or N not a multiple of 8: the vector-ALU path (128 x 128 tiles, sixteen k at a
    time), which accumulates every output in the oracle's order."""
    a = orc.fill_uniform(M * K, dtype, 1, -1, 1).reshape(M, K)
    b = orc.fill_uniform(K * N, dtype, 2, -1, 1).reshape(K, N)
    assert np.array_equal(host.gemm(stream, a, b, ab_dtype=dtype), orc.gemm(a, b, dtype))


def test_gemm_untileable_special_values(host, orc, stream):
    """The vector-ALU path pads its tiles with zeros beyond M, N and K; infinities, NaNs and negative zeros
    in the operands must come out as in the sequential loop, which never sees the padding."""
    M, N, K = 70, 37, 21
    a = orc.fill_uniform(M * K, "f16", 3, -1, 1).reshape(M, K)
    b = orc.fill_uniform(K * N, "f16", 4, -1, 1).reshape(K, N)
    a[3, 5], a[9, 20], a[60, 0], a[69, 20] = 0x7c00, 0xfc00, 0x7e00, 0x7c00      # +inf, -inf, NaN, +inf
    b[20, 36], b[0, 0] = 0x7c00, 0xfc00
    a[11, :] = 0x8000                                                         # a row of -0.0
    got, want = host.gemm(stream, a, b, ab_dtype="f16"), orc.gemm(a, b, "f16")
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok])


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_tiled_identity_and_layout(host, orc, stream, dtype):
    """B = I gives C = A exactly; A[i,j] = j patterns expose any fragment-layout mistake."""
    M, N, K = 512, 512, 512
    a = orc.fill_uniform(M * K, dtype, 3, -1, 1).reshape(M, K)
    eye = orc.from_float(np.eye(K, dtype=np.float32), dtype)
    assert np.array_equal(host.gemm(stream, a, eye, ab_dtype=dtype), orc.to_float(a, dtype))
    # A = I: C = B exactly (exercises the B transpose-in-registers path)
    b = orc.fill_uniform(K * N, dtype, 4, -1, 1).reshape(K, N)
    assert np.array_equal(host.gemm(stream, eye, b, ab_dtype=dtype), orc.to_float(b, dtype))
    # a single non-zero k picks out one row of B scaled by a column of A
    a1 = np.zeros((M, K), np.float32)
    a1[:, 77] = np.arange(M) % 16
    got = host.gemm(stream, orc.from_float(a1, dtype), b, ab_dtype=dtype)
    assert np.array_equal(got, np.outer(a1[:, 77], orc.to_float(b, dtype)[77]).astype(np.float32))


@pytest.mark.parametrize("dtype,M,N,K", [("f16", 512, 768, 4096), ("bf16", 256, 1024, 1024), ("f16", 1024, 256, 64),
                                           ("f16", 256, 256, 32), ("bf16", 512, 256, 96), ("f16", 256, 512, 160)])
def test_gemm_tiled_small_integers_exact(host, orc, stream, dtype, M, N, K):
    """|a|,|b| <= 4: every partial sum is an integer below 2^24, so any
    accumulation order gives the same f32 bits as the integer product."""
    a = orc.fill_int(M * K, dtype, 5, -4, 4).reshape(M, K)
    b = orc.fill_int(K * N, dtype, 6, -4, 4).reshape(K, N)
    want = orc.to_float(a, dtype).astype(np.int64) @ orc.to_float(b, dtype).astype(np.int64)
    got = host.gemm(stream, a, b, ab_dtype=dtype)
    assert np.array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("which", ["plain", "ta", "tb", "acc", "mlp"])
@pytest.mark.parametrize("M,N,K", [(256, 256, 8), (256, 256, 16), (256, 256, 48), (300, 520, 40), (512, 256, 4096 + 24),
                                   (64, 72, 104), (1000, 264, 72)])
def test_gemm_partial_last_k_step(host, orc, stream, which, M, N, K):
    """K a multiple of 8 but not of the 32-wide step: the MFMA path pads the last step with zeros on the
    way into LDS.  Integer operands give the exact product in any order, so any stale or foreign value
    that got multiplied in would show; every operand layout and an epilogue with its own loads."""
    say("gemm partial K step %s %dx%dx%d" % (which, M, N, K))
    if which == "ta" and M % 8:
        M = (M + 7) // 8 * 8
    dtype = "bf16" if which == "mlp" else "f16"
    a = orc.fill_int(M * K, dtype, 91, -4, 4).reshape(M, K)
    b = orc.fill_int(K * N, dtype, 92, -4, 4).reshape(K, N)
    want = orc.to_float(a, dtype).astype(np.int64) @ orc.to_float(b, dtype).astype(np.int64)
    if which == "plain":
        got = _gemm_guarded(host, stream, "imex_gemm_f16_f16_f32", a, b, M, N, K)
    elif which == "ta":
        got = _gemm_guarded(host, stream, "imex_gemm_f16_f16_f32_ta", np.ascontiguousarray(a.T), b, M, N, K)
    elif which == "tb":
        got = _gemm_guarded(host, stream, "imex_gemm_f16_f16_f32_tb", a, np.ascontiguousarray(b.T), M, N, K)
    elif which == "acc":
        c0 = orc.fill_int(M * N, "f32", 93, -1000, 1000).reshape(M, N)
        got = host.gemm(stream, a, b, c=c0, ab_dtype="f16")
        want = want + c0.astype(np.int64)
    else:
        bias = orc.fill_int(N, "f32", 94, -3, 3)
        out = _gemm_guarded(host, stream, "imex_gemm_bf16_bias_silu_bf16", a, b, M, N, K, extra=(bias,), out_np=np.uint16)
        ref = orc.bfloat_to_float(orc.bias_silu_bf16(want.astype(np.float32), bias))
        assert np.max(np.abs(orc.bfloat_to_float(out) - ref)) <= 2.0 ** -7 * np.max(np.abs(ref)) + 1e-6
        return
    assert np.array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("dtype,M,N,K", [("f16", 256, 256, 32), ("bf16", 256, 512, 96), ("f16", 512, 256, 224)])
def test_gemm_tiled_short_k_random(host, orc, stream, dtype, M, N, K):
    """K shorter than the copy pipeline is deep (1, 3 and 7 steps of 32): the
    prologue and the clamped tail copies must not disturb the result."""
    a = orc.fill_uniform(M * K, dtype, 11, -1, 1).reshape(M, K)
    b = orc.fill_uniform(K * N, dtype, 12, -1, 1).reshape(K, N)
    assert gemm_close(host.gemm(stream, a, b, ab_dtype=dtype), orc.gemm(a, b, dtype))


def _gemm_guarded(host, stream, name, sa, sb, M, N, K, extra=(), out_np=np.float32):
    """Launch a GEMM kernel on an output buffer with 256 guard rows behind it; returns the
    [M,N] result after checking that the guard rows kept their fill."""
    guard = 256
    fill = np.full((M + guard, N), 0x7fc1 if out_np == np.uint16 else np.float32(-12345.5), out_np)
    d_a, d_b, d_c = stream.to_device(sa), stream.to_device(sb), stream.to_device(fill)
    extras = [stream.to_device(e) for e in extra]
    try:
        stream.launch(name, [M, N, K], [d_a, d_b] + extras + [d_c, M, N, K])
        stream.wait()
        out = stream.from_device(d_c, (M + guard, N), out_np)
    finally:
        for p in [d_a, d_b, d_c] + extras:
            stream.free(p)
    assert np.array_equal(out[M:], fill[M:]), "%s wrote past row %d" % (name, M)
    return out[:M]


@pytest.mark.parametrize("M,N,K", [(255, 256, 64), (1, 8, 32), (300, 520, 96), (257, 264, 1024), (4000, 1000, 128),
                                   (31, 4104, 64)])
def test_gemm_ragged_tiles(host, orc, stream, M, N, K):
    """M and N that do not divide the 256 x 256 tile (K % 32 == 0, N % 8 == 0): the MFMA path with
    edge tiles.  Integer operands give the exact product in any order; random ones the 5e-3 bar;
    nothing is stored outside C."""
    say("gemm ragged %dx%dx%d" % (M, N, K))
    a = orc.fill_int(M * K, "f16", 5, -4, 4).reshape(M, K)
    b = orc.fill_int(K * N, "f16", 6, -4, 4).reshape(K, N)
    want = orc.to_float(a, "f16").astype(np.int64) @ orc.to_float(b, "f16").astype(np.int64)
    got = _gemm_guarded(host, stream, "imex_gemm_f16_f16_f32", a, b, M, N, K)
    assert np.array_equal(got.astype(np.int64), want)
    a = orc.fill_uniform(M * K, "bf16", 13, -1, 1).reshape(M, K)
    b = orc.fill_uniform(K * N, "bf16", 14, -1, 1).reshape(K, N)
    rows = np.unique(np.concatenate([np.arange(0, M, 61), [M - 1]]))
    got = _gemm_guarded(host, stream, "imex_gemm_bf16_bf16_f32", a, b, M, N, K)
    assert gemm_close(got[rows], orc.gemm_rows(a, b, rows, "bf16"))
    # fused bias + SiLU epilogue and the f16-output one on the same ragged shape
    bias = orc.fill_normal(N, "f32", 15, 0.0, 0.1)
    fused = _gemm_guarded(host, stream, "imex_gemm_bf16_bias_silu_bf16", a, b, M, N, K, extra=(bias,), out_np=np.uint16)
    ref = orc.bfloat_to_float(orc.bias_silu_bf16(orc.gemm_rows(a, b, rows, "bf16"), bias))
    assert np.max(np.abs(orc.bfloat_to_float(fused)[rows] - ref)) <= 5e-3 * np.max(np.abs(ref)) + 2.0 ** -9


@pytest.mark.parametrize("which,M,N,K", [("ta", 248, 264, 64), ("ta", 8, 8, 32), ("tb", 100, 37, 64), ("tb", 300, 515, 96)])
def test_gemm_ragged_tiles_transposed_operands(host, orc, stream, which, M, N, K):
    """Edge tiles with A stored [K,M] (M % 8 == 0) or B stored [N,K] (any N)."""
    a = orc.fill_int(M * K, "f16", 33, -4, 4).reshape(M, K)
    b = orc.fill_int(K * N, "f16", 34, -4, 4).reshape(K, N)
    sa, sb = (np.ascontiguousarray(a.T), b) if which == "ta" else (a, np.ascontiguousarray(b.T))
    want = orc.to_float(a, "f16").astype(np.int64) @ orc.to_float(b, "f16").astype(np.int64)
    got = _gemm_guarded(host, stream, "imex_gemm_f16_f16_f32_" + which, sa, sb, M, N, K)
    assert np.array_equal(got.astype(np.int64), want)


def test_gemm_launch_shape_slack(host, orc, stream):
    """A grid with more or fewer workgroups than tiles (MFMA path: the workgroups stride
    over the tiles) or fewer workgroups than tiles (vector-ALU path) still
    computes every element once."""
    import ctypes as C
    for (M, N, K, grid) in [(256, 256, 64, 9), (100, 36, 130, 2), (1024, 768, 96, 5), (1000, 520, 64, 1)]:
        a = orc.fill_uniform(M * K, "f16", 21, -1, 1).reshape(M, K)
        b = orc.fill_uniform(K * N, "f16", 22, -1, 1).reshape(K, N)
        d_a, d_b, d_c = stream.to_device(a), stream.to_device(b), stream.alloc(M * N * 4)
        fn = stream.kernel("imex_gemm_f16_f16_f32")
        descs, keep = host._pack_params([d_a, d_b, d_c, M, N, K])
        stream.rt.gpuLaunchKernel(stream.handle, fn, grid, 1, 1, 512, 1, 1, 0, C.cast(descs, C.c_void_p), None)
        stream.wait()
        got = stream.from_device(d_c, (M, N), np.float32)
        assert gemm_close(got, orc.gemm(a, b, "f16"))
        for p in (d_a, d_b, d_c):
            stream.free(p)


def test_gemm_config_f16_4096(host, orc, stream):
    M = N = K = 4096
    a = orc.fill_uniform(M * K, "f16", 20246, -1, 1).reshape(M, K)
    b = orc.fill_uniform(K * N, "f16", 20247, -1, 1).reshape(K, N)
    got = host.gemm(stream, a, b, ab_dtype="f16")
    rows = np.array(sorted(set(list(range(0, 4096, 97)) + [1, 255, 256, 2047, 4095])))
    ref = orc.gemm_rows(a, b, rows, "f16")
    err = np.max(np.abs(got[rows] - ref)) / np.max(np.abs(ref))
    say("gemm f16 4096^3: max|d|/max|ref| = %.3e over %d rows" % (err, rows.size))
    assert err <= 5e-3
    # the remaining rows: linearity / checksum  (1^T C) == (1^T A) B in f64
    colsum = got.sum(axis=0, dtype=np.float64)
    want = orc.half_to_float(a).sum(axis=0, dtype=np.float64) @ orc.half_to_float(b).astype(np.float64)
    assert np.max(np.abs(colsum - want)) <= 1e-3 * np.max(np.abs(want)) + 0.05
    # accumulate variant and the reference-signature entry point give C0 + A.B
    c0 = orc.fill_uniform(M * N, "f32", 1, -1, 1).reshape(M, N)
    acc = host.gemm(stream, a, b, c=c0, ab_dtype="f16")
    assert np.max(np.abs(acc - (c0 + got))) <= 1e-4
    d_a, d_b, d_c = stream.to_device(a), stream.to_device(b), stream.to_device(c0)
    fn = stream.kernel("imex_gemm_4kx4kx4k_f16_f16_f32")
    descs, keep = host._pack_params([d_a, d_b, d_c])
    import ctypes as C
    stream.rt.gpuLaunchKernel(stream.handle, fn, 16, 16, 1, 512, 1, 1, 0, C.cast(descs, C.c_void_p), None)
    stream.wait()
    fixed = stream.from_device(d_c, (M, N), np.float32)
    for p in (d_a, d_b, d_c):
        stream.free(p)
    assert np.array_equal(fixed, acc)


@pytest.mark.parametrize("which", ["ta", "tb"])
def test_gemm_transposed_operands(host, orc, stream, which):
    """A stored [K,M] / B stored [N,K] (WG/gemm_4kx4kx4k_transpose_{a,b}.mlir): same
    product as the plain layout; checked the way the reference does, against the
    plain GEMM of the un-transposed copies."""
    kw = {"trans_a": True} if which == "ta" else {"trans_b": True}

    def stored(a, b):
        return (np.ascontiguousarray(a.T), b) if which == "ta" else (a, np.ascontiguousarray(b.T))

    # vector-ALU path: bit-exact against the sequential oracle
    for (M, N, K) in [(5, 7, 9), (100, 36, 130), (300, 260, 50)]:
        a = orc.fill_uniform(M * K, "f16", 31, -1, 1).reshape(M, K)
        b = orc.fill_uniform(K * N, "f16", 32, -1, 1).reshape(K, N)
        sa, sb = stored(a, b)
        assert np.array_equal(host.gemm(stream, sa, sb, **kw), orc.gemm(a, b, "f16"))
    # tiled path: integer operands are exact in any order; non-square so a swapped M/N/K shows
    for (M, N, K) in [(256, 512, 96), (768, 256, 1024)]:
        a = orc.fill_int(M * K, "f16", 33, -4, 4).reshape(M, K)
        b = orc.fill_int(K * N, "f16", 34, -4, 4).reshape(K, N)
        sa, sb = stored(a, b)
        want = orc.to_float(a, "f16").astype(np.int64) @ orc.to_float(b, "f16").astype(np.int64)
        assert np.array_equal(host.gemm(stream, sa, sb, **kw).astype(np.int64), want)
    # layout probes: identity on the transposed side returns the other operand exactly
    M = N = K = 512
    x = orc.fill_uniform(M * K, "f16", 35, -1, 1).reshape(M, K)
    eye = orc.from_float(np.eye(K, dtype=np.float32), "f16")
    if which == "ta":
        assert np.array_equal(host.gemm(stream, np.ascontiguousarray(x.T), eye, **kw), orc.to_float(x, "f16"))
    else:
        assert np.array_equal(host.gemm(stream, eye, np.ascontiguousarray(x.T), **kw), orc.to_float(x, "f16"))
    # random operands at the reference's size and range (-0.5, 0.5), sampled rows + column checksum
    M = N = K = 4096
    a = orc.fill_uniform(M * K, "f16", 36, -0.5, 0.5).reshape(M, K)
    b = orc.fill_uniform(K * N, "f16", 37, -0.5, 0.5).reshape(K, N)
    sa, sb = stored(a, b)
    got = host.gemm(stream, sa, sb, **kw)
    rows = np.array([0, 1, 255, 256, 1999, 4095])
    assert gemm_close(got[rows], orc.gemm_rows(a, b, rows, "f16"))
    colsum = got.sum(axis=0, dtype=np.float64)
    want = orc.half_to_float(a).sum(axis=0, dtype=np.float64) @ orc.half_to_float(b).astype(np.float64)
    assert np.max(np.abs(colsum - want)) <= 1e-3 * np.max(np.abs(want)) + 0.05
    # the reference-signature entry point accumulates onto C
    import ctypes as C
    c0 = orc.fill_uniform(M * N, "f32", 38, -1, 1).reshape(M, N)
    d_a, d_b, d_c = stream.to_device(sa), stream.to_device(sb), stream.to_device(c0)
    fn = stream.kernel("imex_gemm_4kx4kx4k_transpose_a" if which == "ta" else "imex_gemm_4kx4kx4k_transpose_b")
    descs, keep = host._pack_params([d_a, d_b, d_c])
    stream.rt.gpuLaunchKernel(stream.handle, fn, 16, 16, 1, 512, 1, 1, 0, C.cast(descs, C.c_void_p), None)
    stream.wait()
    fixed = stream.from_device(d_c, (M, N), np.float32)
    for p in (d_a, d_b, d_c):
        stream.free(p)
    assert np.max(np.abs(fixed - (c0 + got))) <= 1e-4


def _launch_raw(host, stream, name, args, grid, block=(512, 1, 1)):
    """gpuLaunchKernel with an explicit launch shape (the reference's own, for the fixed-shape entries)."""
    import ctypes as C
    fn = stream.kernel(name)
    descs, keep = host._pack_params(args)
    stream.rt.gpuLaunchKernel(stream.handle, fn, grid[0], grid[1], grid[2], block[0], block[1], block[2], 0,
                              C.cast(descs, C.c_void_p), None)
    stream.wait()
    del keep


def _column_checksum_f64(a_f32, b_f32):
    """(1^T A) B in f64, in column panels so that B is never held whole as f64."""
    s = a_f32.sum(axis=0, dtype=np.float64)
    out = np.empty(b_f32.shape[1], np.float64)
    for n0 in range(0, b_f32.shape[1], 1024):
        out[n0:n0 + 1024] = s @ b_f32[:, n0:n0 + 1024].astype(np.float64)
    return out


STRIDED_ROWS_4096 = np.array(sorted(set(list(range(0, 4096, 97)) + [1, 127, 128, 255, 256, 2047, 2048, 4095])))


def test_gemm_config_mlp_bf16_bias_silu(host, orc, stream):
    M, K, N = 4096, 4096, 11008
    a = orc.fill_normal(M * K, "bf16", 20248, 0.0, 1.0).reshape(M, K)
    b = orc.fill_normal(K * N, "bf16", 20249, 0.0, 0.02).reshape(K, N)
    bias = orc.fill_normal(N, "f32", 20250, 0.0, 0.1)
    got = orc.bfloat_to_float(host.gemm_bias_silu(stream, a, b, bias))
    rows = STRIDED_ROWS_4096  # a stride of 97 lands in every 128-row wavefront block of every 256-row tile
    acc = orc.gemm_rows(a, b, rows, "bf16")
    ref = orc.bfloat_to_float(orc.bias_silu_bf16(acc, bias))
    err = np.max(np.abs(got[rows] - ref)) / np.max(np.abs(ref))
    say("mlp gemm: max|d|/max|ref| = %.3e over %d rows" % (err, rows.size))
    assert err <= 5e-3
    # element-wise: within one bf16 step wherever the value is not tiny
    big = np.abs(ref) > 1e-2
    assert np.max(np.abs(got[rows][big] - ref[big]) / np.abs(ref[big])) <= 2.0 ** -7
    # plain bf16 GEMM with f32 output: the same rows, and every column's sum against (1^T A) B in f64
    plain = host.gemm(stream, a, b, ab_dtype="bf16")
    assert gemm_close(plain[rows], acc)
    want = _column_checksum_f64(orc.bfloat_to_float(a), orc.bfloat_to_float(b))
    assert np.max(np.abs(plain.sum(axis=0, dtype=np.float64) - want)) <= 1e-3 * np.max(np.abs(want)) + 0.05
    # the whole fused output against the epilogue applied (in f64) to that checked f32 product:
    # every element within one bf16 step, so no tile, wavefront block or column strip is left out
    v = plain.astype(np.float64) + bias.astype(np.float64)[None, :]
    want = v / (1.0 + np.exp(-v))
    del v
    d = np.abs(got - want)
    assert np.all(d <= 2.0 ** -7 * np.abs(want) + 1e-6), "fused epilogue differs at %s" % (np.argwhere(d > 2.0 ** -7 * np.abs(want) + 1e-6)[:4],)


def _streamk_against_plain(host, orc, a, b, bias, stream, **kw):
    """The stream-K kernel against the one-workgroup-per-tile kernel on the same operands: the f32 sums
    of a split tile are added in another order (partials, then the finisher's own), so the bf16 results
    agree to a rounding step of the output type, and mostly bit for bit."""
    plain = host.gemm_bias_silu(stream, a, b, bias)
    got = host.gemm_bias_silu(stream, a, b, bias, streamk=True, **kw)
    p, g = orc.bfloat_to_float(plain), orc.bfloat_to_float(got)
    assert np.array_equal(np.isnan(p), np.isnan(g))
    d = np.abs(p - g)
    # a step of the output type, plus the f32 rounding of a sum of K products where the sum nearly cancels
    bad = d > 2.0 ** -7 * np.abs(p) + 1e-4
    assert not bad.any(), (np.argwhere(bad)[:4], p[bad][:4], g[bad][:4])
    return float(np.mean(plain == got))


@pytest.mark.parametrize("M,N,K,grid", [
    (512, 768, 256, None),        # 6 tiles, 4 slabs of 64 k each: one workgroup per tile, nothing to split
    (512, 768, 4096, None),       # 6 tiles over 24 workgroups: every tile split four ways
    (1024, 1280, 2048, (7, 1, 1)),    # 20 tiles on 7 workgroups: two full rounds, 6 tiles dealt out over 7
    (1000, 520, 1024, (5, 1, 1)),     # ragged edge tiles, 12 tiles on 5 workgroups
    (256, 256, 8192, (16, 1, 1)),     # one tile, sixteen parts: a finisher with fifteen partners
    (300, 264, 192, (64, 1, 1)),      # more workgroups than slabs: most ranges are empty
    (512, 512, 96, (3, 1, 1)),        # K % 64 != 0: the kernel takes the ordinary path and ignores the workspace
])
def test_gemm_streamk_small_shapes(host, orc, stream, M, N, K, grid):
    say("stream-K %dx%dx%d grid %s" % (M, N, K, grid))
    a = orc.fill_normal(M * K, "bf16", 31, 0.0, 1.0).reshape(M, K)
    b = orc.fill_normal(K * N, "bf16", 32, 0.0, 0.05).reshape(K, N)
    bias = orc.fill_normal(N, "f32", 33, 0.0, 0.1)
    _streamk_against_plain(host, orc, a, b, bias, stream, grid=grid)
    # integer operands: every order of additions gives the same f32 sums, so the two kernels agree bit for bit
    a = orc.fill_int(M * K, "bf16", 34, -2, 2).reshape(M, K)
    b = orc.fill_int(K * N, "bf16", 35, -2, 2).reshape(K, N)
    assert _streamk_against_plain(host, orc, a, b, np.zeros(N, np.float32), stream, grid=grid) == 1.0
    # ... and twice in a row on one workspace with consecutive epochs (flags of the first launch are stale)
    assert _streamk_against_plain(host, orc, a, b, np.zeros(N, np.float32), stream, grid=grid) == 1.0


def test_gemm_streamk_impatient_finisher(host, orc, stream):
    """A finishing workgroup that is allowed a single look at its partners' flags mostly finds them unset
    and computes the missing slabs itself: the same results, and the kernel ends either way."""
    M, N, K = 768, 512, 4096
    a = orc.fill_int(M * K, "bf16", 36, -2, 2).reshape(M, K)
    b = orc.fill_int(K * N, "bf16", 37, -2, 2).reshape(K, N)
    bias = orc.fill_normal(N, "f32", 38, 0.0, 0.1)
    for grid in ((24, 1, 1), (5, 1, 1)):
        assert _streamk_against_plain(host, orc, a, b, bias, stream, grid=grid, spin_limit=1) == 1.0


def test_gemm_streamk_config_mlp(host, orc, stream):
    """The MLP configuration: 688 tiles on 256 workgroups, two full rounds and 176 tiles dealt out."""
    M, K, N = 4096, 4096, 11008
    a = orc.fill_normal(M * K, "bf16", 20248, 0.0, 1.0).reshape(M, K)
    b = orc.fill_normal(K * N, "bf16", 20249, 0.0, 0.02).reshape(K, N)
    bias = orc.fill_normal(N, "f32", 20250, 0.0, 0.1)
    assert host.launch_shape("imex_gemm_bf16_bias_silu_bf16_streamk", [M, N, K])[0] == (256, 1, 1)
    same = _streamk_against_plain(host, orc, a, b, bias, stream)
    say("stream-K MLP: %.4f of the outputs bit-identical to the plain kernel" % same)
    assert same > 0.95


def test_gemm_split_k_operator_entry(host, orc, stream):
    """imexHipGemmBiasSiluBf16SplitK (include/imex_hip_ops.h): the K-splitting kernel behind one call that
    sizes, allocates and stamps the workspace itself -- a few-tile, deep-K problem, then a larger one (the
    workspace grows), then the first again; each against the one-workgroup-per-tile kernel."""
    ops = host.ops()
    for M, N, K in ((512, 512, 8192), (1024, 1280, 4096), (512, 512, 8192)):
        say("split-K operator entry %dx%dx%d" % (M, N, K))
        a = orc.fill_int(M * K, "bf16", 71, -2, 2).reshape(M, K)
        b = orc.fill_int(K * N, "bf16", 72, -2, 2).reshape(K, N)
        bias = orc.fill_normal(N, "f32", 73, 0.0, 0.1)
        d_a, d_b, d_bias = stream.to_device(a), stream.to_device(b), stream.to_device(bias)
        d_o = stream.to_device(np.full((M, N), 0x7FC1, np.uint16))
        rc = ops.imexHipGemmBiasSiluBf16SplitK(stream.handle, int(d_a), int(d_b), int(d_bias), int(d_o), M, N, K)
        assert rc == 0, ops.imexHipOpsLastError()
        stream.wait()
        got = stream.from_device(d_o, (M, N), np.uint16)
        for p in (d_a, d_b, d_bias, d_o):
            stream.free(p)
        # integer operands: the f32 sums are exact in any order, so the two kernels agree bit for bit
        assert np.array_equal(got, host.gemm_bias_silu(stream, a, b, bias)), (M, N, K)
    assert ops.imexHipGemmBiasSiluBf16SplitK(None, None, None, None, None, 256, 256, 64) == -1
    assert b"queue" in ops.imexHipOpsLastError()


def test_gemm_reference_bias_kernel_4096(host, orc, stream):
    """WG/gemm_4kx4kx4k_f16_f16_f32_bias.mlir:77-116: kernel arguments (bias, C, A, B), grid 16 x 16,
    C = bias[n] + (C + A.B); checked as the test itself does (:160-172): the f32 GEMM onto the initial C,
    then C_ref[i,j] += bias[j].  The initial C is not zero here, so the accumulate is visible."""
    M = N = K = 4096
    a = orc.fill_uniform(M * K, "f16", 61, -0.5, 0.5).reshape(M, K)
    b = orc.fill_uniform(K * N, "f16", 62, -0.5, 0.5).reshape(K, N)
    c0 = orc.fill_uniform(M * N, "f32", 63, -1.0, 1.0).reshape(M, N)
    bias = orc.fill_uniform(N, "f32", 64, -1.0, 1.0)
    d_bias, d_c, d_a, d_b = (stream.to_device(t) for t in (bias, c0, a, b))
    try:
        _launch_raw(host, stream, "imex_gemm_4kx4kx4k_f16_f16_f32_bias", [d_bias, d_c, d_a, d_b], (16, 16, 1))
        got = stream.from_device(d_c, (M, N), np.float32)
        assert np.array_equal(stream.from_device(d_bias, (N,), np.float32), bias)
    finally:
        for p in (d_bias, d_c, d_a, d_b):
            stream.free(p)
    rows = STRIDED_ROWS_4096
    # oracle: the i-k-j loop accumulates onto C0's rows, then the bias loop
    ref = orc.bias_add_rows(orc.gemm_rows(a, b, rows, "f16", c0_rows=c0[rows]), bias)
    err = np.max(np.abs(got[rows] - ref)) / np.max(np.abs(ref))
    say("bias gemm 4096^3: max|d|/max|ref| = %.3e over %d rows" % (err, rows.size))
    assert err <= 5e-3
    assert orc.allclose_f32(got[rows], ref)  # the reference's own check (atol 1e-4, rtol 1e-3)
    # every column: 1^T C = (1^T A) B + 1^T C0 + M bias[n], in f64
    want = (_column_checksum_f64(orc.half_to_float(a), orc.half_to_float(b)) + c0.sum(axis=0, dtype=np.float64)
            + M * bias.astype(np.float64))
    assert np.max(np.abs(got.sum(axis=0, dtype=np.float64) - want)) <= 1e-3 * np.max(np.abs(want)) + 0.05
    # and every element against the accumulate kernel plus the bias (two roundings apart at most)
    acc = host.gemm(stream, a, b, c=c0, ab_dtype="f16")
    assert np.max(np.abs(got - (acc + bias[None, :]))) <= 1e-5


@pytest.mark.parametrize("dtype,M,N,K", [("bf16", 512, 512, 96), ("bf16", 300, 520, 1024), ("f16", 768, 256, 4096)])
def test_gemm_tiled_accumulate_integers_exact(host, orc, stream, dtype, M, N, K):
    """C += A.B on the MFMA path with integer operands and an integer C0: exact in any order."""
    a = orc.fill_int(M * K, dtype, 41, -4, 4).reshape(M, K)
    b = orc.fill_int(K * N, dtype, 42, -4, 4).reshape(K, N)
    c0 = orc.fill_int(M * N, "f32", 43, -1000, 1000).reshape(M, N)
    want = orc.to_float(a, dtype).astype(np.int64) @ orc.to_float(b, dtype).astype(np.int64) + c0.astype(np.int64)
    got = host.gemm(stream, a, b, c=c0, ab_dtype=dtype)
    assert np.array_equal(got.astype(np.int64), want)


def test_gemm_f16_output_4096(host, orc, stream):
    """WG/gemm_4kx4kx4k_f16_f16_f16.mlir at its own size: f32 accumulation, one rounding to f16."""
    M = N = K = 4096
    a = orc.fill_uniform(M * K, "f16", 65, -0.5, 0.5).reshape(M, K)
    b = orc.fill_uniform(K * N, "f16", 66, -0.5, 0.5).reshape(K, N)
    got = orc.half_to_float(host.gemm(stream, a, b, ab_dtype="f16", out_dtype="f16"))
    rows = STRIDED_ROWS_4096
    ref = orc.half_to_float(orc.float_to_half(orc.gemm_rows(a, b, rows, "f16")))
    assert gemm_close(got[rows], ref)
    want = _column_checksum_f64(orc.half_to_float(a), orc.half_to_float(b))
    # 4096 roundings to f16 per column, each below 2^-11 relative
    assert np.max(np.abs(got.sum(axis=0, dtype=np.float64) - want)) <= 2e-3 * np.max(np.abs(want)) + 0.5


def test_gemm_f16_output_variant(host, orc, stream):
    M, N, K = 512, 256, 256
    a = orc.fill_uniform(M * K, "f16", 8, -1, 1).reshape(M, K)
    b = orc.fill_uniform(K * N, "f16", 9, -1, 1).reshape(K, N)
    got = orc.half_to_float(host.gemm(stream, a, b, ab_dtype="f16", out_dtype="f16"))
    ref = orc.gemm(a, b, "f16", out_round="f16")
    assert gemm_close(got, ref)


# ==================== MFMA ceiling measurement kernel ======================
def _ceiling_lds_f16(workgroup, mode):
    """The f16 operands imex_mfma_lds_ceiling_f16 writes into LDS, as (4096 slots, 8)."""
    with np.errstate(over="ignore"):
        i = np.arange(16384, dtype=np.uint32)
        x = (i + np.uint32(workgroup * 7919)) * np.uint32(2654435761)
        x ^= x >> np.uint32(15)
        x *= np.uint32(2246822519)
        x ^= x >> np.uint32(13)
    if mode == 2:
        lo = (x & np.uint32(0x83ff)) | (((x >> np.uint32(10)) % np.uint32(15)) << np.uint32(10))
        hi = ((x >> np.uint32(16)) & np.uint32(0x83ff)) | (((x >> np.uint32(26)) % np.uint32(15)) << np.uint32(10))
    else:
        half = lambda h: (h.astype(np.float32) * np.float32(1.0 / 32768.0) - np.float32(1.0)).astype(np.float16).view(np.uint16).astype(np.uint32)
        lo, hi = half(x & np.uint32(0xffff)), half(x >> np.uint32(16))
    words = lo | (hi << np.uint32(16))
    return words.view(np.uint16).view(np.float16).astype(np.float64).reshape(4096, 8)


@pytest.mark.parametrize("mode", [0, 2])
def test_mfma_ceiling_kernel_computes_what_it_says(host, stream, mode):
    """No oracle and no reference counterpart: the expected sums follow from the published
    operand / accumulator lane layout of MFMA 16x16x32 (A[m = l%16][k = 8(l/16)..+8],
    B likewise in n, C[4(l/16) + r][l%16] in register r), in f64."""
    iters, groups = 5, 3
    say("mfma ceiling probe: %d workgroups x %d steps" % (groups, iters))
    got = host.mfma_lds_ceiling(stream, groups, iters, mode=mode)
    assert got.shape == (groups, 512)
    l = np.arange(64)
    rows = 4 * (l[:, None] // 16) + np.arange(4)[None, :]                      # [lane, r]
    for g in range(groups):
        slots = _ceiling_lds_f16(g, mode)
        for w in range(8):
            lane = w * 64 + l
            total = np.zeros(64)
            for it in range(iters):
                off = (it & 63) * 64
                frag = lambda base: slots[(lane + off + base) & 4095]          # [64 lanes, 8 k]
                def tile(f):                                                     # -> [16, 32]
                    t = np.zeros((16, 32))
                    for k8 in range(4):
                        t[:, 8 * k8:8 * k8 + 8] = f[16 * k8:16 * k8 + 16]
                    return t
                for i in range(8):
                    A = tile(frag(i * 256))
                    for j in range(4):
                        Bt = tile(frag(2048 + j * 256))                          # [n, k]
                        Cm = A @ Bt.T
                        total += Cm[rows, (l % 16)[:, None]].sum(axis=1)
            want = total
            have = got[g, w * 64:(w + 1) * 64].astype(np.float64)
            assert np.all(np.abs(have - want) <= 1e-4 * np.abs(want).max() + 1e-4), (g, w)
    assert not np.any(host.mfma_lds_ceiling(stream, 2, 7, mode=1))
    assert host.mfma_lds_ceiling(stream, 1, 0).shape == (1, 512) and not np.any(host.mfma_lds_ceiling(stream, 1, 0))
