"""Pins the CPU oracle: reference golden vectors, closed forms, exhaustive
conversion checks, and the reference's own statistics code (oracle/_ref)."""
import json
import math
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_vectors.json")) as f:
    GOLD = json.load(f)


def arr(v, shape=None):
    a = np.asarray(v, np.float32)
    return a.reshape(shape) if shape else a


# ---- generators ---------------------------------------------------------------
def test_mt19937_known_answer(orc):
    # [rand.predef]: the 10000th consecutive invocation of a default-constructed
    # std::mt19937 (seed 5489) produces 4123659995.
    assert orc.mt19937_raw(5489, 10000)[-1] == 4123659995


def test_uniform_matches_definition(orc):
    raw = orc.mt19937_raw(20241, 64)
    want = np.array([np.float32(-1.0 + 2.0 * ((w >> 8) / 16777216.0)) for w in raw], np.float32)
    got = orc.fill_uniform(64, "f32", 20241, -1.0, 1.0)
    assert np.array_equal(got, want)
    assert got.min() >= -1.0 and got.max() < 1.0


def test_normal_moments_and_definition(orc):
    x = orc.fill_normal(200000, "f32", 20242, 0.0, 2.0)
    assert abs(float(x.mean())) < 0.02 and abs(float(x.std()) - 2.0) < 0.02
    w = orc.mt19937_raw(20242, 2)
    u1, u2 = ((w[0] >> 8) + 1) / 16777216.0, (w[1] >> 8) / 16777216.0
    r = math.sqrt(-2.0 * math.log(u1))
    assert x[0] == np.float32(2.0 * r * math.cos(2 * math.pi * u2))
    assert x[1] == np.float32(2.0 * r * math.sin(2 * math.pi * u2))


def test_bits_have_no_nan(orc):
    f = orc.fill_bits(100000, "f32", 20245).view(np.float32)
    assert not np.isnan(f).any()
    h = orc.fill_bits(100000, "f16", 1).view(np.float16)
    assert not np.isnan(h).any()
    b = orc.fill_bits(100000, "bf16", 20244)
    assert not np.isnan(orc.bfloat_to_float(b)).any()
    assert len(np.unique(b)) > 30000  # covers the 16-bit space, infinities included


# ---- conversions ----------------------------------------------------------------
def test_half_to_float_exhaustive(orc):
    h = np.arange(65536, dtype=np.uint16)
    got = orc.half_to_float(h)
    want = h.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_bfloat_to_float_exhaustive(orc):
    b = np.arange(65536, dtype=np.uint16)
    assert np.array_equal(orc.bfloat_to_float(b).view(np.uint32), b.astype(np.uint32) << 16)


def test_float_to_half_rne(orc):
    rng = np.random.default_rng(0)
    bits = rng.integers(0, 2 ** 32, 2_000_000, dtype=np.uint64).astype(np.uint32)
    # add every half value, every midpoint between adjacent halves, and neighbours
    h = np.arange(0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mid = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)
    extra = np.concatenate([h, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)),
                            -mid, np.array([65504, 65519.99, 65520, 1e9, np.inf, -np.inf, 0.0, -0.0], np.float32)])
    f = np.concatenate([bits.view(np.float32), extra])
    f = f[~np.isnan(f)]
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.float_to_half(f), want)
    assert orc.float_to_half(np.array([np.nan], np.float32))[0] & 0x7fff == 0x7e00


def test_float_to_bfloat_rne(orc):
    rng = np.random.default_rng(1)
    f = rng.integers(0, 2 ** 32, 1_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    f = f[~np.isnan(f)]
    u = f.view(np.uint32).astype(np.uint64)
    want = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    assert np.array_equal(orc.float_to_bfloat(f), want)
    # values the reference's bf16 tests print after a round trip
    # (OpTest.GEMM_BF16_ACC_F32.mlir:13: 1.999510e-01 -> bf16 -> contributes 14.1006)
    assert orc.bfloat_to_float(orc.float_to_bfloat(np.array([0.199951], np.float32)))[0] == np.float32(0.2001953125)
    # exact ties go to even
    assert orc.float_to_bfloat(np.array([1.00390625], np.float32))[0] == 0x3f80
    assert orc.float_to_bfloat(np.array([1.01171875], np.float32))[0] == 0x3f82


# ---- relu ------------------------------------------------------------------------
def test_relu_golden(orc):
    g = GOLD["relu_f32_4x5_spirv"]
    assert np.array_equal(orc.relu_f32(arr(g["input"])), arr(g["expected"]))
    g = GOLD["relu_olt_f32_4x5"]
    assert np.allclose(orc.relu_olt_f32(arr(g["input"])), arr(g["expected"]), rtol=1e-6)
    # ugt and olt forms agree wherever the input is neither NaN nor -0.0
    assert np.array_equal(orc.relu_f32(arr(g["input"])), orc.relu_olt_f32(arr(g["input"])))


def test_relu_special_values(orc):
    x = np.array([0x7fc00001, 0xffc12345, 0x80000000, 0x00000000, 0x00000001, 0x80000001, 0x7f800000, 0xff800000],
                 np.uint32).view(np.float32)
    y = orc.relu_f32(x).view(np.uint32)
    # NaNs keep their payload, -0.0 -> +0.0, denormal+ kept, -inf -> 0
    assert list(y) == [0x7fc00001, 0xffc12345, 0, 0, 1, 0, 0x7f800000, 0]
    assert orc.relu_olt_f32(np.array([-0.0], np.float32)).view(np.uint32)[0] == 0x80000000


def test_relu_bf16_golden(orc):
    g = GOLD["relu_olt_bf16_4x5"]
    x = orc.float_to_bfloat(arr(g["input"]))
    y = orc.bfloat_to_float(orc.relu_16(x, "bf16"))
    # the printed values are 2-3 digit roundings of bf16 numbers
    assert np.allclose(y, arr(g["expected"]), rtol=4e-3)
    assert np.array_equal(y == 0, arr(g["expected"]) == 0)


# ---- silu ------------------------------------------------------------------------
def test_silu_closed_forms(orc):
    assert orc.silu_f32(np.array([0.0], np.float32))[0] == 0.0
    x = np.linspace(-20, 20, 4001).astype(np.float32)
    y = orc.silu_f32(x).astype(np.float64)
    exact = x.astype(np.float64) / (1.0 + np.exp(-x.astype(np.float64)))
    assert np.max(np.abs(y - exact) / np.maximum(np.abs(exact), 1e-30)) < 4e-7
    # silu(x) - silu(-x) == x up to rounding
    assert np.max(np.abs(y - y[::-1] - x)) < 4e-6
    # limits: large positive -> x, large negative -> -0.0 / tiny
    assert orc.silu_f32(np.array([100.0], np.float32))[0] == np.float32(100.0)
    assert abs(float(orc.silu_f32(np.array([-100.0], np.float32))[0])) < 1e-40
    # op order matters: the oracle multiplies sigmoid * x, with each step rounded
    xv = np.float32(1.3)
    e = np.float32(math.exp(-float(xv)))  # == expf for this input (checked below)
    s = np.float32(1.0) / (e + np.float32(1.0))
    assert orc.silu_f32(np.array([1.3], np.float32))[0] == np.float32(s * xv)


def test_libm_expf_vs_correctly_rounded(orc):
    """The host libm expf the oracle calls (as the reference's CPU lowering does) is
    within 1 ulp of the correctly rounded exponential over the whole finite range,
    and equal to it for almost every input."""
    import ctypes as C
    x = orc.fill_uniform(400000, "f32", 99, -87.0, 88.0)
    got = np.empty_like(x)
    orc.lib().oracle_expf_n(x.ctypes.data_as(C.c_void_p), got.ctypes.data_as(C.c_void_p), C.c_size_t(x.size))
    cr = np.exp(x.astype(np.float64)).astype(np.float32)
    ulps = orc.ulp_distance_f32(got, cr)
    assert np.max(ulps) <= 1
    assert np.count_nonzero(ulps) < x.size // 1000
    # the scalar correctly-rounded helper agrees with numpy's f64 exp on a sample
    sample = np.array([orc.lib().oracle_expf_cr(C.c_float(float(v))) for v in x[:500]], np.float32)
    assert np.array_equal(sample, cr[:500])
    assert got[0] == np.float32(math.exp(float(x[0]))) or ulps[0] == 1


def test_maximumf_closed_forms(orc):
    """arith.maximumf (WG/arith_maximumf.mlir:126): the reference's test draws random values in
    (-0.5, 0.5) and compares with its own CPU loop, so no vector exists; what the operation is
    fixes these: the larger value, +0 above -0 whichever side it is on, infinities ordered like
    numbers, NaN whenever either operand is NaN, and agreement with numpy's maximum elsewhere."""
    inf, nan = np.float32(np.inf), np.float32(np.nan)
    a = np.array([1.0, -2.0, 0.0, -0.0, -0.0, inf, -inf, nan, 3.0, nan, -1e-45, 5e-39], np.float32)
    b = np.array([2.0, -3.0, -0.0, 0.0, -0.0, 1.0, -1.0, 1.0, nan, nan, 1e-45, -5e-39], np.float32)
    got = orc.maximum_f32(a, b)
    want = np.array([2.0, -2.0, 0.0, 0.0, -0.0, inf, -1.0, nan, nan, nan, 1e-45, 5e-39], np.float32)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))  # bit patterns: signed zeros included
    x, y = orc.fill_uniform(10000, "f32", 5, -0.5, 0.5), orc.fill_uniform(10000, "f32", 6, -0.5, 0.5)
    assert np.array_equal(orc.maximum_f32(x, y), np.maximum(x, y))
    assert np.array_equal(orc.maximum_f32(x, y), orc.maximum_f32(y, x))


# ---- fused element-wise chains ------------------------------------------------------
def test_libm_logf_vs_correctly_rounded(orc):
    """The host libm logf the fused chains call is within 1 ulp of the correctly
    rounded logarithm over the positive range, subnormals included."""
    bits = np.concatenate([np.random.default_rng(7).integers(1, 0x7f800000, 400000, dtype=np.uint32),
                           np.array([1, 2, 0x007fffff, 0x00800000, 0x3f800000, 0x3f7fffff, 0x3f800001, 0x7f7fffff],
                                    np.uint32)])
    x = bits.view(np.float32)
    got = orc.logf(x)
    cr = np.log(x.astype(np.float64)).astype(np.float32)
    assert np.max(orc.ulp_distance_f32(got, cr)) <= 1
    special = orc.logf(np.array([0.0, -0.0, np.inf, -1.0, np.nan], np.float32))
    assert special[0] == -np.inf and special[1] == -np.inf and special[2] == np.inf
    assert np.isnan(special[3]) and np.isnan(special[4])


def test_fused_chains_closed_forms(orc):
    """No vector for these chains exists in the reference (its benchmarks feed the
    constants 3.3 and 1.0 and check nothing): the oracle is held against an f64
    evaluation, the benchmark's own constants, and the argument roles."""
    rng = np.random.default_rng(11)
    a = rng.uniform(0.05, 50.0, (37, 53)).astype(np.float32)
    b = rng.uniform(-9.0, 9.0, (37, 53)).astype(np.float32)
    got = orc.loop_fusion_f32(a, b).astype(np.float64)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    exact = (np.log(a64) + np.abs(b64)) - a64
    # three roundings of quantities no larger than max(|log a| + |b|, a) ~ 60
    assert np.max(np.abs(got - exact)) <= 3 * 60 * 2.0 ** -24
    # benchmark constants: (log 3.3 + |1.0|) - 3.3, op by op in f32
    t1 = np.float32(math.log(3.3000000953674316))  # logf is correctly rounded here (checked above to 1 ulp)
    want = np.float32(np.float32(t1 + np.float32(1.0)) - np.float32(3.3))
    one = orc.loop_fusion_f32(np.full(4, 3.3, np.float32), np.full(4, 1.0, np.float32))
    assert np.all(np.abs(one - want) <= np.spacing(np.float32(1.2)))
    # log applies to the FIRST argument, abs to the second: swapping them changes the result
    assert orc.loop_fusion_f32(np.float32([2.0]), np.float32([-8.0]))[0] == np.float32(np.float32(math.log(2.0)) + 8.0) - np.float32(2.0)
    # input fusion: log of the SECOND argument, abs of the first, column sums in row order
    col = orc.input_fusion_f32(b, a).astype(np.float64)   # a > 0 goes under the log
    exact_col = (np.log(a64) + np.abs(b64)).sum(axis=0)
    assert col.shape == (53,)
    assert np.max(np.abs(col - exact_col)) <= 37 * 2 * 400 * 2.0 ** -24
    # order of the adds: row order, starting from +0.0 (reproduced with numpy f32 scalars)
    t = (orc.logf(a) + np.abs(b)).astype(np.float32)
    acc = np.zeros(53, np.float32)
    for i in range(37):
        acc = (acc + t[i]).astype(np.float32)
    assert np.array_equal(orc.input_fusion_f32(b, a), acc)
    # benchmark constants: 512 rows of (log 1.0 + |3.3|) = 512 * 3.3f exactly representable sums? compare to the loop
    c = orc.input_fusion_f32(np.full((512, 8), 3.3, np.float32), np.full((512, 8), 1.0, np.float32))
    acc = np.float32(0.0)
    for _ in range(512):
        acc = np.float32(acc + np.float32(3.3))
    assert np.all(c == acc)


# ---- flash attention -----------------------------------------------------------------
def test_flash_attention_reference_closed_forms(orc):
    n_ctx, d = 256, 64
    f16 = lambda a: orc.from_float(np.asarray(a, np.float32), "f16")
    # the reference's own check input: every element 0.625 -> uniform softmax -> every output 0.625
    # (WG/flash_attention_fwd.mlir:481-485, checked there with allclose)
    x = f16(np.full((2 * n_ctx, d), 0.625))
    out = orc.flash_attention_rows(x, x, x, n_ctx, 0.5, np.arange(2 * n_ctx))
    assert np.all(orc.half_to_float(out) == 0.625)
    # K = 0: uniform probabilities 1/256 (exact in f16), output = f16(mean of V) per head
    rng = np.random.default_rng(5)
    q = f16(rng.uniform(-1, 1, (2 * n_ctx, d)))
    v = f16(rng.uniform(-1, 1, (2 * n_ctx, d)))
    out = orc.half_to_float(orc.flash_attention_rows(q, f16(np.zeros((2 * n_ctx, d))), v, n_ctx, 0.5, [0, 300]))
    vf = orc.half_to_float(v).astype(np.float64)
    assert np.max(np.abs(out[0] - vf[:n_ctx].mean(axis=0))) < 2e-3      # row 0 belongs to head 0
    assert np.max(np.abs(out[1] - vf[n_ctx:].mean(axis=0))) < 2e-3      # row 300 to head 1: heads do not mix
    # one dominant key: q = 8 e_0, key 77 = 8 e_0, others 0 -> score 32 at key 77 -> output = V[77]
    qh = np.zeros((n_ctx, d), np.float32); qh[:, 0] = 8.0
    kh = np.zeros((n_ctx, d), np.float32); kh[77, 0] = 8.0
    v1 = f16(rng.uniform(-1, 1, (n_ctx, d)))
    out = orc.flash_attention_rows(f16(qh), f16(kh), v1, n_ctx, 1.0, [5])
    assert np.max(np.abs(orc.half_to_float(out)[0] - orc.half_to_float(v1)[77])) < 1e-3
    # general case against an f64 evaluation
    k = f16(rng.uniform(-1, 1, (2 * n_ctx, d)))
    rows = np.array([0, 17, 255, 256, 511])
    got = orc.half_to_float(orc.flash_attention_rows(q, k, v, n_ctx, 0.5, rows)).astype(np.float64)
    qf, kf = orc.half_to_float(q).astype(np.float64), orc.half_to_float(k).astype(np.float64)
    for i, r in enumerate(rows):
        h = r // n_ctx
        s = 0.5 * kf[h * n_ctx:(h + 1) * n_ctx] @ qf[r]
        p = np.exp(s - s.max()); p /= p.sum()
        assert np.max(np.abs(got[i] - p @ vf[h * n_ctx:(h + 1) * n_ctx])) < 1e-3


# ---- softmax ---------------------------------------------------------------------
@pytest.mark.parametrize("key", ["softmax_f32_10x20", "softmax_f32_10x20_spirv"])
def test_softmax_golden(orc, key):
    g = GOLD[key]
    x = arr(g["input"], g["shape"])
    want = arr(g["expected"], g["shape"])
    for three_pass in (False, True):
        got = orc.softmax_f32(x, three_pass)
        assert np.max(np.abs(got - want) / want) < 2e-5  # six printed digits
        assert orc.allclose_f32(got, want)


def test_softmax_invariants(orc):
    x = orc.fill_normal(64 * 1024, "f32", 5, 0.0, 2.0).reshape(64, 1024)
    y = orc.softmax_f32(x)
    assert np.max(np.abs(y.sum(axis=1, dtype=np.float64) - 1.0)) < 1e-5
    # shift invariance by a power of two is exact when no rounding occurs in x + c
    xi = np.round(x * 8) / 8
    assert np.array_equal(orc.softmax_f32(xi), orc.softmax_f32((xi + 16).astype(np.float32)))
    # an all-equal row of 1024 gives exactly 2^-10
    eq = np.full((2, 1024), 3.3, np.float32)
    assert np.all(orc.softmax_f32(eq) == np.float32(2.0 ** -10))
    h = orc.softmax_16(orc.float_to_half(eq), "f16")
    assert np.all(h == 0x1400)  # 2^-10 in f16
    # against float64 evaluation
    xd = x.astype(np.float64)
    ed = np.exp(xd - xd.max(axis=1, keepdims=True))
    assert np.max(np.abs(y - ed / ed.sum(axis=1, keepdims=True)) / y) < 2e-5


# ---- reductions --------------------------------------------------------------------
def test_sum_golden(orc):
    g = GOLD["sum_f32_10x20"]
    x = arr(g["input"], g["shape"])
    assert orc.sum_all_f32(x) == g["expected"][0] == 2100.0
    assert np.array_equal(orc.rowsum_f32(x), np.full(10, 210.0, np.float32))
    assert np.array_equal(orc.reduce_outer_f32(x), np.arange(1, 21, dtype=np.float32) * 10)


def test_wg_reduction_vectors(orc):
    g = GOLD["wg_reduction_rows"]
    x = np.repeat(np.arange(g["rows"], dtype=np.float32)[:, None], g["cols"], axis=1)
    assert list(orc.rowsum_f32(x)) == g["expected"]
    # reduction_2D_1D_cross_sg_intra_lane.mlir:105: sum of 0..31 down a column = 496
    col = np.repeat(np.arange(32, dtype=np.float32)[:, None], 32, axis=1)
    assert np.all(orc.reduce_outer_f32(col) == 496.0)
    # reduction_3D_1D_*:91: 256*256 ones = 65536
    assert orc.rowsum_f32(np.ones((1, 65536), np.float32))[0] == 65536.0


def test_rowsum_is_sequential(orc):
    # 2^24 + 1 + 1 ... stays at 2^24 when added left to right in f32
    x = np.concatenate([[np.float32(2 ** 24)], np.ones(100, np.float32)])[None, :]
    assert orc.rowsum_f32(x)[0] == np.float32(2 ** 24)
    assert orc.rowsum_f32(x[:, ::-1].copy())[0] == np.float32(2 ** 24 + 100)
    assert orc.rowsum_f32(np.ones((1, 3), np.float32), init=2.5)[0] == 5.5


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_sixteen_bit_silu_and_outer_reduce_are_widen_compute_round(orc, dtype):
    """The 16-bit forms are defined as: widen exactly, the f32 operation, one rounding.  Pinned by
    composing the f32 oracle with the (exhaustively checked) conversions, and by exact cases."""
    x = orc.fill_uniform(5000, dtype, 301, -8.0, 8.0)
    assert np.array_equal(orc.silu_16(x, dtype), orc.from_float(orc.silu_f32(orc.to_float(x, dtype)), dtype))
    assert orc.to_float(orc.silu_16(orc.from_float(np.zeros(3, np.float32), dtype), dtype), dtype).tolist() == [0, 0, 0]
    m = orc.fill_int(7 * 300, dtype, 302, -8, 8).reshape(7, 300)
    want = 0.5 + orc.to_float(m, dtype).sum(axis=0, dtype=np.float64)          # integers: exact in any order
    assert np.array_equal(orc.to_float(orc.reduce_outer_16(m, dtype, init=0.5), dtype), want.astype(np.float32))
    r = orc.fill_uniform(9 * 257, dtype, 303, -1.0, 1.0).reshape(9, 257)
    assert np.array_equal(orc.reduce_outer_16(r, dtype, init=0.25),
                          orc.from_float(orc.reduce_outer_f32(orc.to_float(r, dtype), init=0.25), dtype))


def test_rowmean_closed_forms(orc):
    """WG/reduction_4D_3D_mean_intra_sg_intra_lane.mlir:115-127: sequential sum, then one division.
    Pinned by what arithmetic fixes: a constant dyadic row of a power-of-two length returns the constant
    exactly; integers 0..63 average 31.5; the sum is sequential (2^24 absorbs ones added after it,
    not before); the division is by the row length, not a multiplication by a rounded reciprocal."""
    assert np.array_equal(orc.rowmean_f32(np.full((3, 64), 0.625, np.float32)), np.full(3, np.float32(0.625)))
    assert orc.rowmean_f32(np.arange(64, dtype=np.float32)[None, :])[0] == np.float32(31.5)
    big = np.concatenate([[np.float32(2 ** 24)], np.ones(63, np.float32)])[None, :]
    assert orc.rowmean_f32(big)[0] == np.float32(2 ** 24) / np.float32(64)
    assert orc.rowmean_f32(big[:, ::-1].copy())[0] == np.float32(2 ** 24 + 63) / np.float32(64)
    x = np.array([[1.0, 2.0, 4.0]], np.float32)   # 7 / 3 correctly rounded differs from 7 * fl(1/3)
    assert orc.rowmean_f32(x)[0] == np.float32(7.0) / np.float32(3.0)
    assert np.float32(7.0) / np.float32(3.0) != np.float32(7.0) * (np.float32(1.0) / np.float32(3.0))
    y = np.random.default_rng(5).uniform(-1, 1, (24, 64)).astype(np.float32)
    assert np.array_equal(orc.rowmean_f32(y), orc.rowsum_f32(y) / np.float32(64))


# ---- transpose ---------------------------------------------------------------------
def test_transpose_golden(orc):
    g = GOLD["transpose_f32_10x20"]
    x = arr(g["input"], g["shape"])
    assert np.array_equal(orc.transpose2d(x), arr(g["expected"], [20, 10]))
    g = GOLD["transpose_bf16_10x20"]
    xb = orc.float_to_bfloat(arr(g["input"], g["shape"]))
    assert np.array_equal(orc.bfloat_to_float(orc.transpose2d(xb)), arr(g["expected"], [20, 10]))


def test_transpose_closed_forms(orc):
    x = np.arange(37 * 53, dtype=np.uint32).reshape(37, 53)
    assert np.array_equal(orc.transpose2d(x), x.T)
    assert np.array_equal(orc.transpose2d(orc.transpose2d(x)), x)
    h = np.arange(17 * 9, dtype=np.uint16).reshape(17, 9)
    assert np.array_equal(orc.transpose2d(h), h.T)
    t = np.arange(5 * 7 * 3, dtype=np.uint32).reshape(5, 7, 3)
    assert np.array_equal(orc.transpose3d(t), t.transpose(2, 1, 0))


# ---- GEMM --------------------------------------------------------------------------
def test_gemm_golden(orc):
    g = GOLD["gemm_f32_3x3"]
    c = orc.gemm(arr(g["A"], [3, 3]), arr(g["B"], [3, 3]), "f32", c=arr(g["C0"], [3, 3]))
    assert np.allclose(c.ravel(), g["expected"], rtol=2e-6)
    g = GOLD["gemm_f16_acc_f32_3x3"]
    a, b = orc.float_to_half(arr(g["A"], [3, 3])), orc.float_to_half(arr(g["B"], [3, 3]))
    c = orc.gemm(a, b, "f16", c=arr(g["C0"], [3, 3]))
    assert np.max(np.abs(c.ravel() - arr(g["expected"]))) < 6e-5  # printed to 1e-4
    assert orc.allclose_f32(c, arr(g["expected"], [3, 3]))
    g = GOLD["gemm_bf16_acc_f32_3x3"]
    a, b = orc.float_to_bfloat(arr(g["A"], [3, 3])), orc.float_to_bfloat(arr(g["B"], [3, 3]))
    c = orc.gemm(a, b, "bf16", c=arr(g["C0"], [3, 3]))
    assert np.max(np.abs(c.ravel() - arr(g["expected"]))) < 6e-5
    g = GOLD["dot_f16_acc_f32_8x16x32"]
    a = orc.float_to_half(np.full((g["M"], g["K"]), g["A_fill"], np.float32))
    b = orc.float_to_half(np.full((g["K"], g["N"]), g["B_fill"], np.float32))
    assert np.all(orc.gemm(a, b, "f16", out_round="f16") == g["expected_fill"])


def test_gemm_closed_forms(orc):
    # B = I  =>  C = A ; A[i,j] = j (gemm_4kx4kx4k_f16_f16_f32.mlir:109-138)
    K = 96
    a = orc.float_to_half(np.tile(np.arange(K, dtype=np.float32), (5, 1)))
    eye = orc.float_to_half(np.eye(K, dtype=np.float32))
    assert np.array_equal(orc.gemm(a, eye, "f16"), orc.half_to_float(a))
    # small integers: exact, so it must equal the integer matmul whatever the order
    ai = orc.fill_int(40 * 200, "bf16", 3, -4, 4).reshape(40, 200)
    bi = orc.fill_int(200 * 24, "bf16", 4, -4, 4).reshape(200, 24)
    want = orc.bfloat_to_float(ai).astype(np.int64) @ orc.bfloat_to_float(bi).astype(np.int64)
    assert np.array_equal(orc.gemm(ai, bi, "bf16").astype(np.int64), want)
    # the row-subset entry point is the same arithmetic
    a = orc.fill_uniform(64 * 128, "f16", 7, -1, 1).reshape(64, 128)
    b = orc.fill_uniform(128 * 32, "f16", 8, -1, 1).reshape(128, 32)
    full = orc.gemm(a, b, "f16")
    rows = np.array([0, 5, 63])
    assert np.array_equal(orc.gemm_rows(a, b, rows, "f16"), full[rows])
    # ... also onto a non-zero C (the reference loads C as the initial accumulator)
    c0 = orc.fill_uniform(64 * 32, "f32", 9, -1, 1).reshape(64, 32)
    assert np.array_equal(orc.gemm_rows(a, b, rows, "f16", c0_rows=c0[rows]), orc.gemm(a, b, "f16", c=c0)[rows])
    assert orc.gemm(a, b, "f16", c=c0)[3, 9] != full[3, 9]
    # k-ascending f32 accumulation with a rounded product: compare with a literal loop
    af, bf = orc.half_to_float(a), orc.half_to_float(b)
    acc = np.float32(0)
    for k in range(128):
        acc = np.float32(acc + np.float32(af[3, k] * bf[k, 9]))
    assert full[3, 9] == acc


def test_bias_and_epilogue(orc):
    c = np.arange(12, dtype=np.float32).reshape(3, 4)
    bias = np.array([10, 20, 30, 40], np.float32)
    assert np.array_equal(orc.bias_add_rows(c, bias), c + bias[None, :])
    acc = orc.fill_normal(8 * 16, "f32", 11, 0, 3).reshape(8, 16)
    b = orc.fill_normal(16, "f32", 12, 0, 0.1)
    got = orc.bias_silu_bf16(acc, b)
    want = orc.float_to_bfloat(orc.silu_f32((acc + b[None, :]).astype(np.float32)))
    assert np.array_equal(got, want)


# ---- allclose / max error -----------------------------------------------------------
def test_allclose_formula(orc):
    ref = np.array([1.0, 100.0, 0.0], np.float32)
    assert orc.allclose_f32(ref + np.array([1e-3, 0.1, 9e-5], np.float32), ref)
    assert not orc.allclose_f32(ref + np.array([1.2e-3, 0, 0], np.float32), ref)
    assert not orc.allclose_f32(ref + np.array([0, 0, 1.1e-4], np.float32), ref)
    # asymmetric in its arguments: the tolerance scales with the second one
    assert orc.allclose_f32(np.array([0.0], np.float32), np.array([1e-4], np.float32))
    ma, mr = orc.max_error_f32(np.array([1.0, 2.0], np.float32), np.array([1.5, 2.0], np.float32))
    assert ma == 0.5 and abs(mr - 0.5 / 1.5) < 1e-12


# ---- statistics -----------------------------------------------------------------------
def test_stats_closed_forms(orc):
    v = np.array([3, 1, 4, 1, 5, 9, 2, 6, 5, 3], np.float32)
    assert orc.stat("min", v) == 1 and orc.stat("max", v) == 9
    assert orc.stat("avg", v) == np.float32(3.9)
    assert orc.stat("median_textbook", v) == 3.5
    assert abs(orc.stat("variance", v) - float(np.var(v))) < 1e-5
    assert abs(orc.stat("stddev", v) - float(np.std(v))) < 1e-5
    s = np.sort(v)
    assert orc.stat("p95", v) == s[9] and orc.stat("p5", v) == s[0]
    assert orc.stat("middle_third_avg", v) == np.float32(s[3:7].sum() / 4)
    assert orc.stat("median_reference", v) == (s[6] + s[5]) / 2  # pivot n/2+1: one past the middle


def test_stats_match_reference_build(orc):
    ref = orc.ref_stats()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    import ctypes as C
    rng = np.random.default_rng(5)
    for n in (3, 4, 5, 10, 99, 100, 1000):
        v = rng.random(n).astype(np.float32) * 3
        p = C.c_void_p(v.ctypes.data)
        pairs = [("min", "min"), ("max", "max"), ("avg", "avg"), ("median_reference", "median"),
                 ("stddev", "stddev"), ("variance", "variance"), ("p95", "p95"), ("p5", "p5"),
                 ("middle_third_avg", "middle_third_avg")]
        for mine, theirs in pairs:
            assert orc.stat(mine, v) == getattr(ref, "ref_stat_" + theirs)(p, n), (mine, n)
