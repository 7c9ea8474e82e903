"""numpy front end of the CPU oracle (oracle/liboracle.so) -- test infrastructure.

Used only by tests, the smoke check and the benchmark's cpu_baseline leg, as the
checker.  16-bit float tensors are uint16 bit patterns plus a dtype name.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(REPO, "oracle")
_LIB_PATH = os.path.join(ORACLE_DIR, "liboracle.so")
_REF_STATS_PATH = os.path.join(ORACLE_DIR, "_ref", "libimex_ref_stats.so")

DT = {"f32": 0, "f16": 1, "bf16": 2}
NP = {"f32": np.float32, "f16": np.uint16, "bf16": np.uint16}

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            subprocess.check_call(["make", "-C", ORACLE_DIR, "liboracle.so"])
        _lib = C.CDLL(_LIB_PATH)
        _lib.oracle_half_to_float.restype = C.c_float
        _lib.oracle_half_to_float.argtypes = [C.c_uint16]
        _lib.oracle_bfloat_to_float.restype = C.c_float
        _lib.oracle_bfloat_to_float.argtypes = [C.c_uint16]
        _lib.oracle_float_to_half.restype = C.c_uint16
        _lib.oracle_float_to_half.argtypes = [C.c_float]
        _lib.oracle_float_to_bfloat.restype = C.c_uint16
        _lib.oracle_float_to_bfloat.argtypes = [C.c_float]
        _lib.oracle_silu_scalar_f32.restype = C.c_float
        _lib.oracle_silu_scalar_f32.argtypes = [C.c_float]
        _lib.oracle_expf_cr.restype = C.c_float
        _lib.oracle_expf_cr.argtypes = [C.c_float]
        _lib.oracle_sum_all_f32.restype = C.c_float
        _lib.oracle_sum_all_f32.argtypes = [C.c_void_p, C.c_int64, C.c_float]
        _lib.oracle_allclose_f32.restype = C.c_int
        for name in ("min", "max", "avg", "median_textbook", "median_reference", "stddev", "variance", "p95", "p5",
                     "middle_third_avg"):
            fn = getattr(_lib, "oracle_stat_" + name)
            fn.restype = C.c_float
            fn.argtypes = [C.c_void_p, C.c_size_t]
        for name in ("relu_f32", "silu_f32", "softmax_f16", "rowsum_f32", "transpose2d", "gemm_rows", "mlp_rows"):
            getattr(_lib, "oracle_time_" + name).restype = C.c_double
    return _lib


def _p(a):
    return C.c_void_p(a.ctypes.data)


def _c(a, dtype=None):
    a = np.ascontiguousarray(a)
    if dtype is not None and a.dtype != dtype:
        a = a.astype(dtype)
    return a


# ---- conversions -------------------------------------------------------------
def half_to_float(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().oracle_half_to_float_n(_p(h), _p(out), C.c_size_t(h.size))
    return out


def bfloat_to_float(b):
    b = _c(b, np.uint16)
    out = np.empty(b.shape, np.float32)
    lib().oracle_bfloat_to_float_n(_p(b), _p(out), C.c_size_t(b.size))
    return out


def float_to_half(f):
    f = _c(f, np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().oracle_float_to_half_n(_p(f), _p(out), C.c_size_t(f.size))
    return out


def float_to_bfloat(f):
    f = _c(f, np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().oracle_float_to_bfloat_n(_p(f), _p(out), C.c_size_t(f.size))
    return out


def to_float(x, dtype):
    if dtype == "f32":
        return _c(x, np.float32)
    return half_to_float(x) if dtype == "f16" else bfloat_to_float(x)


def from_float(f, dtype):
    if dtype == "f32":
        return _c(f, np.float32)
    return float_to_half(f) if dtype == "f16" else float_to_bfloat(f)


# ---- generators ---------------------------------------------------------------
def mt19937_raw(seed, n):
    class G(C.Structure):
        _fields_ = [("mt", C.c_uint32 * 624), ("idx", C.c_int)]
    g = G()
    L = lib()
    L.oracle_mt_seed(C.byref(g), C.c_uint32(seed))
    L.oracle_mt_next.restype = C.c_uint32
    return [L.oracle_mt_next(C.byref(g)) for _ in range(n)]


def fill_uniform(n, dtype, seed, lo, hi):
    out = np.empty(n, NP[dtype])
    lib().oracle_fill_uniform(_p(out), C.c_size_t(n), DT[dtype], C.c_uint32(seed), C.c_double(lo), C.c_double(hi))
    return out


def fill_normal(n, dtype, seed, mu, sigma):
    out = np.empty(n, NP[dtype])
    lib().oracle_fill_normal(_p(out), C.c_size_t(n), DT[dtype], C.c_uint32(seed), C.c_double(mu), C.c_double(sigma))
    return out


def fill_bits(n, dtype, seed):
    out = np.empty(n, np.uint32 if dtype == "f32" else np.uint16)
    lib().oracle_fill_bits_no_nan(_p(out), C.c_size_t(n), DT[dtype], C.c_uint32(seed))
    return out


def fill_int(n, dtype, seed, lo, hi):
    out = np.empty(n, NP[dtype])
    lib().oracle_fill_int_uniform(_p(out), C.c_size_t(n), DT[dtype], C.c_uint32(seed), C.c_int(lo), C.c_int(hi))
    return out


# ---- ops ------------------------------------------------------------------------
def relu_f32(x):
    x = _c(x, np.float32)
    y = np.empty_like(x)
    lib().oracle_relu_f32(_p(x), _p(y), C.c_size_t(x.size))
    return y


def relu_olt_f32(x):
    x = _c(x, np.float32)
    y = np.empty_like(x)
    lib().oracle_relu_olt_f32(_p(x), _p(y), C.c_size_t(x.size))
    return y


def relu_16(x, dtype):
    x = _c(x, np.uint16)
    y = np.empty_like(x)
    lib().oracle_relu_16(_p(x), _p(y), C.c_size_t(x.size), DT[dtype])
    return y


def silu_f32(x):
    x = _c(x, np.float32)
    y = np.empty_like(x)
    lib().oracle_silu_f32(_p(x), _p(y), C.c_size_t(x.size))
    return y


def silu_16(x, dtype):
    x = _c(x, np.uint16)
    y = np.empty_like(x)
    lib().oracle_silu_16(_p(x), _p(y), C.c_size_t(x.size), DT[dtype])
    return y


def expf_n(x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().oracle_expf_n(_p(x), _p(out), C.c_size_t(x.size))
    return out


def maximum_f32(a, b):
    a, b = _c(a, np.float32), _c(b, np.float32)
    out = np.empty_like(a)
    lib().oracle_maximum_f32(_p(a), _p(b), _p(out), C.c_size_t(a.size))
    return out


def loop_fusion_f32(a, b):
    a, b = _c(a, np.float32), _c(b, np.float32)
    out = np.empty_like(a)
    lib().oracle_loop_fusion_f32(_p(a), _p(b), _p(out), C.c_size_t(a.size))
    return out


def input_fusion_f32(a, b):
    a, b = _c(a, np.float32), _c(b, np.float32)
    out = np.empty(a.shape[1], np.float32)
    lib().oracle_input_fusion_f32(_p(a), _p(b), _p(out), C.c_int64(a.shape[0]), C.c_int64(a.shape[1]))
    return out


def flash_attention_rows(q, k, v, n_ctx, sm_scale, rows):
    """f16 bit patterns [(ZH*n_ctx), d]; returns the f16 bit patterns of the listed rows."""
    q, k, v = _c(q, np.uint16), _c(k, np.uint16), _c(v, np.uint16)
    rows = _c(np.asarray(rows), np.int64)
    d = q.shape[1]
    out = np.empty((rows.size, d), np.uint16)
    lib().oracle_flash_attention_rows(_p(q), _p(k), _p(v), _p(out), C.c_int64(n_ctx), C.c_int64(d),
                                      C.c_float(sm_scale), _p(rows), C.c_int64(rows.size))
    return out


def logf(x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().oracle_logf_n(_p(x), _p(out), C.c_size_t(x.size))
    return out


def softmax_f32(x, three_pass=False):
    x = _c(x, np.float32)
    y = np.empty_like(x)
    fn = lib().oracle_softmax_3pass_f32 if three_pass else lib().oracle_softmax_f32
    fn(_p(x), _p(y), C.c_int64(x.shape[0]), C.c_int64(x.shape[1]))
    return y


def softmax_16(x, dtype):
    x = _c(x, np.uint16)
    y = np.empty_like(x)
    lib().oracle_softmax_16(_p(x), _p(y), C.c_int64(x.shape[0]), C.c_int64(x.shape[1]), DT[dtype])
    return y


def rowsum_f32(x, init=0.0):
    x = _c(x, np.float32)
    out = np.empty(x.shape[0], np.float32)
    lib().oracle_rowsum_f32(_p(x), _p(out), C.c_int64(x.shape[0]), C.c_int64(x.shape[1]), C.c_float(init))
    return out


def reduce_outer_16(x, dtype, init=0.0):
    x = _c(x, np.uint16)
    outer = x.shape[0]
    inner = int(np.prod(x.shape[1:]))
    out = np.empty(x.shape[1:], np.uint16)
    lib().oracle_reduce_outer_16(_p(x), _p(out), C.c_int64(outer), C.c_int64(inner), C.c_float(init), DT[dtype])
    return out


def rowmean_f32(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape[0], np.float32)
    lib().oracle_rowmean_f32(_p(x), _p(out), C.c_int64(x.shape[0]), C.c_int64(x.shape[1]))
    return out


def reduce_outer_f32(x, init=0.0):
    x = _c(x, np.float32)
    outer = x.shape[0]
    inner = int(np.prod(x.shape[1:]))
    out = np.empty(x.shape[1:], np.float32)
    lib().oracle_reduce_outer_f32(_p(x), _p(out), C.c_int64(outer), C.c_int64(inner), C.c_float(init))
    return out


def sum_all_f32(x, init=0.0):
    x = _c(x, np.float32)
    return float(lib().oracle_sum_all_f32(_p(x), C.c_int64(x.size), C.c_float(init)))


def transpose2d(x):
    x = _c(x)
    out = np.empty((x.shape[1], x.shape[0]), x.dtype)
    lib().oracle_transpose2d(_p(x), _p(out), C.c_int64(x.shape[0]), C.c_int64(x.shape[1]), C.c_int(x.dtype.itemsize))
    return out


def transpose3d(x):
    x = _c(x)
    d0, d1, d2 = x.shape
    out = np.empty((d2, d1, d0), x.dtype)
    lib().oracle_transpose3d(_p(x), _p(out), C.c_int64(d0), C.c_int64(d1), C.c_int64(d2), C.c_int(x.dtype.itemsize))
    return out


def gemm(a, b, ab_dtype, c=None, out_round="f32"):
    a, b = _c(a), _c(b)
    M, K = a.shape
    N = b.shape[1]
    out = np.zeros((M, N), np.float32) if c is None else _c(c, np.float32).copy()
    lib().oracle_gemm(_p(a), _p(b), _p(out), C.c_int64(M), C.c_int64(N), C.c_int64(K), DT[ab_dtype], DT[out_round])
    return out


def gemm_rows(a, b, rows, ab_dtype, c0_rows=None):
    """Rows `rows` of C0 + A.B (the i-k-j loop accumulates onto what C holds); C0 = 0 when not given."""
    a, b = _c(a), _c(b)
    K = a.shape[1]
    N = b.shape[1]
    rows = np.ascontiguousarray(rows, np.int64)
    out = np.zeros((rows.size, N), np.float32) if c0_rows is None else _c(c0_rows, np.float32).copy()
    assert out.shape == (rows.size, N)
    lib().oracle_gemm_rows(_p(a), _p(b), _p(out), _p(rows), C.c_int64(rows.size), C.c_int64(N), C.c_int64(K),
                           DT[ab_dtype])
    return out


def bias_add_rows(c, bias):
    c = _c(c, np.float32).copy()
    bias = _c(bias, np.float32)
    lib().oracle_bias_add_rows(_p(c), _p(bias), C.c_int64(c.shape[0]), C.c_int64(c.shape[1]))
    return c


def bias_silu_bf16(acc, bias):
    acc = _c(acc, np.float32)
    bias = _c(bias, np.float32)
    out = np.empty(acc.shape, np.uint16)
    lib().oracle_bias_silu_bf16(_p(acc), _p(bias), _p(out), C.c_int64(acc.shape[0]), C.c_int64(acc.shape[1]))
    return out


# ---- checking helpers ----------------------------------------------------------
def allclose_f32(a, ref):
    a, ref = _c(a, np.float32), _c(ref, np.float32)
    return bool(lib().oracle_allclose_f32(_p(a), _p(ref), C.c_size_t(a.size)))


def max_error_f32(a, b):
    a, b = _c(a, np.float32), _c(b, np.float32)
    ma, mr = C.c_double(0), C.c_double(0)
    lib().oracle_max_error_f32(_p(a), _p(b), C.c_size_t(a.size), C.byref(ma), C.byref(mr))
    return ma.value, mr.value


def stat(name, values):
    v = _c(values, np.float32)
    return float(getattr(lib(), "oracle_stat_" + name)(_p(v), C.c_size_t(v.size)))


def ref_stats():
    """The reference's own ExecutionEngineUtils.cpp, if oracle/_ref was built."""
    if not os.path.exists(_REF_STATS_PATH):
        return None
    r = C.CDLL(_REF_STATS_PATH)
    for name in ("min", "max", "avg", "median", "stddev", "variance", "p95", "p5", "middle_third_avg"):
        fn = getattr(r, "ref_stat_" + name)
        fn.restype = C.c_float
        fn.argtypes = [C.c_void_p, C.c_size_t]
    return r


def ulp_distance_f32(a, b):
    """Distance in units in the last place between two f32 arrays (same-sign ordering)."""
    def key(x):
        u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.int64)
        return np.where(u & 0x80000000, -(u & 0x7fffffff), u)
    return np.abs(key(a) - key(b))


# ---- CPU-baseline timing legs ---------------------------------------------------
def time_relu_f32(x, warmup, runs):
    x = _c(x, np.float32)
    return lib().oracle_time_relu_f32(_p(x), C.c_size_t(x.size), C.c_int(warmup), C.c_int(runs))


def time_silu_f32(x, warmup, runs):
    x = _c(x, np.float32)
    return lib().oracle_time_silu_f32(_p(x), C.c_size_t(x.size), C.c_int(warmup), C.c_int(runs))


def time_softmax_f16(x, warmup, runs):
    x = _c(x, np.uint16)
    return lib().oracle_time_softmax_f16(_p(x), C.c_int64(x.shape[0]), C.c_int64(x.shape[1]), C.c_int(warmup),
                                         C.c_int(runs))


def time_rowsum_f32(x, warmup, runs):
    x = _c(x, np.float32)
    return lib().oracle_time_rowsum_f32(_p(x), C.c_int64(x.shape[0]), C.c_int64(x.shape[1]), C.c_int(warmup),
                                        C.c_int(runs))


def time_transpose2d(x, warmup, runs):
    x = _c(x)
    return lib().oracle_time_transpose2d(_p(x), C.c_int64(x.shape[0]), C.c_int64(x.shape[1]),
                                         C.c_int(x.dtype.itemsize), C.c_int(warmup), C.c_int(runs))


def time_gemm_rows(a, b, nrows, ab_dtype):
    a, b = _c(a), _c(b)
    return lib().oracle_time_gemm_rows(_p(a), _p(b), C.c_int64(nrows), C.c_int64(b.shape[1]), C.c_int64(a.shape[1]),
                                       DT[ab_dtype])


def time_mlp_rows(a, b, bias, nrows):
    """ms for the first `nrows` rows of bf16(silu(A.B + bias)): the GEMM loop and the epilogue."""
    a, b, bias = _c(a), _c(b), _c(bias, np.float32)
    return lib().oracle_time_mlp_rows(_p(a), _p(b), _p(bias), C.c_int64(nrows), C.c_int64(b.shape[1]),
                                      C.c_int64(a.shape[1]))
