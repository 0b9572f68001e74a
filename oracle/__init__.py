"""ctypes front end of the CPU oracle (test infrastructure, not part of the product).

Only tests, the smoke check and the benchmark's cpu_baseline leg import this package.
The arithmetic lives in fp8gemm_oracle.c / block_dot.c; this module only marshals numpy
arrays.  `refutils()` loads the library built from the reference's own utils.h when it
was built in this checkout (oracle/_ref/), else returns None.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

CONFIGS = {
    # name: (M, N, K, seed, a_outlier_pct, a_outlier_mul)
    "cfg1": (1024, 512, 2048, 1001, 0.0, 1.0),
    "cfg2": (8192, 7168, 2048, 1002, 0.0, 1.0),
    "cfg3": (2048, 576, 7168, 1003, 0.0, 1.0),
    "cfg4": (8192, 4608, 7168, 1004, 1.0, 50.0),
    "cfg5": (32, 7168, 2048, 1005, 0.0, 1.0),
}


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference checkout exists)."""
    cmd = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)


def lib():
    global _LIB
    if _LIB is not None:
        return _LIB
    path = os.path.join(_HERE, "liboracle.so")
    if not os.path.exists(path):
        build()
    L = C.CDLL(path)
    u8p, f32p, u16p, f64p, i32p = (C.c_void_p,) * 5
    L.oracle_e4m3fn_to_f32.restype = C.c_float
    L.oracle_e4m3fn_to_f32.argtypes = [C.c_uint8]
    L.oracle_f32_to_e4m3fn.restype = C.c_uint8
    L.oracle_f32_to_e4m3fn.argtypes = [C.c_float]
    L.oracle_f32_to_bf16.restype = C.c_uint16
    L.oracle_f32_to_bf16.argtypes = [C.c_float]
    L.oracle_bf16_to_f32.restype = C.c_float
    L.oracle_bf16_to_f32.argtypes = [C.c_uint16]
    for name in ("oracle_f32_to_e4m3fn_array", "oracle_e4m3fn_to_f32_array",
                 "oracle_f32_to_bf16_array", "oracle_bf16_to_f32_array"):
        getattr(L, name).restype = None
        getattr(L, name).argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    L.oracle_ref_gemm_naive.restype = None
    L.oracle_ref_gemm_naive.argtypes = [u8p, u8p, f32p, f32p, u16p, C.c_int, C.c_int, C.c_int]
    L.oracle_ref_gemm.restype = None
    L.oracle_ref_gemm.argtypes = [u8p, u8p, f32p, f32p, u16p, f32p, C.c_int, C.c_int, C.c_int,
                                  C.c_int]
    L.oracle_ref_gemm_f64.restype = None
    L.oracle_ref_gemm_f64.argtypes = [u8p, u8p, f32p, f32p, f64p, C.c_int, C.c_int, C.c_int]
    L.oracle_ref_gemm_points.restype = None
    L.oracle_ref_gemm_points.argtypes = [u8p, u8p, f32p, f32p, i32p, i32p, C.c_int, f32p, u16p,
                                         C.c_int, C.c_int, C.c_int]
    L.oracle_gen_normal_bf16.restype = None
    L.oracle_gen_normal_bf16.argtypes = [f32p, C.c_size_t, C.c_size_t, C.c_uint64, C.c_double,
                                         C.c_double]
    L.oracle_quantize_a_1x128.restype = None
    L.oracle_quantize_a_1x128.argtypes = [f32p, u8p, f32p, C.c_int, C.c_int, C.c_int]
    L.oracle_quantize_b_128x128.restype = None
    L.oracle_quantize_b_128x128.argtypes = [f32p, u8p, f32p, C.c_int, C.c_int, C.c_int]
    L.oracle_make_inputs.restype = None
    L.oracle_make_inputs.argtypes = [u8p, u8p, f32p, f32p, C.c_int, C.c_int, C.c_int, C.c_uint64,
                                     C.c_double, C.c_double]
    L.oracle_compare_bf16.restype = C.c_long
    L.oracle_compare_bf16.argtypes = [u16p, u16p, C.c_size_t, C.c_double, C.c_double,
                                      C.POINTER(C.c_double), C.POINTER(C.c_double)]
    L.oracle_max_threads.restype = C.c_int
    _LIB = L
    return L


def _p(arr):
    return arr.ctypes.data_as(C.c_void_p)


def _chk(arr, dtype):
    assert arr.dtype == dtype and arr.flags.c_contiguous, (arr.dtype, dtype)
    return arr


# ------------------------------------------------------------------ codecs
def e4m3fn_decode(codes):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.shape, np.float32)
    lib().oracle_e4m3fn_to_f32_array(_p(codes), _p(out), codes.size)
    return out


def e4m3fn_encode(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint8)
    lib().oracle_f32_to_e4m3fn_array(_p(x), _p(out), x.size)
    return out


def bf16_encode(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_f32_to_bf16_array(_p(x), _p(out), x.size)
    return out


def bf16_decode(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().oracle_bf16_to_f32_array(_p(h), _p(out), h.size)
    return out


# ------------------------------------------------------------------ GEMM
def _gemm_args(a, b, a_scale, b_scale, m, n, k):
    assert k % 128 == 0 and m > 0 and n > 0
    sn = (n + 127) // 128
    _chk(a, np.uint8), _chk(b, np.uint8), _chk(a_scale, np.float32), _chk(b_scale, np.float32)
    assert a.size == m * k and b.size == n * k
    assert a_scale.size == (k // 128) * m and b_scale.size == (k // 128) * sn


def ref_gemm_naive(a, b, a_scale, b_scale, m, n, k):
    """check.cu:36-48 in utils.h:65-76's loop nest, literally.  Returns bf16 bits [m, n]."""
    _gemm_args(a, b, a_scale, b_scale, m, n, k)
    c = np.empty((m, n), np.uint16)
    lib().oracle_ref_gemm_naive(_p(a), _p(b), _p(a_scale), _p(b_scale), _p(c), m, n, k)
    return c


def ref_gemm(a, b, a_scale, b_scale, m, n, k, nthreads=0, want_f32=False):
    """Same values as ref_gemm_naive, loops arranged for speed.  Returns bf16 bits [m, n]
    (and the fp32 values before the cast when want_f32)."""
    _gemm_args(a, b, a_scale, b_scale, m, n, k)
    c = np.empty((m, n), np.uint16)
    f = np.empty((m, n), np.float32) if want_f32 else None
    lib().oracle_ref_gemm(_p(a), _p(b), _p(a_scale), _p(b_scale), _p(c),
                          _p(f) if want_f32 else None, m, n, k, nthreads)
    return (c, f) if want_f32 else c


def ref_gemm_f64(a, b, a_scale, b_scale, m, n, k):
    """Exact integer block sums, fp64 scaling and accumulation."""
    _gemm_args(a, b, a_scale, b_scale, m, n, k)
    c = np.empty((m, n), np.float64)
    lib().oracle_ref_gemm_f64(_p(a), _p(b), _p(a_scale), _p(b_scale), _p(c), m, n, k)
    return c


def ref_gemm_points(a, b, a_scale, b_scale, rows, cols, m, n, k):
    """ref_gemm_naive's value at the listed (row, col) points: (fp32, bf16 bits)."""
    _gemm_args(a, b, a_scale, b_scale, m, n, k)
    rows = np.ascontiguousarray(rows, np.int32)
    cols = np.ascontiguousarray(cols, np.int32)
    assert rows.shape == cols.shape
    f = np.empty(rows.shape, np.float32)
    h = np.empty(rows.shape, np.uint16)
    lib().oracle_ref_gemm_points(_p(a), _p(b), _p(a_scale), _p(b_scale), _p(rows), _p(cols),
                                 rows.size, _p(f), _p(h), m, n, k)
    return f, h


# ------------------------------------------------------------------ input producers
def gen_normal_bf16(rows, cols, seed, outlier_pct=0.0, outlier_mul=1.0):
    out = np.empty((rows, cols), np.float32)
    lib().oracle_gen_normal_bf16(_p(out), rows, cols, seed, outlier_pct, outlier_mul)
    return out


def quantize_a_1x128(x, bf16_arith=False):
    """x: [M, K] fp32 row-major -> (bytes laid out m + k*M as array [K, M], a_scale [K/128, M]).
    bf16_arith: round every intermediate to bf16, as torch does when quantize.py gets a bf16 tensor."""
    x = np.ascontiguousarray(x, np.float32)
    m, k = x.shape
    assert k % 128 == 0
    q = np.empty((k, m), np.uint8)
    s = np.empty((k // 128, m), np.float32)
    lib().oracle_quantize_a_1x128(_p(x), _p(q), _p(s), m, k, int(bool(bf16_arith)))
    return q, s


def quantize_b_128x128(x, bf16_arith=False):
    """x: [N, K] fp32 row-major -> (bytes n + k*N as array [K, N], b_scale [K/128, ceil(N/128)])."""
    x = np.ascontiguousarray(x, np.float32)
    n, k = x.shape
    assert k % 128 == 0
    q = np.empty((k, n), np.uint8)
    s = np.empty((k // 128, (n + 127) // 128), np.float32)
    lib().oracle_quantize_b_128x128(_p(x), _p(q), _p(s), n, k, int(bool(bf16_arith)))
    return q, s


def make_inputs(m, n, k, seed, a_outlier_pct=0.0, a_outlier_mul=1.0):
    """Seeded N(0,1) -> bf16 -> block quantisation.  Returns a[K,M], b[K,N] uint8 and
    a_scale[K/128,M], b_scale[K/128,ceil(N/128)] fp32, all in the kernel's layouts."""
    a = np.empty((k, m), np.uint8)
    b = np.empty((k, n), np.uint8)
    sa = np.empty((k // 128, m), np.float32)
    sb = np.empty((k // 128, (n + 127) // 128), np.float32)
    lib().oracle_make_inputs(_p(a), _p(b), _p(sa), _p(sb), m, n, k, seed, a_outlier_pct,
                             a_outlier_mul)
    return a, b, sa, sb


def make_config_inputs(name):
    m, n, k, seed, pct, mul = CONFIGS[name]
    return (m, n, k) + make_inputs(m, n, k, seed, pct, mul)


def compare_bf16(c, ref, rtol=1e-2, atol=1e-3):
    """The acceptance rule max|C-ref| <= rtol*max|ref| + atol.  Returns
    dict(bad=count of offending elements, max_err, max_ref, bound)."""
    c = np.ascontiguousarray(c, np.uint16)
    ref = np.ascontiguousarray(ref, np.uint16)
    assert c.shape == ref.shape
    me, mr = C.c_double(), C.c_double()
    bad = lib().oracle_compare_bf16(_p(c), _p(ref), c.size, rtol, atol, C.byref(me), C.byref(mr))
    return dict(bad=int(bad), max_err=me.value, max_ref=mr.value, bound=rtol * mr.value + atol)


def max_threads():
    return int(lib().oracle_max_threads())


# ------------------------------------------------------------------ reference helpers
def refutils():
    """Library of the reference's own utils.h helpers, or None when not built here."""
    path = os.path.join(_HERE, "_ref", "librefutils.so")
    if not os.path.exists(path):
        return None
    try:
        L = C.CDLL(path)
    except OSError:
        return None
    L.ref_genMat.restype = None
    L.ref_genMat.argtypes = [C.c_void_p, C.c_size_t]
    L.ref_row_to_col_major.restype = None
    L.ref_row_to_col_major.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int]
    L.ref_gemmCPU.restype = None
    L.ref_gemmCPU.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                              C.c_size_t]
    L.ref_allClose.restype = C.c_int
    L.ref_allClose.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_float]
    return L
