"""ctypes view of the CPU oracle (oracle/libgern_oracle.so).

Test infrastructure only: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py.  Nothing in the gern_amd package imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libgern_oracle.so")

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(dtype=np.uint32, flags="C_CONTIGUOUS")


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "libgern_oracle.so"])


def _load():
    if not os.path.exists(_LIB):
        build()
    lib = C.CDLL(_LIB)
    i64, u32, sz = C.c_int64, C.c_uint32, C.c_size_t
    sig = {
        "oracle_mt19937_u32": (None, [u32, _u32p, sz]),
        "oracle_fill_uniform": (None, [_f32p, sz, u32, C.c_float, C.c_float]),
        "oracle_fill_normal": (None, [_f32p, sz, u32, C.c_double, C.c_double]),
        "oracle_fill_ascending": (None, [_f32p, i64, i64, i64]),
        "oracle_round_to_bf16": (None, [_f32p, _u16p, _f32p, sz]),
        "oracle_blur_x": (None, [_f32p, i64, i64, i64, _f32p, i64, C.c_int]),
        "oracle_blur_y": (None, [_f32p, i64, i64, i64, _f32p, i64, C.c_int]),
        "oracle_blur_chain": (C.c_int, [_f32p, i64, i64, C.c_char_p, C.c_int, _f32p]),
        "oracle_blur_chain_tiled": (C.c_int, [_f32p, i64, i64, C.c_char_p, C.c_int, i64, i64, _f32p]),
        "oracle_softmax_rows": (None, [_f32p, i64, i64, i64, _f32p, i64]),
        "oracle_gemm_f32": (None, [_f32p, _f32p, _f32p, i64, i64, i64]),
        "oracle_gemm_f32_rows": (None, [_f32p, _f32p, _f32p, i64, i64, i64, i64, i64]),
        "oracle_gemm_bf16_f32acc": (None, [_u16p, _u16p, _f32p, i64, i64, i64]),
        "oracle_gemm_bf16_f32acc_rows": (None, [_u16p, _u16p, _f32p, i64, i64, i64, i64, i64]),
        "oracle_qk_softmax_rows": (None, [_u16p, _u16p, _f32p, i64, i64, i64, C.c_float, i64, i64]),
        "oracle_div_const_fma": (C.c_float, [C.c_float, C.c_float]),
        "oracle_div_const_mismatches": (C.c_uint64, [C.c_float, u32, u32]),
        "oracle_quotient_of_sum": (C.c_float, [C.c_float, C.c_float]),
        "oracle_quotient_mismatches": (C.c_uint64, [C.c_float, u32, u32, C.POINTER(u32), C.POINTER(C.c_float),
                                                    C.POINTER(C.c_float)]),
        "oracle_max_ulp": (u32, [_f32p, _f32p, sz]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


# ---- inputs ---------------------------------------------------------------
def mt19937_u32(seed, n):
    out = np.empty(n, dtype=np.uint32)
    lib().oracle_mt19937_u32(seed, out, n)
    return out


def uniform(shape, seed, lo=0.0, hi=1.0):
    out = np.empty(shape, dtype=np.float32)
    lib().oracle_fill_uniform(out.reshape(-1), out.size, seed, lo, hi)
    return out


def normal(shape, seed, mean=0.0, sigma=1.0):
    out = np.empty(shape, dtype=np.float32)
    lib().oracle_fill_normal(out.reshape(-1), out.size, seed, mean, sigma)
    return out


def ascending(rows, cols):
    out = np.empty((rows, cols), dtype=np.float32)
    lib().oracle_fill_ascending(out, rows, cols, cols)
    return out


def to_bf16(x):
    """Returns (bits uint16, value fp32) of x rounded to bf16, nearest-even."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = np.empty(x.shape, dtype=np.uint16)
    val = np.empty(x.shape, dtype=np.float32)
    lib().oracle_round_to_bf16(x.reshape(-1), bits.reshape(-1), val.reshape(-1), x.size)
    return bits, val


# ---- kernels --------------------------------------------------------------
def blur_chain(img, pattern, stride=3):
    img = np.ascontiguousarray(img, dtype=np.float32)
    rows, cols = img.shape
    nx, ny = pattern.count("x"), pattern.count("y")
    out = np.empty((rows - ny * (stride - 1), cols - nx * (stride - 1)), dtype=np.float32)
    rc = lib().oracle_blur_chain(img, rows, cols, pattern.encode(), stride, out)
    if rc != 0:
        raise ValueError("oracle_blur_chain: bad pattern or shape")
    return out


def blur_chain_tiled(img, pattern, tile_rows, tile_cols, stride=3):
    img = np.ascontiguousarray(img, dtype=np.float32)
    rows, cols = img.shape
    nx, ny = pattern.count("x"), pattern.count("y")
    out = np.empty((rows - ny * (stride - 1), cols - nx * (stride - 1)), dtype=np.float32)
    rc = lib().oracle_blur_chain_tiled(img, rows, cols, pattern.encode(), stride, tile_rows, tile_cols, out)
    if rc != 0:
        raise ValueError("oracle_blur_chain_tiled: bad pattern or shape")
    return out


def softmax_rows(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().oracle_softmax_rows(x, x.shape[0], x.shape[1], x.shape[1], out, x.shape[1])
    return out


def _row_range(rows, M):
    """(first, past-the-last) row to compute; the C code writes exactly these rows."""
    i0, i1 = (0, M) if rows is None else rows
    if not 0 <= i0 <= i1 <= M:
        raise ValueError("rows %r outside [0, %d]" % ((i0, i1), M))
    return int(i0), int(i1)


def gemm_f32(A, B, C_in=None, rows=None):
    A = np.ascontiguousarray(A, dtype=np.float32)
    B = np.ascontiguousarray(B, dtype=np.float32)
    M, K = A.shape
    N = B.shape[1]
    Cm = np.zeros((M, N), dtype=np.float32) if C_in is None else np.array(C_in, dtype=np.float32, order="C")
    i0, i1 = _row_range(rows, M)
    lib().oracle_gemm_f32_rows(A, B, Cm, M, N, K, i0, i1)
    return Cm


def gemm_bf16(A_bits, B_bits, rows=None):
    A_bits = np.ascontiguousarray(A_bits, dtype=np.uint16)
    B_bits = np.ascontiguousarray(B_bits, dtype=np.uint16)
    M, K = A_bits.shape
    N = B_bits.shape[1]
    Cm = np.zeros((M, N), dtype=np.float32)
    i0, i1 = _row_range(rows, M)
    lib().oracle_gemm_bf16_f32acc_rows(A_bits, B_bits, Cm, M, N, K, i0, i1)
    return Cm


def qk_softmax(Q_bits, K_bits, scale, rows=None):
    Q_bits = np.ascontiguousarray(Q_bits, dtype=np.uint16)
    K_bits = np.ascontiguousarray(K_bits, dtype=np.uint16)
    M, D = Q_bits.shape
    N = K_bits.shape[0]
    S = np.zeros((M, N), dtype=np.float32)
    i0, i1 = _row_range(rows, M)
    lib().oracle_qk_softmax_rows(Q_bits, K_bits, S, M, N, D, scale, i0, i1)
    return S


def max_ulp(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32).reshape(-1)
    b = np.ascontiguousarray(b, dtype=np.float32).reshape(-1)
    assert a.size == b.size
    return int(lib().oracle_max_ulp(a, b, a.size))
