"""ctypes view of the reference-derived checker under oracle/_ref/.

oracle/_ref/ holds, when it has been built (oracle/build_ref.sh, needs the
reference tree), one shared object per pipeline: the reference library's own
CPU lowering of the composed program.  Test infrastructure only.
"""
import ctypes as C
import os

import numpy as np

_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_ref")


class MatrixCPU(C.Structure):
    # gern::impl::MatrixCPU: float* data; int64 row, col, lda
    _fields_ = [("data", C.c_void_p), ("row", C.c_int64), ("col", C.c_int64), ("lda", C.c_int64)]


def available():
    return os.path.exists(os.path.join(_DIR, "manifest.txt"))


def _manifest():
    out = {}
    with open(os.path.join(_DIR, "manifest.txt")) as f:
        for line in f:
            parts = line.split()
            if parts:
                out[parts[0]] = (parts[1], parts[2:])
    return out


_cache = {}


def _hook(name):
    if name not in _cache:
        hook, order = _manifest()[name]
        lib = C.CDLL(os.path.join(_DIR, "libref_%s.so" % name))
        fn = getattr(lib, hook)
        fn.restype = None
        fn.argtypes = [C.POINTER(C.c_void_p)]
        _cache[name] = (fn, order)
    return _cache[name]


def _mat(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return MatrixCPU(a.ctypes.data, a.shape[0], a.shape[1], a.shape[1])


def _call(name, values):
    """values: parameter name -> numpy fp32 matrix or int."""
    fn, order = _hook(name)
    keep = []
    args = (C.c_void_p * len(order))()
    for i, pname in enumerate(order):
        v = values[pname]
        obj = _mat(v) if isinstance(v, np.ndarray) else C.c_int64(int(v))
        keep.append(obj)
        args[i] = C.cast(C.pointer(obj), C.c_void_p)
    fn(args)


def blur_chain(img, pattern, tile_rows, tile_cols):
    """Tile sizes must divide the output extents (the reference handles no ragged tiles)."""
    img = np.ascontiguousarray(img, dtype=np.float32)
    nx, ny = pattern.count("x"), pattern.count("y")
    out = np.zeros((img.shape[0] - 2 * ny, img.shape[1] - 2 * nx), dtype=np.float32)
    assert out.shape[0] % tile_rows == 0 and out.shape[1] % tile_cols == 0
    _call("blur_" + pattern, {"input": img, "output": out, "tile_rows": tile_rows, "tile_cols": tile_cols})
    return out


def softmax_rows(x, tile_rows=1):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros_like(x)
    assert x.shape[0] % tile_rows == 0
    _call("softmax_%d" % x.shape[1], {"input": x, "output": out, "tile_rows": tile_rows})
    return out


def gemm(A, B, ti, tj, tk):
    A = np.ascontiguousarray(A, dtype=np.float32)
    B = np.ascontiguousarray(B, dtype=np.float32)
    Cm = np.zeros((A.shape[0], B.shape[1]), dtype=np.float32)
    assert Cm.shape[0] % ti == 0 and Cm.shape[1] % tj == 0 and A.shape[1] % tk == 0
    _call("gemm", {"A": A, "B": B, "C": Cm, "k_dim": A.shape[1], "ti": ti, "tj": tj, "tk": tk})
    return Cm
