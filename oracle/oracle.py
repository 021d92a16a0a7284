"""ctypes binding of the CPU oracle (oracle/acc_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of bench.py.  The library under accelerate-cuda_amd/ never
imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

OP_ADD, OP_MUL, OP_MIN, OP_MAX, OP_FIRST, OP_LAST, OP_AFFINE16 = range(7)
DIR_LEFT, DIR_RIGHT = 0, 1
SCANL, SCANL1, SCANLP, SCANR, SCANR1, SCANRP = range(6)
CLAMP, MIRROR, WRAP, CONSTANT = range(4)

SCAN_KINDS = {"scanl": SCANL, "scanl1": SCANL1, "scanl'": SCANLP,
              "scanr": SCANR, "scanr1": SCANR1, "scanr'": SCANRP}
BOUNDARY = {"clamp": CLAMP, "mirror": MIRROR, "wrap": WRAP, "constant": CONSTANT}


def build(force=False):
    """Compile liboracle.so from acc_oracle.c with the committed Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []),
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_dot_f32.restype = C.c_float
        _lib.orc_dot_f64.restype = C.c_double
        _lib.orc_dot_abs_f64.restype = C.c_double
        _lib.orc_boundary_index.restype = C.c_int64
        _lib.orc_boundary_index.argtypes = [C.c_int, C.c_int64, C.c_int64]
    return _lib


_SUF = {np.dtype(np.int32): ("i32", C.c_int32), np.dtype(np.int64): ("i64", C.c_int64),
        np.dtype(np.float32): ("f32", C.c_float), np.dtype(np.float64): ("f64", C.c_double)}


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype=None):
    return np.ascontiguousarray(a, dtype=dtype)


class OracleError(Exception):
    pass


def _check(rc, what):
    if rc == 2:
        raise OracleError(what + ": empty array")
    if rc != 0:
        raise OracleError("%s: oracle status %d" % (what, rc))


def fold(op, x, seed=None, direction=DIR_LEFT):
    """fold / fold1 (seed=None) along the innermost dimension."""
    x = _c(x)
    suf, ct = _SUF[x.dtype]
    inner = x.shape[-1] if x.ndim else 1
    outer_shape = x.shape[:-1]
    outer = int(np.prod([max(1, s) for s in outer_shape], dtype=np.int64)) if outer_shape else 1
    if x.size == 0 and outer_shape and 0 in outer_shape:
        # Execute.hs:287-289: empty outer extents are forced to 1
        outer_shape = tuple(max(1, s) for s in outer_shape)
    out = np.empty(outer_shape, dtype=x.dtype)
    rc = getattr(lib(), "orc_fold_" + suf)(
        C.c_int(op), C.c_int(seed is not None), ct(0 if seed is None else seed), _p(x),
        C.c_int64(outer), C.c_int64(inner), C.c_int(direction), _p(out))
    _check(rc, "fold")
    return out


def foldseg(op, x, offsets, seed=None, direction=DIR_LEFT):
    x = _c(x)
    offsets = _c(offsets, np.int32)
    suf, ct = _SUF[x.dtype]
    nseg = offsets.size - 1
    out = np.empty(max(nseg, 0), dtype=x.dtype)
    rc = getattr(lib(), "orc_foldseg_" + suf)(
        C.c_int(op), C.c_int(seed is not None), ct(0 if seed is None else seed), _p(x),
        _p(offsets), C.c_int64(nseg), C.c_int(direction), _p(out))
    _check(rc, "foldSeg")
    return out


def foldseg_nd(op, x, offsets, seed=None, direction=DIR_LEFT):
    """foldSeg / fold1Seg along the innermost dimension of every outer row of `x` (rank >= 1)"""
    x = _c(x)
    offsets = _c(offsets, np.int32)
    suf, ct = _SUF[x.dtype]
    nseg = offsets.size - 1
    inner = x.shape[-1]
    outer = int(np.prod(x.shape[:-1], dtype=np.int64))
    out = np.empty(x.shape[:-1] + (max(nseg, 0),), dtype=x.dtype)
    rc = getattr(lib(), "orc_foldseg_nd_" + suf)(
        C.c_int(op), C.c_int(seed is not None), ct(0 if seed is None else seed), _p(x), C.c_int64(outer), C.c_int64(inner),
        _p(offsets), C.c_int64(nseg), C.c_int(direction), _p(out))
    _check(rc, "foldSeg")
    return out


def dot_f32(x, y, direction=DIR_LEFT):
    x = _c(x, np.float32)
    y = _c(y, np.float32)
    assert x.size == y.size
    return np.float32(lib().orc_dot_f32(_p(x), _p(y), C.c_int64(x.size), C.c_int(direction)))


def dot_f64(x, y):
    x = _c(x, np.float32)
    y = _c(y, np.float32)
    return float(lib().orc_dot_f64(_p(x), _p(y), C.c_int64(x.size)))


def dot_abs_f64(x, y):
    x = _c(x, np.float32)
    y = _c(y, np.float32)
    return float(lib().orc_dot_abs_f64(_p(x), _p(y), C.c_int64(x.size)))


def smvm_f32(vals, cols, offsets, x, direction=DIR_LEFT):
    vals = _c(vals, np.float32)
    cols = _c(cols, np.int32)
    offsets = _c(offsets, np.int32)
    x = _c(x, np.float32)
    nrows = offsets.size - 1
    y = np.empty(nrows, dtype=np.float32)
    rc = lib().orc_smvm_f32(_p(vals), _p(cols), _p(offsets), _p(x), C.c_int64(nrows),
                            C.c_int(direction), _p(y))
    _check(rc, "smvm")
    return y


def smvm_f64(vals, cols, offsets, x):
    vals = _c(vals, np.float32)
    cols = _c(cols, np.int32)
    offsets = _c(offsets, np.int32)
    x = _c(x, np.float32)
    nrows = offsets.size - 1
    y = np.empty(nrows, dtype=np.float64)
    ya = np.empty(nrows, dtype=np.float64)
    lib().orc_smvm_f64(_p(vals), _p(cols), _p(offsets), _p(x), C.c_int64(nrows), _p(y), _p(ya))
    return y, ya


def scan(kind, op, x, seed=0):
    """Returns the scan result; for the primed variants a (body, total) pair."""
    if isinstance(kind, str):
        kind = SCAN_KINDS[kind]
    x = _c(x)
    suf, ct = _SUF[x.dtype]
    n = x.size
    nout = n + 1 if kind in (SCANL, SCANR) else n
    out = np.empty(nout, dtype=x.dtype)
    total = np.zeros(1, dtype=x.dtype)
    rc = getattr(lib(), "orc_scan_" + suf)(
        C.c_int(kind), C.c_int(op), ct(seed), _p(x), C.c_int64(n), _p(out), _p(total))
    _check(rc, "scan")
    if kind in (SCANLP, SCANRP):
        return out, total[0]
    return out


def permute(op, defaults, dst, src=None):
    defaults = _c(defaults)
    suf, _ = _SUF[defaults.dtype]
    dst = _c(dst, np.int32)
    if src is not None:
        src = _c(src, defaults.dtype)
        assert src.size == dst.size
    out = np.empty_like(defaults)
    rc = getattr(lib(), "orc_permute_" + suf)(
        C.c_int(op), _p(defaults), C.c_int64(defaults.size), _p(dst),
        _p(src) if src is not None else None, C.c_int64(dst.size), _p(out))
    _check(rc, "permute")
    return out


def zipwith_mul_f32(x, y):
    x = _c(x, np.float32)
    y = _c(y, np.float32)
    assert x.shape == y.shape
    out = np.empty_like(x)
    lib().orc_zipwith_mul_f32(_p(x), _p(y), C.c_int64(x.size), _p(out))
    return out


def backpermute(arr, idx):
    arr = _c(arr)
    idx = _c(idx, np.int32)
    suf, _ = _SUF[arr.dtype]
    out = np.empty(idx.shape, dtype=arr.dtype)
    rc = getattr(lib(), "orc_backpermute_" + suf)(_p(arr), C.c_int64(arr.size), _p(idx),
                                                  C.c_int64(idx.size), _p(out))
    _check(rc, "backpermute")
    return out


def stencil2d(img, taps, divisor=1.0, mode="clamp", constant=0.0, iters=1):
    """taps: list of (dy, dx, coefficient) in evaluation order."""
    img = _c(img, np.float32)
    h, w = img.shape
    dy = np.array([t[0] for t in taps], dtype=np.int32)
    dx = np.array([t[1] for t in taps], dtype=np.int32)
    cf = np.array([t[2] for t in taps], dtype=np.float32)
    m = BOUNDARY[mode] if isinstance(mode, str) else mode
    out = np.empty_like(img)
    tmp = np.empty_like(img)
    rc = lib().orc_stencil2d_iter_f32(_p(img), C.c_int64(h), C.c_int64(w), C.c_int(len(taps)),
                                      _p(dy), _p(dx), _p(cf), C.c_float(divisor), C.c_int(m),
                                      C.c_float(constant), C.c_int(iters), _p(out), _p(tmp))
    _check(rc, "stencil2d")
    return out


def stencil1d(vec, taps, divisor=1.0, mode="clamp", constant=0.0):
    """taps: list of (dx, coefficient)."""
    vec = _c(vec, np.float32)
    dx = np.array([t[0] for t in taps], dtype=np.int32)
    cf = np.array([t[1] for t in taps], dtype=np.float32)
    m = BOUNDARY[mode] if isinstance(mode, str) else mode
    out = np.empty_like(vec)
    rc = lib().orc_stencil1d_f32(_p(vec), C.c_int64(vec.size), C.c_int(len(taps)), _p(dx), _p(cf),
                                 C.c_float(divisor), C.c_int(m), C.c_float(constant), _p(out))
    _check(rc, "stencil1d")
    return out


def boundary_index(mode, i, sz):
    m = BOUNDARY[mode] if isinstance(mode, str) else mode
    return int(lib().orc_boundary_index(m, i, sz))


GAUSS3X3 = [(-1, -1, 1.0), (-1, 0, 2.0), (-1, 1, 1.0),
            (0, -1, 2.0), (0, 0, 4.0), (0, 1, 2.0),
            (1, -1, 1.0), (1, 0, 2.0), (1, 1, 1.0)]
LAPLACE5 = [(-1, 0, 1.0), (0, -1, 1.0), (0, 0, -4.0), (0, 1, 1.0), (1, 0, 1.0)]
