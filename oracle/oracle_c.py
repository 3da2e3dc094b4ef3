"""ctypes view of nklq_oracle.c (numpy arrays in, numpy arrays out)."""
import ctypes as ct
import os
import subprocess

import numpy as _np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libnklq_oracle.so")
_lib = None

_f32p = ct.POINTER(ct.c_float)
_u32p = ct.POINTER(ct.c_uint32)


def build(force=False):
    """Compile nklq_oracle.c with gcc (a second or two)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ct.CDLL(_SO)
        L.orc_quantize_2d.argtypes = [_f32p, _f32p, _f32p, _u32p, ct.c_uint64, ct.c_uint64,
                                      ct.c_float, ct.c_int]
        L.orc_quantize_2d.restype = None
        L.orc_dequantize_2d.argtypes = [_f32p, _u32p, ct.c_uint64, ct.c_uint64, ct.c_float]
        L.orc_dequantize_2d.restype = None
        L.orc_fused_quantize_flat.argtypes = [_f32p, _f32p, _u32p, ct.c_uint64, ct.c_float]
        L.orc_fused_quantize_flat.restype = None
        L.orc_dequant_accumulate.argtypes = [_f32p, ct.POINTER(_u32p), ct.c_int, ct.c_uint64,
                                             ct.c_float, ct.c_int]
        L.orc_dequant_accumulate.restype = None
        L.orc_threads.restype = ct.c_int
        L.orc_set_threads.argtypes = [ct.c_int]
        _lib = L
    return _lib


def _f(a):
    assert a.dtype == _np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(_f32p)


def _u(a):
    assert a.dtype == _np.uint32 and a.flags.c_contiguous
    return a.ctypes.data_as(_u32p)


def _shape2(a):
    if a.ndim == 1:
        return a.shape[0], 1
    assert a.ndim == 2
    return a.shape


def packed_shape(n, k=None):
    m = (n + 15) // 16
    return (m,) if k is None else (m, k)


def quantize(A, thrd, R_in=None):
    """Reference kernel on A (1-D = the (N,1) matrix).  R_in given: a = A + R_in first.

    Returns (C, R) as new arrays."""
    A = _np.ascontiguousarray(A, dtype=_np.float32)
    n, k = _shape2(A)
    R = _np.empty_like(A)
    C = _np.full(packed_shape(n, None if A.ndim == 1 else k), 0xDEADBEEF, dtype=_np.uint32)
    if R_in is None:
        lib().orc_quantize_2d(_f(A), None, _f(R), _u(C), n, k, thrd, 0)
    else:
        R_in = _np.ascontiguousarray(R_in, dtype=_np.float32)
        assert R_in.shape == A.shape
        lib().orc_quantize_2d(_f(A), _f(R_in), _f(R), _u(C), n, k, thrd, 1)
    return C, R


def fused_quantize_inplace(g, r, c, thrd):
    """Flat error-feedback step; r and c are updated in place."""
    assert g.ndim == 1 and r.shape == g.shape and c.shape == packed_shape(g.shape[0])
    lib().orc_fused_quantize_flat(_f(g), _f(r), _u(c), g.shape[0], thrd)


def dequantize(C, n, thrd):
    """Decode C (1-D words or [m,k]) to fp32 of n rows."""
    C = _np.ascontiguousarray(C, dtype=_np.uint32)
    if C.ndim == 1:
        k, shape = 1, (n,)
    else:
        k, shape = C.shape[1], (n, C.shape[1])
    assert C.shape[0] == (n + 15) // 16
    A = _np.full(shape, _np.nan, dtype=_np.float32)
    lib().orc_dequantize_2d(_f(A), _u(C), n, k, thrd)
    return A


def dequant_accumulate(payloads, n, thrd, acc=None):
    """Fixed-order sum of decoded payloads; acc given: continue from it (copy)."""
    payloads = [_np.ascontiguousarray(p, dtype=_np.uint32) for p in payloads]
    for p in payloads:
        assert p.shape == ((n + 15) // 16,)
    ptrs = (_u32p * len(payloads))(*[_u(p) for p in payloads])
    if acc is None:
        out = _np.full((n,), _np.nan, dtype=_np.float32)
        lib().orc_dequant_accumulate(_f(out), ptrs, len(payloads), n, thrd, 0)
    else:
        out = _np.array(acc, dtype=_np.float32, copy=True)
        lib().orc_dequant_accumulate(_f(out), ptrs, len(payloads), n, thrd, 1)
    return out


def threads():
    return lib().orc_threads()


def set_threads(t):
    lib().orc_set_threads(int(t))
