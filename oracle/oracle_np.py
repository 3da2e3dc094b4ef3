"""Whole-array numpy restatement of necklace/cuda/quantize.py — TEST INFRASTRUCTURE ONLY.

Independent of nklq_oracle.c: where the C file walks (x, y, i) like a
reference thread, this one classifies the whole array at once and packs by
reshaping to (m, 16, k) and shifting, so the two agree only if both read the
reference's bit layout (quantize.py:35-51: code of row 16x+i at bit 2i of
word (x, y)) the same way.  All arithmetic is float32 (the jit signature at
quantize.py:16 types A, R and thrd as float32).
"""
import numpy as np

CMP_RATIO = 16  # quantize.py:8


def _as2d(a):
    return a.reshape(-1, 1) if a.ndim == 1 else a


def quantize(A, thrd, R_in=None):
    """Returns (C uint32, R float32).  R_in given: a = fl32(A + R_in) first."""
    A = np.asarray(A, dtype=np.float32)
    t = np.float32(thrd)
    a = A if R_in is None else (A + np.asarray(R_in, dtype=np.float32)).astype(np.float32)
    a2 = _as2d(a)
    n, k = a2.shape
    with np.errstate(invalid="ignore"):
        ge = a2 >= t  # quantize.py:41, tested first
        le = (a2 <= -t) & ~ge  # quantize.py:44, only reached when :41 is false
    R = np.where(ge, a2 - t, np.where(le, a2 + t, a2)).astype(np.float32)
    # untouched elements keep their exact bits (np.where copies, so -0.0 and NaN payloads survive)
    codes = ge.astype(np.uint32) | (le.astype(np.uint32) << np.uint32(1))
    m = (n + CMP_RATIO - 1) // CMP_RATIO
    padded = np.zeros((m * CMP_RATIO, k), dtype=np.uint32)
    padded[:n] = codes
    shifts = (2 * np.arange(CMP_RATIO, dtype=np.uint32)).reshape(1, CMP_RATIO, 1)
    C = np.bitwise_or.reduce(padded.reshape(m, CMP_RATIO, k) << shifts, axis=1).astype(np.uint32)
    if A.ndim == 1:
        return C.reshape(m), R.reshape(n)
    return C, R


def dequantize(C, n, thrd):
    C = np.asarray(C, dtype=np.uint32)
    t = np.float32(thrd)
    C2 = _as2d(C)
    m, k = C2.shape
    assert m == (n + CMP_RATIO - 1) // CMP_RATIO
    shifts = (2 * np.arange(CMP_RATIO, dtype=np.uint32)).reshape(1, CMP_RATIO, 1)
    codes = ((C2.reshape(m, 1, k) >> shifts) & np.uint32(3)).reshape(m * CMP_RATIO, k)[:n]
    out = np.zeros((n, k), dtype=np.float32)  # codes 00 and 11 -> +0.0 (quantize.py:86-87)
    out[codes == 1] = t
    out[codes == 2] = -t
    return out.reshape(n) if C.ndim == 1 else out


def dequant_accumulate(payloads, n, thrd, acc=None):
    s = np.zeros(n, dtype=np.float32) if acc is None else np.array(acc, dtype=np.float32, copy=True)
    for p in payloads:  # strictly in payload order
        s = (s + dequantize(np.asarray(p, dtype=np.uint32).reshape(-1), n, thrd)).astype(np.float32)
    return s
