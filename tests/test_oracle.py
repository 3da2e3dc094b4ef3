"""Pins the CPU checker (oracle/) before anything is compared against it.

The reference (necklace/cuda/quantize.py) ships no vectors, so the pins are:
hand-worked known-answer vectors, two independent restatements agreeing,
exhaustive neighbourhoods of +-t, and invariants the kernel text implies.
"""
import numpy as np
import pytest

import oracle
from conftest import (assert_bits_equal, assert_words_equal, bits_to_f32, f32_bits,
                      kat_quant_cases)

IMPLS = [("c", oracle.c), ("vec", oracle.vec)]
THRESHOLDS = [0.005, 1e-3, 2e-3, 1e-2, 0.3, 0.5]


@pytest.mark.parametrize("name,impl", IMPLS)
def test_quantize_kat(kat, name, impl):
    for cname, a, t, words, r, _ in kat_quant_cases(kat):
        C, R = impl.quantize(a, t)
        assert_words_equal(C, words, f"{name}:{cname} words")
        assert_bits_equal(R, r, f"{name}:{cname} residual")


@pytest.mark.parametrize("name,impl", IMPLS)
def test_threshold_crosses_as_fp32(kat, name, impl):
    """Passing the double 0.005 must behave like its fp32 rounding (jit signature, quantize.py:16)."""
    v = [x for x in kat["quantize"] if "thrd_double" in x][0]
    a = bits_to_f32(v["a_bits"])
    C, R = impl.quantize(a, v["thrd_double"])
    assert [f"{w:08X}" for w in C] == v["words"]
    assert [f"{b:08X}" for b in f32_bits(R)] == v["r_bits"]


@pytest.mark.parametrize("name,impl", IMPLS)
def test_dequantize_kat(kat, name, impl):
    for v in kat["dequantize"]:
        t = float(bits_to_f32([v["thrd_bits"]])[0])
        words = np.array([int(h, 16) for h in v["words"]], dtype=np.uint32)
        out = impl.dequantize(words, v["n"], t)
        assert_bits_equal(out, bits_to_f32(v["out_bits"]), f"{name}:{v['name']}")


def _nan_bits(hexes):
    return bits_to_f32([("7FC00000" if h == "NAN" else h) for h in hexes])


@pytest.mark.parametrize("name,impl", IMPLS)
def test_fused_kat(kat, name, impl):
    """Error-feedback step a = fl32(g + r_in), worked by hand: signed zeros, sums that round onto
    +-t, NaN residual."""
    for v in kat["fused"]:
        t = float(bits_to_f32([v["thrd_bits"]])[0])
        g, r_in = bits_to_f32(v["g_bits"]), bits_to_f32(v["r_in_bits"])
        with np.errstate(invalid="ignore"):
            C, R = impl.quantize(g, t, R_in=r_in)
        assert [f"{w:08X}" for w in C] == v["words"], f"{name}:{v['name']}"
        assert_bits_equal(R, _nan_bits(v["r_bits"]), f"{name}:{v['name']} residual")


@pytest.mark.parametrize("name,impl", IMPLS)
def test_accumulate_kat(kat, name, impl):
    for v in kat["accumulate"]:
        t = float(bits_to_f32([v["thrd_bits"]])[0])
        pl = [np.array([int(h, 16) for h in p], dtype=np.uint32) for p in v["payload_words"]]
        start = bits_to_f32(v["acc_in_bits"]) if "acc_in_bits" in v else None
        out = impl.dequant_accumulate(pl, v["n"], t, acc=None if start is None else start.copy())
        assert_bits_equal(out, _nan_bits(v["acc_bits"]), f"{name}:{v['name']}")
        # continuing a running sum from memory gives the same bits as one pass
        half = impl.dequant_accumulate(pl[:1], v["n"], t, acc=None if start is None else start.copy())
        out2 = impl.dequant_accumulate(pl[1:], v["n"], t, acc=half)
        assert_bits_equal(out2, out, f"{name}:{v['name']} split")


def _neighbourhood(t32, width=8):
    """Every fp32 within `width` ulps of +t and -t, plus specials."""
    tb = int(np.float32(t32).view(np.uint32))
    pos = np.arange(tb - width, tb + width + 1, dtype=np.int64).astype(np.uint32)
    neg = pos | np.uint32(0x80000000)
    special = np.array([0x00000000, 0x80000000, 0x00000001, 0x80000001, 0x007FFFFF, 0x807FFFFF,
                        0x00800000, 0x80800000, 0x7F7FFFFF, 0xFF7FFFFF, 0x7F800000, 0xFF800000,
                        0x7FC00000, 0xFFC00001], dtype=np.uint32)
    return np.concatenate([pos, neg, special]).view(np.float32)


@pytest.mark.parametrize("thrd", THRESHOLDS + [0.0, -0.25, 1e-45])
def test_invariants_around_threshold(thrd):
    """What quantize.py:41-49 implies element by element, checked on both restatements."""
    t = np.float32(thrd)
    a = _neighbourhood(t) if thrd > 0 else _neighbourhood(np.float32(0.25))
    for name, impl in IMPLS:
        C, R = impl.quantize(a, thrd)
        codes = (C.repeat(16) >> np.tile(2 * np.arange(16, dtype=np.uint32), C.size))[: a.size] & 3
        with np.errstate(invalid="ignore"):
            ge = a >= t
            le = (a <= -t) & ~ge
        assert ((codes == 1) == ge).all(), name
        assert ((codes == 2) == le).all(), name
        assert (codes != 3).all(), name
        mid = codes == 0
        assert_bits_equal(R[mid], a[mid], f"{name} untouched residual")
        assert_bits_equal(R[ge], (a[ge] - t).astype(np.float32), f"{name} a-t")
        assert_bits_equal(R[le], (a[le] + t).astype(np.float32), f"{name} a+t")
        # bits past the end of the last word stay zero
        used = a.size % 16
        if used:
            assert int(C[-1]) >> (2 * used) == 0, name


@pytest.mark.parametrize("n", list(range(1, 50)) + [255, 256, 257, 1023, 4097])
def test_two_restatements_agree_flat(n):
    rng = np.random.default_rng(1000 + n)
    a = rng.normal(0, 0.01, n).astype(np.float32)
    r0 = rng.normal(0, 0.003, n).astype(np.float32)
    for thrd in (0.005, 1e-3):
        Cc, Rc = oracle.c.quantize(a, thrd)
        Cv, Rv = oracle.vec.quantize(a, thrd)
        assert_words_equal(Cc, Cv, "plain words")
        assert_bits_equal(Rc, Rv, "plain residual")
        Cc, Rc = oracle.c.quantize(a, thrd, R_in=r0)
        Cv, Rv = oracle.vec.quantize(a, thrd, R_in=r0)
        assert_words_equal(Cc, Cv, "fused words")
        assert_bits_equal(Rc, Rv, "fused residual")
        assert_bits_equal(oracle.c.dequantize(Cc, n, thrd), oracle.vec.dequantize(Cv, n, thrd), "deq")


@pytest.mark.parametrize("n,k", [(1, 1), (16, 16), (17, 5), (33, 7), (224, 224), (100, 3), (5, 64)])
def test_two_restatements_agree_2d_and_column_property(n, k):
    rng = np.random.default_rng(n * 1000 + k)
    A = (rng.random((n, k)) - 0.5).astype(np.float32) * 2  # the value range of test_11, quantize.py:151
    Cc, Rc = oracle.c.quantize(A, 0.5)
    Cv, Rv = oracle.vec.quantize(A, 0.5)
    assert_words_equal(Cc, Cv)
    assert_bits_equal(Rc, Rv)
    # column y of the matrix form is the flat form of that column
    for y in {0, k // 2, k - 1}:
        Cf, Rf = oracle.c.quantize(np.ascontiguousarray(A[:, y]), 0.5)
        assert_words_equal(Cc[:, y], Cf, f"col {y}")
        assert_bits_equal(Rc[:, y], Rf, f"col {y}")
    assert_bits_equal(oracle.c.dequantize(Cc, n, 0.5), oracle.vec.dequantize(Cv, n, 0.5))


def test_dequantize_exhaustive_codes_and_positions():
    t = np.float32(0.3)
    want = {0: np.float32(0.0), 1: t, 2: -t, 3: np.float32(0.0)}
    for name, impl in IMPLS:
        for pos in range(16):
            for code in range(4):
                for background in (0x00000000, 0xFFFFFFFF):
                    w = (background & ~(3 << (2 * pos)) | (code << (2 * pos))) & 0xFFFFFFFF
                    out = impl.dequantize(np.array([w], dtype=np.uint32), 16, 0.3)
                    assert out[pos].view(np.uint32) == want[code].view(np.uint32), (name, pos, code)


def test_round_trip_and_idempotence():
    """quantize(decode(C)) == C for t > 0, and decode(C) has zero residual."""
    rng = np.random.default_rng(7)
    n = 10007
    a = rng.standard_t(3, n).astype(np.float32) * np.float32(1e-3)
    for name, impl in IMPLS:
        C, R = impl.quantize(a, 2e-3)
        d = impl.dequantize(C, n, 2e-3)
        C2, R2 = impl.quantize(d, 2e-3)
        assert_words_equal(C2, C, name)
        assert not R2.any(), name
        # a == decode + residual up to one rounding of the subtraction
        assert np.allclose(d.astype(np.float64) + R, a, rtol=0, atol=1e-9), name


def test_chunk_invariance():
    """Chunks that start on a multiple of 16 reproduce the whole-vector result."""
    rng = np.random.default_rng(11)
    n = 5000 + 7
    g = rng.normal(0, 5e-3, n).astype(np.float32)
    r = rng.normal(0, 1e-3, n).astype(np.float32)
    Cw, Rw = oracle.c.quantize(g, 1e-2, R_in=r)
    Cs, Rs = [], []
    for lo in range(0, n, 1600):
        C, R = oracle.c.quantize(g[lo:lo + 1600], 1e-2, R_in=r[lo:lo + 1600])
        Cs.append(C)
        Rs.append(R)
    assert_words_equal(np.concatenate(Cs), Cw)
    assert_bits_equal(np.concatenate(Rs), Rw)


def test_fused_inplace_matches_functional_and_error_feedback_conserves():
    rng = np.random.default_rng(3)
    n = 4099
    r = np.zeros(n, dtype=np.float32)
    c = np.zeros((n + 15) // 16, dtype=np.uint32)
    total_sent = np.zeros(n, dtype=np.float64)
    total_grad = np.zeros(n, dtype=np.float64)
    for step in range(10):
        g = rng.normal(0, 1e-3, n).astype(np.float32)
        Cf, Rf = oracle.vec.quantize(g, 1e-3, R_in=r)
        oracle.c.fused_quantize_inplace(g, r, c, 1e-3)
        assert_words_equal(c, Cf, f"step {step}")
        assert_bits_equal(r, Rf, f"step {step}")
        total_sent += oracle.c.dequantize(c, n, 1e-3)
        total_grad += g
    # error feedback: what was sent plus what is still owed equals what came in
    assert np.allclose(total_sent + r, total_grad, rtol=0, atol=1e-7)


def test_accumulate_matches_numpy_and_ignores_tail_bits():
    rng = np.random.default_rng(5)
    n = 1000 + 13
    m = (n + 15) // 16
    pl = []
    for p in range(8):
        codes = rng.choice([0, 1, 2], size=m * 16, p=[0.9, 0.05, 0.05]).astype(np.uint32)
        codes[n:] = 0
        w = np.bitwise_or.reduce(codes.reshape(m, 16) << (2 * np.arange(16, dtype=np.uint32)), axis=1)
        pl.append(w.astype(np.uint32))
    a = oracle.c.dequant_accumulate(pl, n, 1e-3)
    b = oracle.vec.dequant_accumulate(pl, n, 1e-3)
    assert_bits_equal(a, b)
    dirty = [p.copy() for p in pl]
    for p in dirty:
        p[-1] |= np.uint32(0xFFFFFFFF << (2 * (n % 16)) & 0xFFFFFFFF)
    assert_bits_equal(oracle.c.dequant_accumulate(dirty, n, 1e-3), a)
    base = rng.normal(0, 1, n).astype(np.float32)
    assert_bits_equal(oracle.c.dequant_accumulate(pl, n, 1e-3, acc=base),
                      oracle.vec.dequant_accumulate(pl, n, 1e-3, acc=base))
