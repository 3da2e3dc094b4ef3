"""The C-ABI library loads, exports what include/nklq.h declares, and rejects bad
arguments before touching a GPU.  No kernel is launched here."""
import ctypes as ct
import os
import re

import pytest

from conftest import ROOT
from necklace_amd import _lib


def _declared(header="nklq.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nklq_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    L = _lib.lib()
    names = _declared()
    assert len(names) >= 8
    for n in names:
        assert hasattr(L, n), f"{n} declared in nklq.h but not exported"
    assert sorted(_lib.SYMBOLS) == names
    # what only serves measurements stays out of the product library
    for n in _lib.TUNING_SYMBOLS:
        assert not hasattr(L, n), f"{n} belongs to the measurement build only"


def test_the_measurement_build_exports_both_headers():
    T = _lib.tuning_lib()
    extra = _declared("nklq_tuning.h")
    assert sorted(_lib.TUNING_SYMBOLS) == extra
    for n in _declared() + extra:
        assert hasattr(T, n), f"{n} not exported by the measurement build"
    assert T.nklq_version() == _lib.lib().nklq_version()
    ok = 0x1000
    assert T.nklq_copy_f32(None, None, 0, None) == 0
    assert T.nklq_copy_f32(ok, ok + 2, 64, None) == -2
    assert T.nklq_copy_f32(ok, ok + 16, 64, None) == -4
    assert T.nklq_tuning_sum_interleaved_f32(None, None, 8, 0, 6, 0.5, None) == 0
    assert T.nklq_tuning_sum_interleaved_f32(ok, ok + 0x100000, 8, 1000, 6, 0.5, None) == -3   # not whole tiles
    assert T.nklq_tuning_sum_interleaved_f32(ok, ok + 0x100000, 8, 1024, 5, 0.5, None) == -3   # run below a tile's words
    assert T.nklq_tuning_sum_interleaved_f32(ok, ok + 0x100000, 17, 1024, 6, 0.5, None) == -3
    assert T.nklq_tuning_sum_interleaved_f32(ok, None, 8, 1024, 6, 0.5, None) == -1
    assert T.nklq_tuning_sum_interleaved_f32(ok, ok + 1024, 8, 1024, 6, 0.5, None) == -4       # words inside acc


def test_version_and_header_constants_agree():
    text = open(os.path.join(ROOT, "include", "nklq.h")).read()
    ver = int(re.search(r"#define NKLQ_VERSION (\d+)", text).group(1))
    assert _lib.lib().nklq_version() == ver
    mx = int(re.search(r"#define NKLQ_MAX_PAYLOADS_PER_LAUNCH (\d+)", text).group(1))
    assert _lib.NKLQ_MAX_PAYLOADS_PER_LAUNCH == mx


@pytest.mark.parametrize("n,k,want", [(0, 1, 0), (1, 1, 1), (16, 1, 1), (17, 1, 2), (224, 224, 14 * 224),
                                      (25557032, 1, 1597315), (354823168, 1, 22176448),
                                      (2800000000, 1, 175000000), (17, 3, 6)])
def test_packed_words(n, k, want):
    assert _lib.packed_words(n, k) == want


def test_argument_errors_are_reported_without_a_launch():
    L = _lib.lib()
    ok_ptr, odd_ptr = 0x1000, 0x1002
    # empty input: success, nothing to do
    assert L.nklq_quantize_f32(None, None, None, None, 0, 5, 0.5, 0, None) == 0
    assert L.nklq_dequantize_f32(None, None, 7, 0, 0.5, None) == 0
    assert L.nklq_dequant_accumulate_f32(None, None, 1, 0, 0.5, 0, None) == 0
    # null pointers
    assert L.nklq_quantize_f32(None, None, ok_ptr, ok_ptr + 64, 4, 1, 0.5, 0, None) == -1
    assert L.nklq_quantize_f32(ok_ptr, None, ok_ptr, ok_ptr + 64, 4, 1, 0.5, 1, None) == -1
    assert L.nklq_dequantize_f32(None, ok_ptr, 4, 1, 0.5, None) == -1
    # misaligned
    assert L.nklq_quantize_f32(odd_ptr, None, ok_ptr, ok_ptr + 64, 4, 1, 0.5, 0, None) == -2
    assert L.nklq_dequantize_f32(ok_ptr, odd_ptr, 4, 1, 0.5, None) == -2
    # sizes
    assert L.nklq_quantize_f32(ok_ptr, None, ok_ptr, ok_ptr + 64, 2 ** 40, 2 ** 40, 0.5, 0, None) == -3
    assert L.nklq_dequant_accumulate_f32(ok_ptr, None, 0, 4, 0.5, 0, None) == -3
    # outputs on top of each other
    assert L.nklq_quantize_f32(ok_ptr, None, ok_ptr + 64, ok_ptr, 4, 1, 0.5, 0, None) == -4
    arr = (ct.c_void_p * 1)(ok_ptr)
    assert L.nklq_dequant_accumulate_f32(ok_ptr, arr, 1, 4, 0.5, 0, None) == -4
    for code in (0, -1, -2, -3, -4):
        assert L.nklq_strerror(code)
    with pytest.raises(_lib.NklqError):
        _lib.check(-2)


def test_partial_overlaps_are_refused_without_a_launch():
    """Byte-range checks: an output may coincide exactly with an input (the in-place forms), any
    other overlap that involves an output is NKLQ_EALIAS.  Every case returns before a launch."""
    L = _lib.lib()
    vp, u64 = ct.c_void_p, ct.c_uint64
    base = 0x100000
    n = 4096                      # 16 KiB of fp32, 256 words (1 KiB) of codes
    g, r, c = base, base + 0x10000, base + 0x20000
    q = lambda g_, rin, rout, c_, add=1: L.nklq_quantize_f32(g_, rin, rout, c_, n, 1, 0.5, add, None)
    assert q(g, r, r, g + 4 * 100) == -4            # codes land in the middle of g
    assert q(g, r, r, r + 4 * n - 8) == -4          # codes straddle the end of the residual
    assert q(g, r, g + 8, c) == -4                  # residual out shifted against g
    assert q(g, r, r + 4, c) == -4                  # residual out shifted against residual in
    assert q(g, r, r, r - 1020) == -4               # the last word of c is the first float of the residual
    assert L.nklq_dequantize_f32(g, g + 4 * (n - 1), n, 1, 0.5, None) == -4     # words start inside out
    arr = (vp * 2)(c, g + 64)
    assert L.nklq_dequant_accumulate_f32(g, arr, 2, n, 0.5, 0, None) == -4      # second payload inside acc
    # one row: as many code words as elements, so c can coincide exactly with an input; only the
    # residual output has in-place partners (r_in, g)
    q1 = lambda g_, rin, rout, c_: L.nklq_quantize_f32(g_, rin, rout, c_, 1, n, 0.5, 1, None)
    assert q1(g, r, r, g) == -4                     # code words exactly on top of the gradient
    assert q1(g, r, c, r) == -4                     # code words exactly on top of the residual input
    assert q1(g, r, c, c) == -4                     # the two outputs on top of each other
    assert L.nklq_dequantize_f32(g, g, 1, n, 0.5, None) == -4                   # floats written over their own words
    arr1 = (vp * 1)(g)
    assert L.nklq_dequant_accumulate_f32(g, arr1, 1, 1, 0.5, 1, None) == -4     # one element, one word, same place
    gs1, rs1, cs1, ns1 = (vp * 1)(g), (vp * 1)(r), (vp * 1)(g), (u64 * 1)(1)
    assert L.nklq_quantize_multi_f32(1, gs1, rs1, cs1, ns1, 0.5, 1, None) == -4  # c[0] == g[0], one element
    # many vectors: an output of one vector on top of a buffer of another
    gs, rs, cs = (vp * 2)(g, g + 0x4000), (vp * 2)(r, r + 0x4000), (vp * 2)(c, r + 0x4000 - 16)
    ns = (u64 * 2)(n, n)
    assert L.nklq_quantize_multi_f32(2, gs, rs, cs, ns, 0.5, 1, None) == -4     # c[1] ends inside r[1]
    cs2 = (vp * 2)(c, c + 512)
    assert L.nklq_quantize_multi_f32(2, gs, rs, cs2, ns, 0.5, 1, None) == -4    # c[1] starts inside c[0]
    accs = (vp * 2)(g, g + 4 * n - 4)
    woff = (u64 * 2)(0, 256)
    bases = (vp * 1)(c)
    assert L.nklq_dequant_accumulate_multi_f32(2, accs, ns, woff, bases, 1, 0.5, 0, 1.0, None) == -4  # acc[1] over acc[0]
    accs = (vp * 2)(g, g + 0x4000)
    bases = (vp * 1)(g + 0x4000 + 4 * n - 1024)
    assert L.nklq_dequant_accumulate_multi_f32(2, accs, ns, woff, bases, 1, 0.5, 0, 1.0, None) == -4  # message over acc[1]


def _round_trip(cases):
    for which, good, bad in cases:
        before = _lib.tune(which)
        for v in good:
            _lib.tune(which, v)
            assert _lib.tune(which) == v
        for v in bad:
            with pytest.raises(ValueError):
                _lib.tune(which, v)
        assert _lib.tune(which) == good[-1]
        _lib.tune(which, before)
    with pytest.raises(ValueError):
        _lib.tune(9, 1)
    with pytest.raises(ValueError):
        _lib.tune(_lib.N_TUNE, 1)


def test_tune_knobs_round_trip():
    """The product library has one workgroup shape: its first three knobs take their default only."""
    interleave = ((3, (0, 1, 2, 3, 4, 5, 6), (7,)), (4, (0, 3, 6), (7,)), (5, (0, 3, 6), (7,)), (6, (0, 1, 2), (3,)))
    _round_trip(((0, (1,), (2, 3, 4)), (1, (256,), (64, 96, 1024)), (2, (1,), (0,))) + interleave)
    with _lib.use_tuning_library():
        _round_trip(((0, (1, 2, 4), (3,)), (1, (64, 128, 256, 512, 1024), (96,)), (2, (0, 1), ())) + interleave)
    assert _lib.lib() is not _lib.tuning_lib()


def test_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "SO_PATH", str(tmp_path / "libnklq.so"))
    with pytest.raises(ImportError):
        _lib.lib()


def test_the_package_never_touches_the_cpu_checker():
    pkg = os.path.join(ROOT, "necklace_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the checker"
