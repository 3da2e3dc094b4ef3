"""The C-ABI library loads, exports what include/nklq.h declares, and rejects bad
arguments before touching a GPU.  No kernel is launched here."""
import ctypes as ct
import os
import re

import pytest

from conftest import ROOT
from necklace_amd import _lib


def _declared():
    text = open(os.path.join(ROOT, "include", "nklq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nklq_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    L = _lib.lib()
    names = _declared()
    assert len(names) >= 8
    for n in names:
        assert hasattr(L, n), f"{n} declared in nklq.h but not exported"
    assert sorted(_lib.SYMBOLS) == names


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


def test_tune_knobs_round_trip():
    for which, good, bad in ((0, (1, 2, 4), 3), (1, (64, 128, 256, 512, 1024), 96), (2, (0, 1), None),
                             (3, (0, 1, 2, 3, 4, 5, 6), 7), (4, (0, 3, 6), 7)):
        before = _lib.tune(which)
        for v in good:
            _lib.tune(which, v)
            assert _lib.tune(which) == v
        if bad is not None:
            with pytest.raises(ValueError):
                _lib.tune(which, bad)
        _lib.tune(which, before)
    with pytest.raises(ValueError):
        _lib.tune(9, 1)


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
