import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # a fresh checkout has no built libraries (they are not in version control): build them once
    from necklace_amd.csrc import build as hip_build
    hip_build.ensure_built()
    import oracle
    oracle.c.lib()


def bits_to_f32(hexes):
    return np.array([int(h, 16) for h in hexes], dtype=np.uint32).view(np.float32)


def f32_bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def assert_bits_equal(got, want, what=""):
    """Bit-for-bit fp32 equality, except that any NaN matches any NaN."""
    got = np.ascontiguousarray(got, dtype=np.float32)
    want = np.ascontiguousarray(want, dtype=np.float32)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    gb, wb = got.view(np.uint32), want.view(np.uint32)
    bad = (gb != wb) & ~(np.isnan(got) & np.isnan(want))
    if bad.any():
        idx = np.flatnonzero(bad.reshape(-1))[:8]
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {bad.size} elements differ; first at {idx.tolist()}: "
            f"got {[hex(x) for x in gb.reshape(-1)[idx]]} want {[hex(x) for x in wb.reshape(-1)[idx]]}")


def assert_words_equal(got, want, what=""):
    got = np.ascontiguousarray(got).view(np.uint32)
    want = np.ascontiguousarray(want).view(np.uint32)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    bad = got != want
    if bad.any():
        idx = np.flatnonzero(bad.reshape(-1))[:8]
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {bad.size} words differ; first at {idx.tolist()}: "
            f"got {[hex(x) for x in got.reshape(-1)[idx]]} want {[hex(x) for x in want.reshape(-1)[idx]]}")


@pytest.fixture(scope="session")
def kat():
    with open(os.path.join(ROOT, "tests", "golden", "kat_vectors.json")) as f:
        return json.load(f)


def kat_quant_cases(kat):
    out = []
    for v in kat["quantize"]:
        shape = tuple(v["shape"])
        a = bits_to_f32(v["a_bits"]).reshape(shape)
        t = float(bits_to_f32([v["thrd_bits"]])[0])
        words = np.array([int(h, 16) for h in v["words"]], dtype=np.uint32)
        if len(shape) == 2:
            words = words.reshape((shape[0] + 15) // 16, shape[1])
        r = bits_to_f32([("7FC00000" if h == "NAN" else h) for h in v["r_bits"]]).reshape(shape)
        out.append((v["name"], a, t, words, r, v))
    return out
