"""Seeded random shapes, offsets, thresholds and payload counts against the CPU oracle.

Not a search for a known failure: a broad sweep of the argument space the hand-picked cases of
test_gpu_parity.py sample only at its corners."""
import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal, assert_words_equal
from gpu_util import dev, host_words, pack_codes_np, words_like
from necklace_amd.cuda import quantize as q

pytestmark = pytest.mark.gpu


def _values(rng, n, thrd):
    """Gradient-like values with a share of exact +-thrd, zeros and tiny numbers mixed in."""
    a = (rng.standard_normal(n) * abs(thrd) * rng.choice([0.3, 1.0, 3.0])).astype(np.float32)
    k = max(1, n // 50)
    idx = rng.integers(0, n, size=4 * k)
    t32 = np.float32(thrd)
    a[idx[:k]] = t32
    a[idx[k:2 * k]] = -t32
    a[idx[2 * k:3 * k]] = 0.0
    a[idx[3 * k:]] = np.float32(1e-42)
    return a


@pytest.mark.parametrize("seed", range(6))
def test_flat_random_lengths_offsets_thresholds(seed):
    rng = np.random.default_rng(1000 + seed)
    for _ in range(25):
        n = int(rng.choice([rng.integers(1, 70), rng.integers(70, 5000), rng.integers(5000, 300000)]))
        thrd = float(rng.choice([0.5, 0.3, 1e-2, 2e-3, 1e-3, 5e-3]))
        og, orr = int(rng.integers(0, 8)), int(rng.integers(0, 8))
        a, r0 = _values(rng, n, thrd), _values(rng, n, thrd * 0.5)
        gbuf = torch.zeros(n + 16, device="cuda")
        rbuf = torch.zeros(n + 16, device="cuda")
        A, R = gbuf[og:og + n], rbuf[orr:orr + n]
        A.copy_(torch.from_numpy(a))
        R.copy_(torch.from_numpy(r0))
        C = words_like(n)
        fused = bool(rng.integers(0, 2))
        q.cu_fn_matrix_quantize_e(A, C, R, thrd, add_residual=fused)
        want_c, want_r = oracle.c.quantize(a, thrd, R_in=r0 if fused else None)
        what = f"seed={seed} n={n} thrd={thrd} og={og} or={orr} fused={fused}"
        assert_words_equal(host_words(C), want_c, what)
        assert_bits_equal(R.cpu().numpy(), want_r, what)
        assert float(rbuf[:orr].abs().sum()) == 0.0 and float(rbuf[orr + n:].abs().sum()) == 0.0, what
        out = torch.full((n + 16,), 9.0, device="cuda")
        q.cu_fn_matrix_dequantize_e(out[orr:orr + n], C, None, thrd)
        assert_bits_equal(out[orr:orr + n].cpu().numpy(), oracle.c.dequantize(want_c, n, thrd), what)
        assert float(out[:orr].sum()) == 9.0 * orr and float(out[orr + n:].sum()) == 9.0 * (16 - orr), what


@pytest.mark.parametrize("seed", range(4))
def test_matrix_random_shapes(seed):
    rng = np.random.default_rng(2000 + seed)
    for _ in range(12):
        n = int(rng.choice([rng.integers(1, 40), rng.integers(40, 600)]))
        k = int(rng.choice([rng.integers(1, 70), rng.integers(64, 700), 256, 512, 1000]))
        thrd = float(rng.choice([0.5, 1e-2, 1e-3]))
        A, R0 = _values(rng, n * k, thrd).reshape(n, k), _values(rng, n * k, thrd * 0.5).reshape(n, k)
        fused = bool(rng.integers(0, 2))
        dA, dR, dC = dev(A), dev(R0), words_like(n, k)
        q.cu_fn_matrix_quantize_e(dA, dC, dR, thrd, add_residual=fused)
        want_c, want_r = oracle.c.quantize(A, thrd, R_in=R0 if fused else None)
        what = f"seed={seed} n={n} k={k} thrd={thrd} fused={fused}"
        assert_words_equal(host_words(dC), want_c, what)
        assert_bits_equal(dR.cpu().numpy(), want_r, what)
        junk = rng.integers(0, 2 ** 32, size=want_c.shape, dtype=np.uint64).astype(np.uint32)
        dB = torch.full((n, k), 7.0, device="cuda")
        q.cu_fn_matrix_dequantize_e(dB, dev(junk), None, thrd)
        assert_bits_equal(dB.cpu().numpy(), oracle.c.dequantize(junk, n, thrd), what)


@pytest.mark.parametrize("seed", range(4))
def test_accumulate_random_counts_lengths_offsets(seed):
    rng = np.random.default_rng(3000 + seed)
    for _ in range(10):
        n = int(rng.choice([rng.integers(1, 1100), rng.integers(1100, 9000), rng.integers(9000, 200000)]))
        K = int(rng.integers(1, 40))
        thrd = float(rng.choice([1e-3, 2e-3, 0.5, 0.3]))
        off = int(rng.integers(0, 8))
        pl = [pack_codes_np(rng.choice([0, 1, 2, 3], size=n, p=[0.7, 0.14, 0.14, 0.02]).astype(np.uint32), n)
              for _ in range(K)]
        base = _values(rng, n, thrd * 3)
        for acc0 in (False, True):
            buf = torch.full((n + 16,), 2.0, device="cuda")
            acc = buf[off:off + n]
            if acc0:
                acc.copy_(torch.from_numpy(base))
            q.cu_fn_dequantize_accumulate_e(acc, [dev(w) for w in pl], thrd, accumulate=acc0)
            want = oracle.c.dequant_accumulate(pl, n, thrd, acc=base if acc0 else None)
            what = f"seed={seed} n={n} K={K} thrd={thrd} off={off} accumulate={acc0}"
            assert_bits_equal(acc.cpu().numpy(), want, what)
            assert float(buf[:off].sum()) == 2.0 * off and float(buf[off + n:].sum()) == 2.0 * (16 - off), what
