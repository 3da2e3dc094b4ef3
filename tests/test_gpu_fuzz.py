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


@pytest.mark.parametrize("seed", range(3))
def test_many_vectors_random_lists(seed):
    """The many-vectors entry points on random lists (1 to 230 vectors of 1 to 200,000 elements,
    random gaps between them inside one arena, 1 to 9 messages): every vector equals its own flat
    result and nothing between the vectors is written."""
    rng = np.random.default_rng(4000 + seed)
    for _ in range(4):
        count = int(rng.choice([rng.integers(1, 10), rng.integers(10, 97), rng.integers(97, 230)]))
        ns = [int(rng.choice([rng.integers(1, 300), rng.integers(300, 5000), rng.integers(5000, 200000)]))
              for _ in range(count)]
        thrd, K = float(rng.choice([1e-3, 2e-3, 0.5])), int(rng.integers(1, 10))
        fused, acc0 = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        divisor = float(rng.choice([1.0, K, 3.0]))
        what = f"seed={seed} count={count} total={sum(ns)} thrd={thrd} K={K} fused={fused} acc0={acc0} / {divisor}"
        gaps = rng.integers(1, 9, size=count)
        starts = np.cumsum([4] + [n + int(g) for n, g in zip(ns, gaps)])[:-1]
        size = int(starts[-1]) + ns[-1] + 8
        between = np.ones(size, bool)
        for s, n in zip(starts, ns):
            between[s:s + n] = False
        a, r0 = _values(rng, size, thrd), _values(rng, size, thrd * 0.5)
        r0[between] = 5.0
        g_arena, r_arena = dev(a), dev(r0)
        wn = [(n + 15) // 16 for n in ns]
        woffs = [int(w) for w in np.cumsum([0] + wn)[:-1]]
        total_words = sum(wn)
        msgs = rng.integers(0, 2 ** 32, size=(K, total_words + 4), dtype=np.uint64).astype(np.uint32)
        recv = dev(msgs)
        q.cu_fn_quantize_multi_e([g_arena[s:s + n] for s, n in zip(starts, ns)],
                                 [recv[0, w:w + m] for w, m in zip(woffs, wn)],
                                 [r_arena[s:s + n] for s, n in zip(starts, ns)], thrd, add_residual=fused)
        got_r, got_w = r_arena.cpu().numpy(), host_words(recv)
        for i, (s, n) in enumerate(zip(starts, ns)):
            want_c, want_r = oracle.c.quantize(a[s:s + n], thrd, R_in=r0[s:s + n] if fused else None)
            assert_words_equal(got_w[0, woffs[i]:woffs[i] + wn[i]], want_c, f"{what}: vector {i} n={n}")
            assert_bits_equal(got_r[s:s + n], want_r, f"{what}: vector {i} n={n}")
        assert (got_r[between] == 5.0).all(), what
        assert np.array_equal(got_w[0, total_words:], msgs[0, total_words:]) and np.array_equal(got_w[1:], msgs[1:]), what
        base = _values(rng, size, thrd)
        base[between] = 9.0
        o_arena = dev(base)
        q.cu_fn_dequantize_accumulate_multi_e([o_arena[s:s + n] for s, n in zip(starts, ns)], woffs, recv, thrd,
                                              accumulate=acc0, divisor=divisor)
        got = o_arena.cpu().numpy()
        for i, (s, n) in enumerate(zip(starts, ns)):
            want = oracle.c.dequant_accumulate([got_w[k, woffs[i]:woffs[i] + wn[i]] for k in range(K)], n, thrd,
                                               acc=base[s:s + n] if acc0 else None)
            if divisor != 1.0:
                want = (want / np.float32(divisor)).astype(np.float32)
            assert_bits_equal(got[s:s + n], want, f"{what}: sum of vector {i} n={n}")
        assert (got[between] == 9.0).all(), what
