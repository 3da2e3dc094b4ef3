"""The five benchmark workloads at their full sizes, HIP path vs the CPU oracle.

Every comparison is on identical inputs: data is generated once (numpy on the
host, or torch on the GPU and downloaded) and handed to both sides.
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal, assert_words_equal
from gpu_util import (dev, host_words, random_payloads_gpu, resnet50_segment_sizes, student_t3_gpu,
                      words_like)
from necklace_amd import _lib
from necklace_amd.cuda import quantize as q

pytestmark = pytest.mark.gpu


def test_config1_flat_and_square():
    """N = 1,048,576, g ~ N(0, 0.01), r = 0, thrd 0.005, one step; as the flat vector and as the
    1024 x 1024 matrix the reference wrapper itself could run (bpg=8, tpb=128)."""
    n = 1 << 20
    rng = np.random.default_rng(20240101)
    g = rng.normal(0, 0.01, n).astype(np.float32)
    # flat, fused with a zero residual
    want_c, want_r = oracle.c.quantize(g, 0.005, R_in=np.zeros(n, np.float32))
    dg, dr, dc = dev(g), torch.zeros(n, device="cuda"), words_like(n)
    q.cu_fn_matrix_quantize_e(dg, dc, dr, 0.005, add_residual=True)
    assert_words_equal(host_words(dc), want_c)
    assert_bits_equal(dr.cpu().numpy(), want_r)
    assert host_words(dc).size == 65536
    # square, the reference kernel as is
    G = g.reshape(1024, 1024)
    want_c2, want_r2 = oracle.c.quantize(G, 0.005)
    dG, dR, dC = dev(G), torch.empty(1024, 1024, device="cuda"), words_like(1024, 1024)
    q.cu_fn_matrix_quantize_e(dG, dC, dR, 0.005, bpg=8, tpb=128)
    assert_words_equal(host_words(dC), want_c2)
    assert_bits_equal(dR.cpu().numpy(), want_r2)
    assert want_c2.shape == (64, 1024)
    # same numbers, different bit layout: the two packings must not be confused
    assert not np.array_equal(want_c2.reshape(-1), want_c)
    dB = torch.empty(1024, 1024, device="cuda")
    q.cu_fn_matrix_dequantize_e(dB, dC, dR, 0.005)
    assert_bits_equal(dB.cpu().numpy(), oracle.c.dequantize(want_c2, 1024, 0.005))


def test_config2_resnet50_ten_error_feedback_steps():
    """25,557,032 elements in 161 segments (sigma log-uniform in [1e-4, 1e-2]), thrd 1e-3, 10 steps,
    residual carried; codes and residual compared after every step."""
    sizes = resnet50_segment_sizes()
    n = sum(sizes)
    rng = np.random.default_rng(2)
    sigma = np.repeat((10.0 ** rng.uniform(-4, -2, len(sizes))).astype(np.float32), sizes)
    r_host = np.zeros(n, dtype=np.float32)
    c_host = np.zeros((n + 15) // 16, dtype=np.uint32)
    dr, dc = torch.zeros(n, device="cuda"), words_like(n)
    assert n % 16 == 8
    sent = 0
    for step in range(10):
        g = np.random.default_rng([2, step]).standard_normal(n, dtype=np.float32) * sigma
        oracle.c.fused_quantize_inplace(g, r_host, c_host, 1e-3)
        q.cu_fn_matrix_quantize_e(dev(g), dc, dr, 1e-3, add_residual=True)
        got_c = host_words(dc)
        assert_words_equal(got_c, c_host, f"step {step}")
        assert_bits_equal(dr.cpu().numpy(), r_host, f"step {step}")
        assert int(got_c[-1]) >> 16 == 0  # the last word holds 8 codes
        sent += int(np.count_nonzero(got_c))
    assert sent > 0


def test_config3_receive_side_64_buckets():
    """64 buckets, lengths uniform in [1M, 8M] and not multiples of 16; per bucket the local payload
    (quantize of a seeded gradient) and 7 peers (P(0)=0.9) are decoded and summed in order 0..7."""
    rng = np.random.default_rng(3)
    lens = []
    while len(lens) < 64:
        v = int(rng.integers(1_000_000, 8_000_001))
        if v % 16:
            lens.append(v)
    thrd = 1e-3
    total = 0
    for b, n in enumerate(lens):
        g = student_t3_gpu(n, 1000 + b, scale=1e-3)
        local = words_like(n)
        resid = torch.empty(n, device="cuda")
        q.cu_fn_matrix_quantize_e(g, local, resid, thrd, sync=False)
        peers = random_payloads_gpu(7, n, 2000 + b, garbage_tail=(b % 8 == 5))
        acc = torch.full((n,), float("nan"), device="cuda")
        payloads = [local] + list(peers.unbind(0))
        q.cu_fn_dequantize_accumulate_e(acc, payloads, thrd)
        host_pl = [host_words(p) for p in payloads]
        want = oracle.c.dequant_accumulate(host_pl, n, thrd)
        assert_bits_equal(acc.cpu().numpy(), want, f"bucket {b} n={n}")
        total += n
    assert 64_000_000 <= total <= 512_000_000


def test_config4_gpt2_medium_fused_step_and_round_trip():
    """354,823,168 elements, g = 1e-3 * Student-t(3), r0 ~ N(0, 1e-4), thrd 2e-3: one fused step
    compared in full with the oracle, then the decode round trip."""
    n, thrd = 354_823_168, 2e-3
    g = student_t3_gpu(n, 4)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(44)
    r = torch.randn(n, device="cuda", generator=gen) * 1e-4
    g_host, r_host = g.cpu().numpy(), r.cpu().numpy()
    a = g + r  # fl32(g + r0), the value the step quantizes
    c = words_like(n)
    q.cu_fn_matrix_quantize_e(g, c, r, thrd, add_residual=True)
    c_host = np.empty((n + 15) // 16, dtype=np.uint32)
    oracle.c.fused_quantize_inplace(g_host, r_host, c_host, thrd)
    assert_words_equal(host_words(c), c_host)
    assert torch.equal(r.view(torch.int32), dev(r_host).view(torch.int32)), "residual bits differ"
    assert c_host.size == 22_176_448
    # round trip: decode, compare with the oracle's decode, re-quantize the decode -> same codes
    d = torch.empty(n, device="cuda")
    q.cu_fn_matrix_dequantize_e(d, c, None, thrd)
    want_d = oracle.c.dequantize(c_host, n, thrd)
    assert torch.equal(d.view(torch.int32), dev(want_d).view(torch.int32)), "decode differs"
    c2, r2 = words_like(n), torch.empty(n, device="cuda")
    q.cu_fn_matrix_quantize_e(d, c2, r2, thrd)
    assert torch.equal(c2, c)
    assert not bool(r2.any())
    # what was sent plus what is still owed is the input, up to one rounding of the subtraction
    err = (d.double() + r.double() - a.double()).abs()
    assert bool((err <= a.double().abs() * 2.0 ** -23).all())


def test_config5_hbm_sizing_chunked_error_feedback():
    """2.8e9 elements resident (11.2 GB gradient + 11.2 GB residual + 0.7 GB codes), N(0, 5e-3),
    thrd 1e-2, 5 steps in 268,435,456-element chunks.  One whole-vector launch (indices beyond
    2^31) must equal the chunked result; chunks are checked against the oracle by streaming
    them through the host: all of them on the first and last step, three per step otherwise."""
    n, chunk, thrd = 2_800_000_000, 268_435_456, 1e-2
    starts = list(range(0, n, chunk))
    assert len(starts) == 11 and n - starts[-1] == 115_645_440
    g = torch.empty(n, device="cuda")
    r = torch.zeros(n, device="cuda")
    c = torch.empty((n + 15) // 16, dtype=torch.int32, device="cuda")
    gen = torch.Generator(device="cuda")
    for step in range(5):
        gen.manual_seed(500 + step)
        for lo in starts:
            hi = min(n, lo + chunk)
            torch.randn(hi - lo, device="cuda", generator=gen, out=g[lo:hi])
            g[lo:hi].mul_(5e-3)
        if step == 0:
            r_whole, c_whole = r.clone(), torch.empty_like(c)
            q.cu_fn_matrix_quantize_e(g, c_whole, r_whole, thrd, add_residual=True)
        check = range(len(starts)) if step in (0, 4) else (0, 5, len(starts) - 1)
        for ci, lo in enumerate(starts):
            hi = min(n, lo + chunk)
            verify = ci in check
            if verify:
                g_host, r_host = g[lo:hi].cpu().numpy(), r[lo:hi].cpu().numpy()
            q.cu_fn_matrix_quantize_e(g[lo:hi], c[lo // 16:(hi + 15) // 16], r[lo:hi], thrd,
                                      add_residual=True, sync=False)
            if verify:
                c_host = np.empty((hi - lo + 15) // 16, dtype=np.uint32)
                oracle.c.fused_quantize_inplace(g_host, r_host, c_host, thrd)
                assert_words_equal(host_words(c[lo // 16:(hi + 15) // 16]), c_host, f"step {step} chunk {ci}")
                assert torch.equal(r[lo:hi].view(torch.int32), dev(r_host).view(torch.int32)), \
                    f"residual differs: step {step} chunk {ci}"
        torch.cuda.synchronize()
        if step == 0:
            assert torch.equal(c_whole, c), "whole-vector launch differs from the chunked result"
            assert torch.equal(r_whole.view(torch.int32), r.view(torch.int32))
            del r_whole, c_whole
    assert int((c != 0).sum()) > 0
    # the receive side at the same size, one launch each (element indices beyond 2^31): the decode
    # of all 175,000,000 words and the sum of two payloads, into the gradient's buffer; first,
    # middle and last chunk against the oracle
    del r
    c2 = c.clone()
    c2[::3] = 0
    q.cu_fn_matrix_dequantize_e(g, c, None, thrd)
    for lo in (starts[0], starts[8], starts[-1]):
        hi = min(n, lo + chunk)
        want = oracle.c.dequantize(host_words(c[lo // 16:(hi + 15) // 16]), hi - lo, thrd)
        assert torch.equal(g[lo:hi].view(torch.int32), dev(want).view(torch.int32)), f"decode of chunk at {lo}"
    q.cu_fn_dequantize_accumulate_e(g, [c, c2], thrd)
    for lo in (starts[0], starts[8], starts[-1]):
        hi = min(n, lo + chunk)
        pl = [host_words(x[lo // 16:(hi + 15) // 16]) for x in (c, c2)]
        want = oracle.c.dequant_accumulate(pl, hi - lo, thrd)
        assert torch.equal(g[lo:hi].view(torch.int32), dev(want).view(torch.int32)), f"sum of chunk at {lo}"


@pytest.mark.parametrize("n,k", [(4099, 8191), (1_000_003, 17), (100_003, 384), (50_001, 385), (2_000_001, 3),
                                 (20_011, 1023), (9_001, 2047), (20_005, 1000),
                                 (16, 4_000_001), (100, 1_000_003), (144, 500_001)])   # a few bands, at the benchmark's sizes
def test_large_matrices_every_kernel_regime_against_the_oracle(n, k):
    """Tens of millions of elements per shape: many workgroups per XCD, padded grids (word rows in
    groups of 8, band ranges in runs), rows off 128-byte lines; fused step with a residual, then the
    decode of the words into the same buffer."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(n + k)
    thrd = 2e-3
    A = torch.randn(n, k, device="cuda", generator=gen) * 1e-3
    R = torch.randn(n, k, device="cuda", generator=gen) * 1e-3
    C = torch.full(((n + 15) // 16, k), -1, dtype=torch.int32, device="cuda")
    a_host, r_host = A.cpu().numpy(), R.cpu().numpy()
    q.cu_fn_matrix_quantize_e(A, C, R, thrd, add_residual=True)
    want_c, want_r = oracle.c.quantize(a_host, thrd, R_in=r_host)
    assert_words_equal(C.cpu().numpy().view(np.uint32), want_c, f"{n}x{k} codes")
    assert_bits_equal(R.cpu().numpy(), want_r, f"{n}x{k} residual")
    del a_host, r_host, want_r
    q.cu_fn_matrix_dequantize_e(R, C, None, thrd)
    assert_bits_equal(R.cpu().numpy(), oracle.c.dequantize(want_c, n, thrd), f"{n}x{k} decode")


def test_flat_decode_of_more_code_words_than_the_memory_side_cache_holds():
    """From 2^30 elements the flat decode adds prefetch workgroups by itself (the code words then
    exceed the 256 MB cache).  4.3 GB of output: windows of it are compared with the oracle, at the
    start (no prefetch has run yet), across block boundaries, around 2^32 bytes and at the end."""
    n = (1 << 30) + 4099
    gen = torch.Generator(device="cuda")
    gen.manual_seed(30)
    dc = torch.randint(-2 ** 31, 2 ** 31 - 1, ((n + 15) // 16,), dtype=torch.int32, device="cuda", generator=gen)
    out = torch.full((n,), 9.0, device="cuda")
    q.cu_fn_matrix_dequantize_e(out, dc, None, 2e-3)
    block = 256 * 1024                     # elements of one block of 256 workgroups
    for lo in (0, 15 * block, 16 * block - 4096, 1000 * block - 1024, (1 << 30) - (1 << 20), n - (1 << 20) - 3):
        lo -= lo % 16
        hi = min(n, lo + (1 << 21))
        words = dc[lo // 16:(hi + 15) // 16].cpu().numpy().view(np.uint32)
        assert_bits_equal(out[lo:hi].cpu().numpy(), oracle.c.dequantize(words, hi - lo, 2e-3), f"window at {lo}")
    # and nothing but {+t, -t, +0} anywhere
    t = torch.tensor(2e-3, dtype=torch.float32, device="cuda")
    assert bool(((out == t) | (out == -t) | (out == 0)).all())


@pytest.mark.parametrize("n,k", [(4099, 8191), (20_011, 1023), (1_000_003, 17), (40_000, 8191), (300, 100_003)])
def test_matrix_decode_in_ranges_behind_a_pass_over_the_code_words(n, k):
    """With the prefetch knob on, a matrix of 2^24 elements or more is decoded in ranges of bands
    (at most 64 MiB of code words each; 40,000 x 8191 takes two, 300 x 100,003 three), each behind a
    pass that reads the range's words.  Same bits as the decode in one piece, and as the oracle
    on windows that include the seams."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(n + k)
    C = torch.randint(-2 ** 31, 2 ** 31 - 1, ((n + 15) // 16, k), dtype=torch.int32, device="cuda", generator=gen)
    one, ranged = torch.full((n, k), 9.0, device="cuda"), torch.full((n, k), 9.0, device="cuda")
    old = _lib.tune(_lib.TUNE_DECODE_PREFETCH)
    try:
        _lib.tune(_lib.TUNE_DECODE_PREFETCH, 2)
        q.cu_fn_matrix_dequantize_e(one, C, None, 2e-3)
        _lib.tune(_lib.TUNE_DECODE_PREFETCH, 1)
        q.cu_fn_matrix_dequantize_e(ranged, C, None, 2e-3)
    finally:
        _lib.tune(_lib.TUNE_DECODE_PREFETCH, old)
    assert torch.equal(one.view(torch.int32), ranged.view(torch.int32))
    bands = max(8, (1 << 24) // k // 8 * 8)
    for r0 in (0, 16 * bands - 16, n - min(n, 48)):
        r0 = max(0, min(r0, n - 1)) // 16 * 16
        r1 = min(n, r0 + 48)
        words = C[r0 // 16:(r1 + 15) // 16].cpu().numpy().view(np.uint32)
        assert_bits_equal(ranged[r0:r1].cpu().numpy(), oracle.c.dequantize(words, r1 - r0, 2e-3), f"rows {r0}..{r1}")


@pytest.mark.parametrize("n,k", [(46_349, 46_341), (268_435_461, 9)])
def test_matrix_forms_beyond_2_31_elements(n, k):
    """Matrices of more than 2^31 elements (8.6 and 9.7 GB per array) through the row kernels and
    the band kernels in one launch: slabs of whole word rows at the start, either side of element
    2^31, and at the ragged end are checked against the oracle (a slab of rows 16a..16b of a
    row-major matrix is a matrix of its own, with the word rows a..b)."""
    thrd, m = 2e-3, (n + 15) // 16
    assert n * k > 2 ** 31
    A = torch.empty(n, k, device="cuda")
    R = torch.empty(n, k, device="cuda")
    gen = torch.Generator(device="cuda")
    gen.manual_seed(n % 1000 + k)
    rows_per_piece = max(16, (1 << 26) // k // 16 * 16)
    for lo in range(0, n, rows_per_piece):
        hi = min(n, lo + rows_per_piece)
        torch.randn(hi - lo, k, device="cuda", generator=gen, out=A[lo:hi])
        torch.randn(hi - lo, k, device="cuda", generator=gen, out=R[lo:hi])
    A.mul_(1e-3)
    R.mul_(1e-3)
    C = torch.full((m, k), -1, dtype=torch.int32, device="cuda")
    slab = max(1, (1 << 22) // (16 * k))                      # word rows per slab: about 4 M elements
    mid = (2 ** 31 // k) // 16                                # the word row that holds element 2^31
    slabs = [(0, slab), (max(0, mid - slab // 2), min(m, mid + slab)), (m - slab, m)]
    before = [(A[16 * a:min(n, 16 * b)].cpu().numpy(), R[16 * a:min(n, 16 * b)].cpu().numpy()) for a, b in slabs]
    q.cu_fn_matrix_quantize_e(A, C, R, thrd, add_residual=True)
    wants = []
    for (a, b), (a_host, r_host) in zip(slabs, before):
        want_c, want_r = oracle.c.quantize(a_host, thrd, R_in=r_host)
        assert_words_equal(C[a:b].cpu().numpy().view(np.uint32), want_c, f"{n}x{k} codes of word rows {a}..{b}")
        assert_bits_equal(R[16 * a:min(n, 16 * b)].cpu().numpy(), want_r, f"{n}x{k} residual of word rows {a}..{b}")
        wants.append(want_c)
    assert int((C == -1).sum()) == 0                          # every word was written: no code is ever 11
    q.cu_fn_matrix_dequantize_e(A, C, None, thrd)
    for (a, b), want_c in zip(slabs, wants):
        rows = min(n, 16 * b) - 16 * a
        assert_bits_equal(A[16 * a:16 * a + rows].cpu().numpy(), oracle.c.dequantize(want_c, rows, thrd),
                          f"{n}x{k} decode of word rows {a}..{b}")


@pytest.mark.parametrize("og,orr,oo", [(1, 1, 1), (0, 3, 31), (4, 4, 8), (16, 0, 16), (0, 16, 5)])
def test_large_flat_views_off_cache_lines(og, orr, oo):
    """20 M elements cut out of larger buffers at element offsets: the residual (and the decode
    target) start off a 128-byte line, which takes the run-dealt quantize and the line-shifted
    decode; the guard elements around the views must stay untouched."""
    n, thrd = 20_000_003, 2e-3
    gen = torch.Generator(device="cuda")
    gen.manual_seed(og * 100 + orr * 10 + oo)
    gbuf = torch.randn(n + 64, device="cuda", generator=gen) * 1e-3
    rbuf = torch.randn(n + 64, device="cuda", generator=gen) * 1e-3
    obuf = torch.full((n + 64,), 9.0, device="cuda")
    g, r, out = gbuf[og:og + n], rbuf[orr:orr + n], obuf[oo:oo + n]
    g_host, r_host = g.cpu().numpy(), r.cpu().numpy()
    guard_lo, guard_hi = rbuf[:orr].clone(), rbuf[orr + n:].clone()
    C = words_like(n)
    q.cu_fn_matrix_quantize_e(g, C, r, thrd, add_residual=True)
    want_c, want_r = oracle.c.quantize(g_host, thrd, R_in=r_host)
    assert_words_equal(host_words(C), want_c, "codes")
    assert_bits_equal(r.cpu().numpy(), want_r, "residual")
    assert torch.equal(rbuf[:orr], guard_lo) and torch.equal(rbuf[orr + n:], guard_hi)
    q.cu_fn_matrix_dequantize_e(out, C, None, thrd)
    assert_bits_equal(out.cpu().numpy(), oracle.c.dequantize(want_c, n, thrd), "decode")
    assert float(obuf[:oo].sum()) == 9.0 * oo and float(obuf[oo + n:].sum()) == 9.0 * (64 - oo)
