"""Forms of the C-ABI that the Python wrappers never use, straight through ctypes, against the CPU oracle:

* nklq_quantize_f32 with add_residual = 1 and THREE distinct buffers (g, r_in, r_out): the
  error-feedback step of necklace/cuda/quantize.py:41-49 applied to g + r_in, written to a residual
  buffer of its own; also r_out == g with a separate r_in.  Every kernel family (flat on and off a
  128-byte line, tail only, bands, row tiles) with the three bases at different element offsets, so
  that each alignment branch of the dispatch is taken;
* the sums over more than NKLQ_MAX_PAYLOADS_PER_LAUNCH payloads (consecutive launches that continue
  one running sum, the division folded into the last): decode of necklace/cuda/quantize.py:80-87.
"""
import ctypes as ct

import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal, assert_words_equal
from gpu_util import dev, host_words
from necklace_amd import _lib
from necklace_amd.frmwrk.pytorch import ptcomp

pytestmark = pytest.mark.gpu

PAD = 64  # floats around every view: 256 bytes, so that a view at offset 0 starts on a 128-byte line


def _view(n, off, fill):
    buf = torch.full((n + 2 * PAD,), fill, dtype=torch.float32, device="cuda")
    assert buf.data_ptr() % 128 == 0
    return buf, buf[PAD + off:PAD + off + n]


def _untouched_outside(buf, off, n, fill):
    lo, hi = PAD + off, PAD + off + n
    return bool((buf[:lo] == fill).all()) and bool((buf[hi:] == fill).all())


def _quantize_three_buffers(A, R0, thrd, og, oi, oo, oc, rout_is_g=False):
    """nklq_quantize_f32(g, r_in, r_out, c, add_residual=1) with g, r_in, r_out at element offsets
    og, oi, oo past a 128-byte line and c at word offset oc.  Returns nothing; asserts everything."""
    L = _lib.lib()
    flat = A.ndim == 1
    n, k = (A.shape[0], 1) if flat else A.shape
    tot, m = n * k, (n + 15) // 16
    gbuf, g = _view(tot, og, 3.0)
    ibuf, rin = _view(tot, oi, 5.0)
    obuf, rout = (gbuf, g) if rout_is_g else _view(tot, oo, 7.0)
    cbuf = torch.full((m * k + 2 * PAD,), -1, dtype=torch.int32, device="cuda")
    c = cbuf[PAD + oc:PAD + oc + m * k]
    g.copy_(torch.from_numpy(A.reshape(-1)))
    rin.copy_(torch.from_numpy(R0.reshape(-1)))
    what = f"n={n} k={k} offsets g={og} r_in={oi} r_out={oo} c={oc} r_out_is_g={rout_is_g}"
    print(what, flush=True)
    _lib.check(L.nklq_quantize_f32(g.data_ptr(), rin.data_ptr(), rout.data_ptr(), c.data_ptr(), n, k, thrd, 1,
                                   torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    want_c, want_r = oracle.c.quantize(A, thrd, R_in=R0)
    assert_words_equal(host_words(c), want_c.reshape(-1), what)
    assert_bits_equal(rout.cpu().numpy(), want_r.reshape(-1), what)
    assert np.array_equal(rin.cpu().numpy().view(np.uint32), R0.reshape(-1).view(np.uint32)), f"r_in modified: {what}"
    if not rout_is_g:
        assert np.array_equal(g.cpu().numpy().view(np.uint32), A.reshape(-1).view(np.uint32)), f"g modified: {what}"
        assert _untouched_outside(obuf, oo, tot, 7.0), what
    assert _untouched_outside(gbuf, og, tot, 3.0), what
    assert _untouched_outside(ibuf, oi, tot, 5.0), what
    assert int((cbuf[:PAD + oc] != -1).sum()) == 0 and int((cbuf[PAD + oc + m * k:] != -1).sum()) == 0, what


def _data(shape, seed, thrd):
    rng = np.random.default_rng(seed)
    A = rng.normal(0, thrd, shape).astype(np.float32)
    R0 = rng.normal(0, 0.6 * thrd, shape).astype(np.float32)
    flatA, flatR = A.reshape(-1), R0.reshape(-1)
    flatA[::41] = np.float32(thrd)  # sums that land exactly on the threshold and next to it
    flatR[::41] = 0.0
    flatA[5::97] = -0.0
    flatR[5::97] = 0.0              # (-0) + (+0) = +0: the add is not a copy
    return A, R0


# (g, r_in, r_out, c) offsets in elements past a 128-byte line.  r_out decides the kernel (off a line:
# the run-dealing flat kernel / pinned tiles); all three 16-byte aligned or not decides ALIGNED.
OFFSETS = [(0, 0, 0, 0), (0, 0, 4, 0), (1, 2, 3, 1), (3, 0, 1, 2), (0, 1, 0, 3), (2, 2, 2, 0), (4, 8, 32, 0),
           (0, 0, 1, 0), (1, 1, 0, 0)]


@pytest.mark.parametrize("n", [1, 100, 255, 256 * 40, 256 * 40 + 17, (1 << 20) + 5])
@pytest.mark.parametrize("og,oi,oo,oc", OFFSETS)
def test_flat_fused_out_of_place(n, og, oi, oo, oc):
    A, R0 = _data((n,), n + og + 3 * oi + 7 * oo, 2e-3)
    _quantize_three_buffers(A, R0, 2e-3, og, oi, oo, oc)


@pytest.mark.parametrize("n,k", [(5000, 3), (403, 65), (50, 384), (16, 3), (47, 17),      # bands
                                 (300, 385), (129, 1000), (40, 8191), (33, 1024), (100, 2048),
                                 (520, 4099), (16 * 41, 4128)])                              # row tiles
@pytest.mark.parametrize("og,oi,oo,oc", OFFSETS)
def test_matrix_fused_out_of_place(n, k, og, oi, oo, oc):
    A, R0 = _data((n, k), n * 13 + k + og + 3 * oi + 7 * oo, 0.01)
    _quantize_three_buffers(A, R0, 0.01, og, oi, oo, oc)


@pytest.mark.parametrize("shape", [(100,), (256 * 40 + 17,), (70001,), (5000, 3), (403, 65), (300, 385), (40, 8191)])
@pytest.mark.parametrize("og,oi", [(0, 0), (0, 1), (3, 2), (4, 0)])
def test_residual_written_over_the_gradient_with_a_separate_residual_in(shape, og, oi):
    A, R0 = _data(shape, sum(shape) + og + 5 * oi, 0.01)
    _quantize_three_buffers(A, R0, 0.01, og, oi, og, 0, rout_is_g=True)


def test_code_words_on_top_of_a_one_row_input_are_refused():
    """With one row the packed words are as many as the elements: c == g (or r_in) is an exact
    coincidence of an output with an input that is not its in-place partner."""
    L = _lib.lib()
    k = 512
    g = torch.zeros(k, device="cuda")
    r = torch.zeros(k, device="cuda")
    ro = torch.zeros(k, device="cuda")
    for rows, cols in ((1, k), (k, 1)):
        assert L.nklq_quantize_f32(g.data_ptr(), r.data_ptr(), ro.data_ptr(), g.data_ptr(), rows, cols, 0.5, 1, None) == -4
        assert L.nklq_quantize_f32(g.data_ptr(), r.data_ptr(), ro.data_ptr(), r.data_ptr(), rows, cols, 0.5, 1, None) == -4
        assert L.nklq_dequantize_f32(g.data_ptr(), g.data_ptr(), rows, cols, 0.5, None) == -4
    torch.cuda.synchronize()
    assert float(g.abs().sum()) == 0.0


# ------------------------------------------------------------------ more payloads than one launch takes

def _messages(rng, K, words):
    return rng.integers(0, 2 ** 32, size=(K, words), dtype=np.uint64).astype(np.uint32)


@pytest.mark.parametrize("K", [17, 32, 33])
@pytest.mark.parametrize("accumulate", [0, 1])
@pytest.mark.parametrize("divisor", [1.0, None, 32.0])   # None: the payload count itself
def test_many_vectors_sum_over_more_than_sixteen_payloads(K, accumulate, divisor):
    L = _lib.lib()
    div = float(K) if divisor is None else divisor
    rng = np.random.default_rng(K * 10 + accumulate)
    sizes = [1, 17, 1023, 1024, 1025, 5000, 70001, 4096 * 3 + 5]
    thrd = 1e-3
    woffs, w = [], 0
    for n in sizes:
        woffs.append(w)
        w += (n + 15) // 16 + 3
    msgs = _messages(rng, K, w)
    dmsgs = dev(msgs)
    arena = torch.zeros(sum(sizes) + 4 * len(sizes), device="cuda")
    accs, bases, pos = [], [], 0
    for i, n in enumerate(sizes):
        off = pos + (i % 4)
        base = rng.normal(0, 1e-2, n).astype(np.float32)
        base[::9] = -0.0
        arena[off:off + n].copy_(torch.from_numpy(base))
        accs.append(arena[off:off + n])
        bases.append(base)
        pos += n + 4
    cnt = len(sizes)
    print(f"K={K} accumulate={accumulate} divisor={div}", flush=True)
    _lib.check(L.nklq_dequant_accumulate_multi_f32(
        cnt, (ct.c_void_p * cnt)(*[a.data_ptr() for a in accs]), (ct.c_uint64 * cnt)(*sizes),
        (ct.c_uint64 * cnt)(*woffs), (ct.c_void_p * K)(*[dmsgs[p].data_ptr() for p in range(K)]), K, thrd,
        accumulate, div, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    for i, n in enumerate(sizes):
        pl = [msgs[p, woffs[i]:woffs[i] + (n + 15) // 16].copy() for p in range(K)]
        want = oracle.c.dequant_accumulate(pl, n, thrd, acc=bases[i] if accumulate else None)
        want = (want / np.float32(div)).astype(np.float32)
        assert_bits_equal(accs[i].cpu().numpy(), want, f"vector {i} n={n} K={K} accumulate={accumulate} / {div}")


@pytest.mark.parametrize("kn", [17, 33])
@pytest.mark.parametrize("average", [True, False])
def test_compressor_with_more_than_sixteen_workers(kn, average):
    """GradCompressor.decompress_sum over kn > 16 receive slots: two or three launches per step."""
    rng = np.random.default_rng(kn)
    sizes = [3000, 10, 4097, 1001, 70000]
    thrd = 2e-3
    gc = ptcomp.GradCompressor(sizes, kn, thrd=thrd, rank=kn - 2)
    grads_np = [rng.normal(0, 2e-3, n).astype(np.float32) for n in sizes]
    grads = [dev(g) for g in grads_np]
    gc.compress(grads)
    torch.cuda.synchronize()
    own = gc.comp.clone()
    msgs = _messages(rng, kn, gc.layout.total_words)
    gc.recv.copy_(dev(msgs))
    gc.recv[gc.rank, :gc.layout.total_words].copy_(own)
    msgs[gc.rank] = own.cpu().numpy().view(np.uint32)
    gc.decompress_sum(grads, average=average, sync=True)
    for i, n in enumerate(sizes):
        if not gc.grd_cmps[i]:
            assert_bits_equal(grads[i].cpu().numpy(), grads_np[i], f"parameter {i} is below the size threshold")
            continue
        wo, nw = gc.layout.word_offset[i], gc.layout.words[i]
        want_own, _ = oracle.c.quantize(grads_np[i], thrd, R_in=np.zeros(n, np.float32))
        assert_words_equal(msgs[gc.rank, wo:wo + nw], want_own, f"parameter {i}: own payload")
        want = oracle.c.dequant_accumulate([msgs[p, wo:wo + nw].copy() for p in range(kn)], n, thrd)
        if average:
            want = (want / np.float32(kn)).astype(np.float32)
        assert_bits_equal(grads[i].cpu().numpy(), want, f"parameter {i} kn={kn} average={average}")


# ------------------------------------------------------------------ few bands, many columns

@pytest.mark.parametrize("n,k", [(16, 400_001), (7, 100_003), (100, 100_003), (144, 50_001), (33, 20_000), (129, 4_096),
                                 (40, 12_345), (257, 1_000)])
@pytest.mark.parametrize("in_place", [True, False])
def test_wide_matrices_of_a_few_bands(n, k, in_place):
    """Fewer than 8 bands of 16 rows, or a last group of fewer than 8: the tile map then cuts the
    bands into segments so that every XCD has work; rows on and off 128-byte lines; the residual
    updated in place (tiles that share lines at their edges) and written to a buffer of its own
    (windows moved onto lines, the codes of each window's last columns computed by its neighbour too)."""
    A, R0 = _data((n, k), n * 3 + k, 0.01)
    if in_place:
        L = _lib.lib()
        g, r = dev(A), dev(R0)
        m = (n + 15) // 16
        c = torch.full((m, k), -1, dtype=torch.int32, device="cuda")
        _lib.check(L.nklq_quantize_f32(g.data_ptr(), r.data_ptr(), r.data_ptr(), c.data_ptr(), n, k, 0.01, 1,
                                       torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        want_c, want_r = oracle.c.quantize(A, 0.01, R_in=R0)
        assert_words_equal(host_words(c), want_c, f"n={n} k={k}")
        assert_bits_equal(r.cpu().numpy(), want_r, f"n={n} k={k}")
        out = torch.full((n, k), 9.0, device="cuda")
        _lib.check(L.nklq_dequantize_f32(out.data_ptr(), c.data_ptr(), n, k, 0.01, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert_bits_equal(out.cpu().numpy(), oracle.c.dequantize(want_c, n, 0.01), f"decode n={n} k={k}")
    else:
        for og, oi, oo, oc in ((0, 0, 0, 0), (1, 2, 3, 1), (0, 0, 5, 0)):
            _quantize_three_buffers(A, R0, 0.01, og, oi, oo, oc)


@pytest.mark.parametrize("thrd", [0.0, -0.25, float("nan")])
def test_tiles_with_thresholds_that_code_a_zero(thrd):
    """With t <= 0 a value of 0 gets code 01: the lanes past the end of a row must not contribute codes."""
    n, k = 37, 1_003
    A, R0 = _data((n, k), 5, 0.01)
    for og, oi, oo, oc in ((0, 0, 0, 0), (1, 2, 3, 1)):
        _quantize_three_buffers(A, R0, thrd, og, oi, oo, oc)
    g, r = dev(A), dev(R0)
    c = torch.full(((n + 15) // 16, k), -1, dtype=torch.int32, device="cuda")
    _lib.check(_lib.lib().nklq_quantize_f32(g.data_ptr(), r.data_ptr(), r.data_ptr(), c.data_ptr(), n, k, thrd, 1,
                                            torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    with np.errstate(invalid="ignore"):
        want_c, want_r = oracle.c.quantize(A, thrd, R_in=R0)
    assert_words_equal(host_words(c), want_c, f"thrd={thrd}")
    assert_bits_equal(r.cpu().numpy(), want_r, f"thrd={thrd}")


# ------------------------------------------------------------------ the remembered overlap check

def test_a_remembered_overlap_check_is_for_exactly_those_tables():
    """The many-vectors calls skip their overlap check when the tables are the ones the thread's last
    checked call had; any other table, also one that differs in a single address, is checked again."""
    import ctypes as ct
    L = _lib.lib()
    vp, u64 = ct.c_void_p, ct.c_uint64
    n = 4096
    rng = np.random.default_rng(9)
    g = [torch.from_numpy(rng.normal(0, 0.01, n).astype(np.float32)).cuda() for _ in range(2)]
    r = [torch.zeros(n, device="cuda") for _ in range(2)]
    c = [torch.zeros(n // 16, dtype=torch.int32, device="cuda") for _ in range(2)]
    ns = (u64 * 2)(n, n)
    tab = lambda ts: (vp * 2)(*[t.data_ptr() for t in ts])
    good = (tab(g), tab(r), tab(c))
    bad_c = (vp * 2)(c[0].data_ptr(), r[1].data_ptr() + 4 * n - 64)      # c[1] ends inside r[1]
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(3):
        assert L.nklq_quantize_multi_f32(2, *good, ns, 0.01, 1, stream) == 0
        assert L.nklq_quantize_multi_f32(2, good[0], good[1], bad_c, ns, 0.01, 1, stream) == -4
    torch.cuda.synchronize()
    for i in range(2):   # three error-feedback steps were launched, none of the refused calls wrote anything
        want_r = np.zeros(n, np.float32)
        for _ in range(3):
            want_c, want_r = oracle.c.quantize(g[i].cpu().numpy(), 0.01, R_in=want_r)
        assert_words_equal(host_words(c[i]), want_c, f"vector {i}")
        assert_bits_equal(r[i].cpu().numpy(), want_r, f"vector {i}")
    acc = [torch.empty(n, device="cuda") for _ in range(2)]
    msg = torch.cat(c).contiguous()
    woff = (u64 * 2)(0, n // 16)
    bases = (vp * 1)(msg.data_ptr())
    over = (vp * 2)(acc[0].data_ptr(), acc[0].data_ptr() + 4 * n - 4)    # acc[1] starts inside acc[0]
    for _ in range(3):
        assert L.nklq_dequant_accumulate_multi_f32(2, tab(acc), ns, woff, bases, 1, 0.01, 0, 1.0, stream) == 0
        assert L.nklq_dequant_accumulate_multi_f32(2, over, ns, woff, bases, 1, 0.01, 0, 1.0, stream) == -4
    torch.cuda.synchronize()
    for i in range(2):
        assert_bits_equal(acc[i].cpu().numpy(),
                          oracle.c.dequantize(msg[i * (n // 16):(i + 1) * (n // 16)].cpu().numpy().view(np.uint32), n, 0.01))
