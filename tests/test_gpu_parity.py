"""HIP kernels vs the CPU oracle, through the C-ABI, bit for bit.

Codes and residuals: exact bits (NaN matches NaN).  Sums: 0 ULP.
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal, assert_words_equal, bits_to_f32, kat_quant_cases
from gpu_util import dev, gpu_dequantize, gpu_quantize, host_words, pack_codes_np, words_like
from necklace_amd import _lib
from necklace_amd.cuda import quantize as q

pytestmark = pytest.mark.gpu

FLAT_SIZES = list(range(1, 50)) + [63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4095, 4096, 4097,
                                   8191, 12289, 65536 + 5, 1048576 + 17]


def _knobs():
    """Launch geometries to run every flat test under; results must not depend on them."""
    default = tuple(_lib.tune(i) for i in range(_lib.N_TUNE))
    return [default, (1, 64, 1, 3, 1, 0), (2, 128, 0, 0, 2, 1), (4, 256, 1, 3, 3, 2), (4, 1024, 0, 5, 6, 4),
            (2, 512, 1, 6, 0, 6), (1, 1024, 1, 1, 4, 5)]


@pytest.fixture(params=_knobs(), ids=lambda k: f"u{k[0]}-wg{k[1]}-nt{k[2]}-x{k[3]}-xd{k[4]}-xa{k[5]}")
def knobs(request):
    """The default geometry runs on the product library, the others on the measurement build of the
    same source (the only one that carries them)."""
    if request.param == _knobs()[0]:
        yield request.param
        return
    with _lib.use_tuning_library():
        old = [_lib.tune(i) for i in range(_lib.N_TUNE)]
        for i, v in enumerate(request.param):
            _lib.tune(i, v)
        yield request.param
        for i, v in enumerate(old):
            _lib.tune(i, v)


def test_kat_vectors_on_gpu(kat):
    for name, a, t, words, r, _ in kat_quant_cases(kat):
        C, R = gpu_quantize(a, t)
        assert_words_equal(C, words, name)
        assert_bits_equal(R, r, name)
    for v in kat["dequantize"]:
        t = float(bits_to_f32([v["thrd_bits"]])[0])
        words = np.array([int(h, 16) for h in v["words"]], dtype=np.uint32)
        assert_bits_equal(gpu_dequantize(words, v["n"], t), bits_to_f32(v["out_bits"]), v["name"])
    nan_bits = lambda hs: bits_to_f32([("7FC00000" if h == "NAN" else h) for h in hs])
    for v in kat["fused"]:
        t = float(bits_to_f32([v["thrd_bits"]])[0])
        C, R = gpu_quantize(bits_to_f32(v["g_bits"]), t, r_in_np=bits_to_f32(v["r_in_bits"]))
        assert [f"{w:08X}" for w in C] == v["words"], v["name"]
        assert_bits_equal(R, nan_bits(v["r_bits"]), v["name"])
    for v in kat["accumulate"]:
        t = float(bits_to_f32([v["thrd_bits"]])[0])
        pl = [dev(np.array([int(h, 16) for h in p], dtype=np.uint32)) for p in v["payload_words"]]
        if "acc_in_bits" in v:
            acc = dev(bits_to_f32(v["acc_in_bits"]))
            q.cu_fn_dequantize_accumulate_e(acc, pl, t, accumulate=True)
        else:
            acc = torch.full((v["n"],), 3.0, device="cuda")
            q.cu_fn_dequantize_accumulate_e(acc, pl, t)
        assert_bits_equal(acc.cpu().numpy(), nan_bits(v["acc_bits"]), v["name"])


def test_flat_sizes_all_knobs(knobs):
    for n in FLAT_SIZES:
        rng = np.random.default_rng(n)
        a = rng.normal(0, 0.01, n).astype(np.float32)
        r0 = rng.normal(0, 0.004, n).astype(np.float32)
        Cw, Rw = oracle.c.quantize(a, 0.005)
        C, R = gpu_quantize(a, 0.005)
        assert_words_equal(C, Cw, f"plain n={n}")
        assert_bits_equal(R, Rw, f"plain n={n}")
        Cw, Rw = oracle.c.quantize(a, 0.005, R_in=r0)
        C, R = gpu_quantize(a, 0.005, r_in_np=r0)
        assert_words_equal(C, Cw, f"fused n={n}")
        assert_bits_equal(R, Rw, f"fused n={n}")
        assert_bits_equal(gpu_dequantize(Cw, n, 0.005), oracle.c.dequantize(Cw, n, 0.005), f"deq n={n}")


@pytest.mark.parametrize("og,orr", [(1, 1), (2, 3), (3, 0), (0, 1), (1, 2)])
def test_flat_views_at_any_element_offset(og, orr, knobs):
    """Gradient views cut out of a flat buffer: base addresses only 4-byte aligned."""
    for n in (5, 100, 4096 + 3, 70001):
        rng = np.random.default_rng(n + og * 10 + orr)
        a = rng.normal(0, 1e-3, n).astype(np.float32)
        r0 = rng.normal(0, 5e-4, n).astype(np.float32)
        Cw, Rw = oracle.c.quantize(a, 1e-3, R_in=r0)
        C, R = gpu_quantize(a, 1e-3, r_in_np=r0, offset=(og, orr))
        assert_words_equal(C, Cw, f"n={n}")
        assert_bits_equal(R, Rw, f"n={n}")
        assert_bits_equal(gpu_dequantize(Cw, n, 1e-3, offset=orr), oracle.c.dequantize(Cw, n, 1e-3))


@pytest.mark.parametrize("thrd", [0.005, 1e-3, 2e-3, 1e-2, 0.3, 0.5, 0.0, -0.25, 1e-45])
def test_every_float_near_the_threshold_and_specials(thrd):
    t = np.float32(thrd if thrd > 0 else 0.25)
    tb = int(t.view(np.uint32))
    pos = np.arange(tb - 64, tb + 65, dtype=np.int64).astype(np.uint32)
    special = np.array([0x00000000, 0x80000000, 0x00000001, 0x80000001, 0x007FFFFF, 0x807FFFFF,
                        0x00800000, 0x80800000, 0x7F7FFFFF, 0xFF7FFFFF, 0x7F800000, 0xFF800000,
                        0x7FC00000, 0xFFC00001, 0x7F800001], dtype=np.uint32)
    a = np.concatenate([pos, pos | np.uint32(0x80000000), special]).view(np.float32)
    # plain: denormals, signed zeros, infinities and NaN go through untouched or shifted by t
    Cw, Rw = oracle.c.quantize(a, thrd)
    C, R = gpu_quantize(a, thrd)
    assert_words_equal(C, Cw)
    assert_bits_equal(R, Rw)
    # fused with residuals that land the sum on and around the threshold
    with np.errstate(invalid="ignore"):  # inf - inf among the special values
        r0 = (np.float32(t) - a).astype(np.float32)
    r0[~np.isfinite(r0)] = 0
    Cw, Rw = oracle.c.quantize(a, thrd, R_in=r0)
    C, R = gpu_quantize(a, thrd, r_in_np=r0)
    assert_words_equal(C, Cw)
    assert_bits_equal(R, Rw)


@pytest.mark.parametrize("n,k", [(224, 224), (17, 3), (33, 7), (16, 4), (100, 64), (5, 256), (1000, 12),
                                 (1, 1), (31, 2), (64, 1000), (513, 260)])
def test_matrix_layout(n, k):
    """Column-packed (n, k) form; (224, 224) with values in [-1, 0) and thrd 0.5 is the
    reference's own smoke input (necklace/cuda/quantize.py:141-153)."""
    rng = np.random.default_rng(n * 7 + k)
    A = (rng.random((n, k)).astype(np.float32) - np.float32(1.0))
    R0 = rng.normal(0, 0.3, (n, k)).astype(np.float32)
    Cw, Rw = oracle.c.quantize(A, 0.5)
    C, R = gpu_quantize(A, 0.5)
    assert_words_equal(C, Cw)
    assert_bits_equal(R, Rw)
    Cw2, Rw2 = oracle.c.quantize(A, 0.5, R_in=R0)
    C, R = gpu_quantize(A, 0.5, r_in_np=R0)
    assert_words_equal(C, Cw2)
    assert_bits_equal(R, Rw2)
    assert_bits_equal(gpu_dequantize(Cw, n, 0.5, k=k), oracle.c.dequantize(Cw, n, 0.5))
    # all four codes, whatever sits in the words
    junk = rng.integers(0, 2 ** 32, size=Cw.shape, dtype=np.uint64).astype(np.uint32)
    assert_bits_equal(gpu_dequantize(junk, n, 0.5, k=k), oracle.c.dequantize(junk, n, 0.5))


@pytest.mark.parametrize("n,k", [(5000, 3), (2003, 17), (700, 255), (100, 257), (130, 511), (40, 1023), (40, 1024),
                                 (40, 1025), (33, 1030), (50, 4099), (20, 8191), (129, 2048), (16, 1000),
                                 (300, 384), (300, 385), (70, 513), (90, 666), (49, 799), (64, 800), (64, 801)])
@pytest.mark.parametrize("og,orr,oc", [(0, 0, 0), (1, 1, 1), (3, 2, 0), (0, 1, 3)])
def test_matrix_forms_inside_larger_buffers(n, k, og, orr, oc):
    """Every column regime (bands of a few columns, one band per workgroup, row tiles; k a multiple
    of 32, of 4, odd) with the matrices starting at any element of larger buffers; nothing outside
    the views may be written."""
    rng = np.random.default_rng(n * 31 + k + og + 2 * orr + 4 * oc)
    thrd = 0.01
    A = rng.normal(0, 0.01, (n, k)).astype(np.float32)
    A.reshape(-1)[:: 37] = np.float32(thrd)  # exact hits
    R0 = rng.normal(0, 0.004, (n, k)).astype(np.float32)
    m = (n + 15) // 16
    gbuf = torch.zeros(n * k + 8, device="cuda")
    rbuf = torch.full((n * k + 8,), 7.0, device="cuda")
    cbuf = torch.full((m * k + 8,), -1, dtype=torch.int32, device="cuda")
    dA = gbuf[og:og + n * k].view(n, k)
    dR = rbuf[orr:orr + n * k].view(n, k)
    dC = cbuf[oc:oc + m * k].view(m, k)
    dA.copy_(torch.from_numpy(A))
    for fused in (False, True):
        if fused:
            dR.copy_(torch.from_numpy(R0))
        q.cu_fn_matrix_quantize_e(dA, dC, dR, thrd, add_residual=fused)
        want_c, want_r = oracle.c.quantize(A, thrd, R_in=R0 if fused else None)
        what = f"n={n} k={k} offsets={og},{orr},{oc} fused={fused}"
        assert_words_equal(host_words(dC), want_c, what)
        assert_bits_equal(dR.cpu().numpy(), want_r, what)
        assert float(rbuf[:orr].sum()) == 7.0 * orr and float(rbuf[orr + n * k:].sum()) == 7.0 * (8 - orr), what
        assert int(cbuf[:oc].sum()) == -oc and int(cbuf[oc + m * k:].sum()) == -(8 - oc), what
        assert np.array_equal(dA.cpu().numpy().view(np.uint32), A.view(np.uint32)), what
    junk = rng.integers(0, 2 ** 32, size=(m, k), dtype=np.uint64).astype(np.uint32)
    dC.copy_(dev(junk))
    rbuf.fill_(9.0)
    q.cu_fn_matrix_dequantize_e(dR, dC, None, thrd)
    assert_bits_equal(dR.cpu().numpy(), oracle.c.dequantize(junk, n, thrd), f"decode n={n} k={k}")
    assert float(rbuf[:orr].sum()) == 9.0 * orr and float(rbuf[orr + n * k:].sum()) == 9.0 * (8 - orr)


def test_in_place_forms():
    """R may be A itself (plain), and the fused step updates R in place."""
    rng = np.random.default_rng(99)
    n = 10000 + 9
    a = rng.normal(0, 0.01, n).astype(np.float32)
    Cw, Rw = oracle.c.quantize(a, 0.005)
    A = dev(a)
    C = words_like(n)
    q.cu_fn_matrix_quantize_e(A, C, A, 0.005)  # residual written over the input
    assert_words_equal(host_words(C), Cw)
    assert_bits_equal(A.cpu().numpy(), Rw)


def test_reference_style_calls():
    """kernel[grid, block, stream](...), to_device=True, explicit stream, uint32 words."""
    rng = np.random.default_rng(5)
    n = 224
    A = (rng.random((n, n)).astype(np.float32) - np.float32(1.0))
    Cw, Rw = oracle.c.quantize(A, 0.5)
    # to_device=True with host arrays (necklace/cuda/quantize.py:105-108)
    dA, dC, dR = q.cu_fn_matrix_quantize_e(A, np.zeros((14, n), np.uint32), np.empty_like(A), 0.5,
                                           to_device=True)
    assert dC.dtype == torch.uint32
    assert_words_equal(host_words(dC), Cw)
    assert_bits_equal(dR.cpu().numpy(), Rw)
    # subscripted kernel object on a stream of its own (:112)
    s = torch.cuda.Stream()
    dA, dC2, dR2 = dev(A), words_like(n, n), torch.empty(n, n, device="cuda")
    s.wait_stream(torch.cuda.current_stream())
    q.cu_knl_matrix_quantize_e[(8, 8), (8, 128), s](dA, dC2, dR2, 0.5)
    s.synchronize()
    assert_words_equal(host_words(dC2), Cw)
    dB = torch.empty(n, n, device="cuda")
    q.cu_fn_matrix_dequantize_e(dB, dC2, dR2, 0.5, stream=s)
    assert_bits_equal(dB.cpu().numpy(), oracle.c.dequantize(Cw, n, 0.5))


@pytest.mark.parametrize("k_payloads", [1, 2, 8, 16, 17, 35])
def test_accumulate_fixed_order(k_payloads, knobs):
    for n in (1, 15, 16, 17, 1000 + 13, 4096, 100003):
        rng = np.random.default_rng(n + k_payloads)
        pl = []
        for p in range(k_payloads):
            codes = rng.choice([0, 1, 2, 3], size=n, p=[0.6, 0.19, 0.19, 0.02]).astype(np.uint32)
            w = pack_codes_np(codes, n)
            if n % 16:
                w[-1] |= np.uint32((0xFFFFFFFF << (2 * (n % 16))) & 0xFFFFFFFF)  # garbage past the end
            pl.append(w)
        want = oracle.c.dequant_accumulate(pl, n, 1e-3)
        acc = torch.full((n,), 5.0, device="cuda")
        dpl = [dev(w) for w in pl]
        q.cu_fn_dequantize_accumulate_e(acc, dpl, 1e-3)
        assert_bits_equal(acc.cpu().numpy(), want, f"n={n}")
        base = rng.normal(0, 1e-2, n).astype(np.float32)
        want2 = oracle.c.dequant_accumulate(pl, n, 1e-3, acc=base)
        acc2 = dev(base)
        q.cu_fn_dequantize_accumulate_e(acc2, torch.stack(dpl), 1e-3, accumulate=True)
        assert_bits_equal(acc2.cpu().numpy(), want2, f"n={n} accumulate")


@pytest.mark.parametrize("thrd", [0.0, -0.0, -0.25, 1e-45, 3e38, float("inf"), float("-inf"), float("nan")])
def test_accumulate_and_decode_with_unusual_thresholds(thrd):
    """Zero, negative, denormal, huge and non-finite thresholds decode exactly like the reference
    (the sum then takes the compare-and-select form instead of the fused multiply-add one)."""
    rng = np.random.default_rng(77)
    n = 5000 + 11
    pl = [pack_codes_np(rng.integers(0, 4, size=n).astype(np.uint32), n) for _ in range(5)]
    base = rng.normal(0, 1, n).astype(np.float32)
    base[::7] = -0.0
    for acc0 in (None, base):
        with np.errstate(invalid="ignore", over="ignore"):
            want = oracle.c.dequant_accumulate(pl, n, thrd, acc=acc0)
        acc = torch.full((n,), 5.0, device="cuda") if acc0 is None else dev(acc0)
        q.cu_fn_dequantize_accumulate_e(acc, [dev(w) for w in pl], thrd, accumulate=acc0 is not None)
        assert_bits_equal(acc.cpu().numpy(), want, f"thrd={thrd}")
    assert_bits_equal(gpu_dequantize(pl[0], n, thrd), oracle.c.dequantize(pl[0], n, thrd), f"decode thrd={thrd}")


@pytest.mark.parametrize("tbits", [0x00800000, 0x00FFFFFF, 0x01000000, 0x01000001, 0x03800000, 0x7E7FFFFF, 0x7F000000, 0x7F7FFFFF])
def test_accumulate_at_the_ends_of_the_exponent_range(tbits):
    """Thresholds around the smallest normal numbers (t/2 exact or not: that decides between the
    fused multiply-add form and the compare-and-select form) and the largest finite ones, with
    running sums of the threshold's own magnitude: results that are denormal, cancel to zero or
    overflow must carry the same bits as a plain left-to-right fp32 sum."""
    t = float(np.array([tbits], dtype=np.uint32).view(np.float32)[0])
    rng = np.random.default_rng(tbits & 0xFFFF)
    n = 4096 + 37
    pl = [pack_codes_np(rng.integers(0, 4, size=n).astype(np.uint32), n) for _ in range(6)]
    with np.errstate(over="ignore"):
        base = (rng.uniform(-3, 3, n) * t).astype(np.float32)      # a few thresholds away from zero
    base[::5] = (rng.integers(-3, 4, size=len(base[::5])) * np.float32(t)).astype(np.float32) if t < 1e38 else base[::5]
    for acc0 in (None, base):
        with np.errstate(invalid="ignore", over="ignore"):
            want = oracle.c.dequant_accumulate(pl, n, t, acc=None if acc0 is None else acc0.copy())
        acc = torch.full((n,), 5.0, device="cuda") if acc0 is None else dev(acc0)
        q.cu_fn_dequantize_accumulate_e(acc, [dev(w) for w in pl], t, accumulate=acc0 is not None)
        assert_bits_equal(acc.cpu().numpy(), want, f"t=0x{tbits:08X} accumulate={acc0 is not None}")


def test_accumulate_keeps_signed_zero_like_the_reference():
    """-0.0 + (+0.0) is +0.0: an all-zero payload turns a -0.0 running sum into +0.0, on both sides."""
    n = 2048 + 3
    zeros = np.zeros((n + 15) // 16, dtype=np.uint32)
    base = np.full(n, -0.0, dtype=np.float32)
    want = oracle.c.dequant_accumulate([zeros], n, 1e-3, acc=base)
    acc = dev(base)
    q.cu_fn_dequantize_accumulate_e(acc, [dev(zeros)], 1e-3, accumulate=True)
    assert_bits_equal(acc.cpu().numpy(), want)
    assert not np.signbit(want).any()


def test_round_trip_and_zero_residual_on_gpu():
    rng = np.random.default_rng(21)
    n = 1 << 20
    a = rng.standard_t(3, n).astype(np.float32) * np.float32(1e-3)
    C, R = gpu_quantize(a, 2e-3)
    d = gpu_dequantize(C, n, 2e-3)
    C2, R2 = gpu_quantize(d, 2e-3)
    assert_words_equal(C2, C)
    assert not R2.any()


def test_many_vectors_in_one_launch(knobs):
    """nklq_quantize_multi_f32 / nklq_dequant_accumulate_multi_f32: 105 vectors of awkward lengths
    (more than one table of 96), some at odd element offsets, each equal to its own flat result."""
    sizes = [1, 15, 16, 17, 255, 256, 257, 511, 1023, 1024, 1025, 2047, 4096, 5000, 70001] * 7
    rng = np.random.default_rng(314)
    thrd, K = 1e-3, 3
    arena_g = torch.zeros(sum(sizes) + 4 * len(sizes), device="cuda")
    arena_r = torch.zeros_like(arena_g)
    grads, resis, comps, gh, rh = [], [], [], [], []
    pos = 0
    for i, n in enumerate(sizes):
        off = pos + (i % 4)  # every alignment class of the base address
        g = rng.normal(0, 1e-3, n).astype(np.float32)
        r = rng.normal(0, 5e-4, n).astype(np.float32)
        arena_g[off:off + n].copy_(torch.from_numpy(g))
        arena_r[off:off + n].copy_(torch.from_numpy(r))
        grads.append(arena_g[off:off + n])
        resis.append(arena_r[off:off + n])
        comps.append(words_like(n))
        gh.append(g)
        rh.append(r)
        pos += n + 4
    q.cu_fn_quantize_multi_e(grads, comps, resis, thrd, add_residual=True)
    for i, n in enumerate(sizes):
        want_c, want_r = oracle.c.quantize(gh[i], thrd, R_in=rh[i])
        assert_words_equal(host_words(comps[i]), want_c, f"vector {i} n={n}")
        assert_bits_equal(resis[i].cpu().numpy(), want_r, f"vector {i} n={n}")
    # plain form: residual only written
    outs = [torch.full((n,), 3.0, device="cuda") for n in sizes]
    q.cu_fn_quantize_multi_e(grads, comps, outs, thrd, add_residual=False)
    for i in (0, 4, 9, 14, 44, 95, 96, 104):
        want_c, want_r = oracle.c.quantize(gh[i], thrd)
        assert_words_equal(host_words(comps[i]), want_c)
        assert_bits_equal(outs[i].cpu().numpy(), want_r)
    # receive side: K messages, vector i's words at word_offsets[i] in each
    woffs, w = [], 0
    for n in sizes:
        woffs.append(w)
        w += (n + 15) // 16 + 1  # a gap word between vectors
    msgs = rng.integers(0, 2 ** 32, size=(K, w), dtype=np.uint64).astype(np.uint32)
    dmsgs = dev(msgs)
    for acc0 in (False, True):
        accs = [torch.full((n,), 0.5, device="cuda") for n in sizes]
        q.cu_fn_dequantize_accumulate_multi_e(accs, woffs, dmsgs, thrd, accumulate=acc0)
        for i, n in enumerate(sizes):
            pl = [msgs[k, woffs[i]:woffs[i] + (n + 15) // 16].copy() for k in range(K)]
            want = oracle.c.dequant_accumulate(pl, n, thrd, acc=np.full(n, 0.5, np.float32) if acc0 else None)
            assert_bits_equal(accs[i].cpu().numpy(), want, f"vector {i} n={n} accumulate={acc0}")
    # with the division by the number of workers folded in (7 is not a power of two)
    accs = [torch.empty(n, device="cuda") for n in sizes]
    q.cu_fn_dequantize_accumulate_multi_e(accs, woffs, dmsgs, thrd, divisor=7.0)
    for i, n in enumerate(sizes):
        pl = [msgs[k, woffs[i]:woffs[i] + (n + 15) // 16].copy() for k in range(K)]
        want = (oracle.c.dequant_accumulate(pl, n, thrd) / np.float32(7.0)).astype(np.float32)
        assert_bits_equal(accs[i].cpu().numpy(), want, f"vector {i} n={n} divided")


@pytest.mark.parametrize("divisor", [2.0, 8.0, 64.0, 0.25, -4.0, 2.0 ** 100, 2.0 ** -100, 2.0 ** 126, 2.0 ** -126,
                                     2.0 ** 127, 2.0 ** -127, 3.0, 1.0000001, float("inf")])
@pytest.mark.parametrize("thrd", [1e-3, 3e-38, 1e38])
def test_division_folded_into_the_sum(divisor, thrd):
    """The `/ kn` after the sum is a true IEEE division.  For a divisor that is a power of two the
    kernel multiplies by the exact reciprocal instead, which must give the same bits everywhere:
    quotients that are denormal, that underflow to zero, that overflow, and divisors whose
    reciprocal is not a normal number (those, like every other divisor, are divided)."""
    rng = np.random.default_rng(77)
    n, K = 5000 + 11, 5
    msgs = rng.integers(0, 2 ** 32, size=(K, (n + 15) // 16), dtype=np.uint64).astype(np.uint32)
    with np.errstate(over="ignore"):  # thrd = 1e38: some values become infinite, on purpose
        base = (rng.standard_normal(n) * thrd * 2).astype(np.float32)
    base[:4] = [0.0, -0.0, np.float32(thrd), -np.float32(thrd)]
    for acc0 in (False, True):
        acc = dev(base.copy())
        q.cu_fn_dequantize_accumulate_multi_e([acc], [0], dev(msgs), thrd, accumulate=acc0, divisor=divisor)
        with np.errstate(all="ignore"):
            want = (oracle.c.dequant_accumulate(list(msgs), n, thrd, acc=base if acc0 else None)
                    / np.float32(divisor)).astype(np.float32)
        assert_bits_equal(acc.cpu().numpy(), want, f"divisor={divisor} thrd={thrd} accumulate={acc0}")


def test_two_host_threads_on_two_streams():
    """The library keeps no per-call state: two host threads driving two streams at once get the
    same bits as one after the other."""
    import threading
    rng = np.random.default_rng(55)
    n = 3_000_000 + 5
    work = []
    for i in range(2):
        g = rng.normal(0, 1e-3, n).astype(np.float32)
        r = rng.normal(0, 5e-4, n).astype(np.float32)
        work.append((g, r, oracle.c.quantize(g, 1e-3, R_in=r)))
    results, errors = [None, None], []

    def run(i):
        try:
            torch.cuda.set_device(0)
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                dg, dr, dc = dev(work[i][0]), dev(work[i][1]), words_like(n)
                for _ in range(20):  # keep both streams busy at the same time
                    dr.copy_(dev(work[i][1]))
                    q.cu_fn_matrix_quantize_e(dg, dc, dr, 1e-3, add_residual=True, stream=s, sync=False)
                s.synchronize()
                results[i] = (host_words(dc), dr.cpu().numpy())
        except Exception as exc:  # surfaced below, in the main thread
            errors.append(exc)

    threads = [threading.Thread(target=run, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(2):
        assert_words_equal(results[i][0], work[i][2][0], f"thread {i}")
        assert_bits_equal(results[i][1], work[i][2][1], f"thread {i}")


def test_one_thread_turns_the_knobs_while_another_launches():
    """The launch knobs are process-wide atomics and every call works from one snapshot of them:
    a thread that keeps changing them must not disturb the results (or the launches) of another.
    (On the measurement build: the product library has one workgroup shape.)"""
    with _lib.use_tuning_library():
        _turn_the_knobs_while_another_thread_launches()


def _turn_the_knobs_while_another_thread_launches():
    import threading
    rng = np.random.default_rng(56)
    n = 1_000_000 + 77
    g = rng.normal(0, 1e-3, n).astype(np.float32)
    r = rng.normal(0, 5e-4, n).astype(np.float32)
    want_c, want_r = oracle.c.quantize(g, 1e-3, R_in=r)
    want_d = oracle.c.dequantize(want_c, n, 1e-3)
    old = [_lib.tune(i) for i in range(_lib.N_TUNE)]
    stop = threading.Event()

    def turn():
        k = 0
        while not stop.is_set():
            k += 1
            _lib.tune(_lib.TUNE_CHUNKS_PER_WAVE, (1, 2, 4)[k % 3])
            _lib.tune(_lib.TUNE_WORKGROUP_SIZE, (64, 128, 256, 512, 1024)[k % 5])
            _lib.tune(_lib.TUNE_NONTEMPORAL, k % 2)
            _lib.tune(_lib.TUNE_XCD_INTERLEAVE_LOG2, k % 7)
            _lib.tune(_lib.TUNE_XCD_INTERLEAVE_LOG2_DECODE, (k // 2) % 7)
            _lib.tune(_lib.TUNE_XCD_INTERLEAVE_LOG2_ACCUMULATE, (k // 3) % 7)

    t = threading.Thread(target=turn)
    t.start()
    try:
        dg, dr0 = dev(g), dev(r)
        for _ in range(40):
            dr, dc = dr0.clone(), words_like(n)
            q.cu_fn_matrix_quantize_e(dg, dc, dr, 1e-3, add_residual=True)
            assert_words_equal(host_words(dc), want_c)
            assert_bits_equal(dr.cpu().numpy(), want_r)
            out = torch.full((n,), 5.0, device="cuda")
            q.cu_fn_dequantize_accumulate_e(out, [dc, dc], 1e-3)
            q.cu_fn_matrix_dequantize_e(out, dc, None, 1e-3)
            assert_bits_equal(out.cpu().numpy(), want_d)
    finally:
        stop.set()
        t.join()
        for i, v in enumerate(old):
            _lib.tune(i, v)



@pytest.mark.parametrize("n", [8_388_608, 8_388_608 + 5, 20_000_003, (256 + 8) * 1024 * 40 + 777])
def test_flat_decode_with_prefetching_workgroups(n):
    """The flat decode with its prefetch workgroups switched on (the library does that by itself only
    from 2^30 elements): 8 extra workgroups behind every 256, which only read code words ahead; the
    256 in front must still write exactly their pieces.  Product geometry and two others."""
    rng = np.random.default_rng(n % 1000)
    words = rng.integers(0, 2 ** 32, size=(n + 15) // 16, dtype=np.uint64).astype(np.uint32)
    want = oracle.c.dequantize(words, n, 3e-3)
    dc = dev(words)
    old = _lib.tune(_lib.TUNE_DECODE_PREFETCH)
    try:
        for mode in (1, 2, 0):
            _lib.tune(_lib.TUNE_DECODE_PREFETCH, mode)
            out = torch.full((n,), 9.0, device="cuda")
            q.cu_fn_matrix_dequantize_e(out, dc, None, 3e-3)
            assert_bits_equal(out.cpu().numpy(), want, f"n={n} prefetch knob {mode}")
    finally:
        _lib.tune(_lib.TUNE_DECODE_PREFETCH, old)
    with _lib.use_tuning_library():
        old = [_lib.tune(i) for i in range(_lib.N_TUNE)]
        try:
            _lib.tune(_lib.TUNE_DECODE_PREFETCH, 1)
            for u, wg in ((2, 128), (1, 512)):
                _lib.tune(_lib.TUNE_CHUNKS_PER_WAVE, u)
                _lib.tune(_lib.TUNE_WORKGROUP_SIZE, wg)
                out = torch.full((n,), 9.0, device="cuda")
                q.cu_fn_matrix_dequantize_e(out, dc, None, 3e-3)
                assert_bits_equal(out.cpu().numpy(), want, f"n={n} prefetch, {u} chunks per wave, workgroup {wg}")
        finally:
            for i, v in enumerate(old):
                _lib.tune(i, v)


def test_empty_inputs_are_no_ops():
    e = torch.empty(0, device="cuda")
    w = torch.empty(0, dtype=torch.int32, device="cuda")
    q.cu_fn_matrix_quantize_e(e, w, e.clone(), 0.5)
    q.cu_fn_matrix_dequantize_e(e, w, None, 0.5)
    q.cu_fn_dequantize_accumulate_e(e, [w], 0.5)
    q.cu_fn_quantize_multi_e([e], [w], [e.clone()], 0.5)
    q.cu_fn_quantize_multi_e([], [], [], 0.5)
    m = torch.empty(0, 7, device="cuda")
    q.cu_fn_matrix_quantize_e(m, torch.empty(0, 7, dtype=torch.int32, device="cuda"), m.clone(), 0.5)
    torch.cuda.synchronize()


def test_nbutils_helpers_and_kernel_object_decode():
    """The device helpers of necklace/cuda/nbutils.py:11-39 on torch, and the subscripted decode
    kernel (necklace/cuda/quantize.py:134)."""
    from necklace_amd.cuda import nbutils
    nbutils.cuda_select_device(0)
    assert nbutils.cuda_current_context() == torch.device("cuda", 0)
    s = nbutils.cuda_stream()
    rng = np.random.default_rng(9)
    n = 64
    A = (rng.random((n, n)).astype(np.float32) - np.float32(1.0))
    dA = nbutils.cuda_to_device(A, s)
    dC = nbutils.cuda_to_device(np.zeros((4, n), np.uint32), s)
    dR = nbutils.cuda_to_device(np.empty_like(A), s)
    s.synchronize()
    assert nbutils.cuda_devarr_c_void_p(dA).value == dA.data_ptr()
    q.cu_knl_matrix_quantize_e[(4, 4), (8, 128), s](dA, dC, dR, 0.5)
    dB = torch.empty(n, n, device="cuda")
    q.cu_knl_matrix_dequantize_e[(4, 4), (8, 128), s](dB, dC, dR, 0.5)
    s.synchronize()
    want_c, want_r = oracle.c.quantize(A, 0.5)
    assert_words_equal(host_words(dC), want_c)
    assert_bits_equal(dR.cpu().numpy(), want_r)
    assert_bits_equal(dB.cpu().numpy(), oracle.c.dequantize(want_c, n, 0.5))
    # to_device=True decode from host arrays
    hB, hC, _ = q.cu_fn_matrix_dequantize_e(np.empty_like(A), want_c, None, 0.5, to_device=True)
    assert_bits_equal(hB.cpu().numpy(), oracle.c.dequantize(want_c, n, 0.5))


def test_the_reference_smoke_runs_and_is_consistent(capsys):
    A, B, C, R = q.test_11()
    out = capsys.readouterr().out
    assert "quantize:" in out and "dequantize:" in out
    want_c, want_r = oracle.c.quantize(A.cpu().numpy(), 0.5)
    assert_words_equal(host_words(C), want_c)
    assert_bits_equal(R.cpu().numpy(), want_r)
    assert_bits_equal(B.cpu().numpy(), oracle.c.dequantize(want_c, 224, 0.5))
