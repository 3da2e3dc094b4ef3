"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

from necklace_amd.cuda import quantize as q


def dev(a):
    """numpy -> GPU tensor (uint32 travels as int32 bits)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    return torch.from_numpy(a).cuda()


def host_words(t):
    return t.cpu().numpy().view(np.uint32)


def words_like(n, k=None, fill=-1):
    """Packed-code tensor pre-filled with garbage: every valid word must be overwritten."""
    m = (n + 15) // 16
    shape = (m,) if k is None else (m, k)
    return torch.full(shape, fill, dtype=torch.int32, device="cuda")


def gpu_quantize(a_np, thrd, r_in_np=None, offset=(0, 0)):
    """Run the library on a copy of the inputs.  offset = (element offset of g, of r) inside
    larger buffers, to exercise base addresses that are not 16-byte aligned."""
    a_np = np.ascontiguousarray(a_np, dtype=np.float32)
    flat = a_np.ndim == 1
    og, orr = offset
    if flat:
        n = a_np.shape[0]
        gbuf = torch.zeros(n + 8, dtype=torch.float32, device="cuda")
        rbuf = torch.full((n + 8,), 7.0, dtype=torch.float32, device="cuda")
        A = gbuf[og:og + n]
        R = rbuf[orr:orr + n]
        A.copy_(torch.from_numpy(a_np))
        C = words_like(n)
    else:
        n, k = a_np.shape
        A = dev(a_np)
        R = torch.full_like(A, 7.0)
        C = words_like(n, k)
    if r_in_np is not None:
        R.copy_(torch.from_numpy(np.ascontiguousarray(r_in_np, dtype=np.float32)))
    q.cu_fn_matrix_quantize_e(A, C, R, thrd, add_residual=r_in_np is not None)
    if flat:
        # the library must not write outside the views
        assert float(rbuf[:orr].sum()) == 7.0 * orr and float(rbuf[orr + n:].sum()) == 7.0 * (8 - orr)
    assert np.array_equal(A.cpu().numpy().view(np.uint32), a_np.view(np.uint32)), "input A was modified"
    return host_words(C), R.cpu().numpy()


def gpu_dequantize(words_np, n, thrd, k=None, offset=0):
    if k is None:
        buf = torch.full((n + 8,), 9.0, dtype=torch.float32, device="cuda")
        A = buf[offset:offset + n]
    else:
        A = torch.full((n, k), 9.0, dtype=torch.float32, device="cuda")
    q.cu_fn_matrix_dequantize_e(A, dev(words_np), None, thrd)
    if k is None:
        assert float(buf[:offset].sum()) == 9.0 * offset and float(buf[offset + n:].sum()) == 9.0 * (8 - offset)
    return A.cpu().numpy()


def pack_codes_np(codes, n):
    m = (n + 15) // 16
    pad = np.zeros(m * 16, dtype=np.uint32)
    pad[:n] = codes[:n]
    return np.bitwise_or.reduce(pad.reshape(m, 16) << (2 * np.arange(16, dtype=np.uint32)), axis=1).astype(np.uint32)


def student_t3_gpu(n, seed, scale=1e-3):
    """scale * Student-t(3) generated on the GPU (z / sqrt(chi2_3/3)); the oracle gets a download
    of the very same values, so no second generator is involved."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    slab = 1 << 26
    for lo in range(0, n, slab):
        m = min(slab, n - lo)
        z = torch.randn(m, device="cuda", generator=gen)
        chi = torch.zeros(m, device="cuda")
        for _ in range(3):
            chi += torch.randn(m, device="cuda", generator=gen) ** 2
        out[lo:lo + m] = z * torch.rsqrt(chi / 3.0) * scale
    return out


def random_payloads_gpu(k, n, seed, p_zero=0.9, garbage_tail=False):
    """k packed payloads [k, ceil(n/16)] (int32 bits) of i.i.d. codes: P(0)=p_zero, P(1)=P(2),
    never 3; bits past n are 0, or all ones with garbage_tail."""
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    m = (n + 15) // 16
    half = (1.0 - p_zero) / 2
    u = torch.rand(k, m * 16, device="cuda", generator=gen)
    codes = (u < half).to(torch.int64) + 2 * ((u >= half) & (u < 2 * half)).to(torch.int64)
    if n < m * 16:
        codes[:, n:] = 3 if garbage_tail else 0
    shifts = (2 * torch.arange(16, device="cuda", dtype=torch.int64)).view(1, 1, 16)
    words = (codes.view(k, m, 16) << shifts).sum(-1)
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words)
    return words.to(torch.int32).contiguous()


def resnet50_segment_sizes():
    """Element counts of ResNet-50's 161 parameter tensors, in module order."""
    sizes = [64 * 3 * 7 * 7, 64, 64]
    inplanes = 64
    for planes, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
        for b in range(blocks):
            sizes += [planes * inplanes, planes, planes,
                      planes * planes * 9, planes, planes,
                      4 * planes * planes, 4 * planes, 4 * planes]
            if b == 0:
                sizes += [4 * planes * inplanes, 4 * planes, 4 * planes]
            inplanes = 4 * planes
    sizes += [1000 * 2048, 1000]
    assert len(sizes) == 161 and sum(sizes) == 25_557_032
    return sizes
