"""2-bit gradient quantization on MI355X — drop-in for necklace/cuda/quantize.py.

Same public names and keyword arguments as the reference module; the work is
done by the HIP kernels of libnklq.so (include/nklq.h).  Differences a caller
can see, all deliberate:

* `A`, `C`, `R` are torch tensors on the GPU (or numpy arrays with
  ``to_device=True``) instead of numba device arrays; `C` may be torch.uint32
  or torch.int32 (same bits);
* 1-D tensors are accepted and mean the matrix (N, 1): word w packs elements
  16w .. 16w+15;
* `bpg` / `tpb` are accepted and ignored: the library sizes its own launch and
  always covers the whole input, where the reference's fixed (bpg, bpg) grid
  covers at most 16*bpg*tpb/16 word rows x bpg*tpb columns
  (necklace/cuda/quantize.py:98,112);
* the column guard is ``y < A.shape[1]``; the reference tests y against
  ``A.shape[0]`` (:29-31), which only works for square inputs;
* extra keyword arguments: ``add_residual`` (error feedback: a = A + R before
  quantizing, R updated in place) and ``sync`` (the reference always blocks
  until the stream is idle, :104; pass ``sync=False`` to stay asynchronous);
* contiguous tensors only.  The library's entry points take a base pointer and
  (rows, columns) with no leading dimension, so a row-strided view (``M[:, :k]``
  of a wider matrix, a transposed or channels_last tensor) raises ValueError
  here instead of being read with the wrong stride; numba device arrays carry
  their strides and the reference kernels would index such a view correctly.
  necklace's own callers pass flattened gradients
  (necklace/frmwrk/pytorch/ptprms.py:262,374), which
  are contiguous; a caller that holds a strided view passes ``x.contiguous()``
  and copies the residual back.  1-D slices of a flat buffer (``flat[a:b]``) are
  contiguous and are taken at any element offset.
"""
import ctypes as ct

import numpy as np
import torch

from .. import _lib
from . import nbutils

CMP_RATIO = 16  # necklace/cuda/quantize.py:8

g = 0b01  # a >= thrd
e = 0b00  # -thrd < a < thrd
l = 0b10  # a <= -thrd
msk = 0b11  # or mask

_WORD_DTYPES = (torch.int32, torch.uint32)


def packed_rows(n):
    """m of necklace/cuda/quantize.py:145-147."""
    return (n + CMP_RATIO - 1) // CMP_RATIO


def _shape2(t):
    if t.dim() == 1:
        return t.shape[0], 1
    return t.shape[0], t.shape[1]


def _check_f32(name, t, any_rank=False):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a torch tensor, got {type(t).__name__}")
    if t.dtype != torch.float32:
        raise TypeError(f"{name}: expected float32, got {t.dtype}")
    if not any_rank and t.dim() not in (1, 2):
        raise TypeError(f"{name}: expected 1 or 2 dimensions, got {t.dim()}")
    if not t.is_cuda:
        raise TypeError(f"{name}: expected a GPU tensor (pass to_device=True for host arrays)")
    if not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")


def _check_words(name, t, n, k, ndim):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a torch tensor, got {type(t).__name__}")
    if t.dtype not in _WORD_DTYPES:
        raise TypeError(f"{name}: expected uint32 or int32, got {t.dtype}")
    if not t.is_cuda:
        raise TypeError(f"{name}: expected a GPU tensor")
    if not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")
    want = (packed_rows(n),) if ndim == 1 else (packed_rows(n), k)
    if tuple(t.shape) != want and not (ndim == 1 and tuple(t.shape) == (want[0], 1)):
        raise ValueError(f"{name}: shape {tuple(t.shape)} does not match {want} for {n} rows")


def _to_device(x):
    if isinstance(x, torch.Tensor):
        return x.cuda()
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _finish(stream, device, sync):
    if not sync:
        return
    if stream is None:
        torch.cuda.current_stream(device).synchronize()
    elif isinstance(stream, int):
        torch.cuda.synchronize(device)
    else:
        stream.synchronize()


class _on_device:
    """`with torch.cuda.device(d)` only when d is not already the current device: the library launches
    on the current HIP device, and switching back and forth costs more than a small kernel takes."""
    __slots__ = ("ctx",)

    def __init__(self, device):
        self.ctx = None if device.index == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


_fn_cache = {}


def _fn(name):
    """The bound ctypes function of the library in use, looked up once per library."""
    L = _lib.lib()
    f = _fn_cache.get((L, name))
    if f is None:
        f = _fn_cache[(L, name)] = getattr(L, name)
    return f


def _quantize(A, C, R, thrd, add_residual, stream, sync):
    _check_f32("A", A)
    _check_f32("R", R)
    if A.shape != R.shape:
        raise ValueError(f"A {tuple(A.shape)} and R {tuple(R.shape)} differ in shape")
    n, k = _shape2(A)
    _check_words("C", C, n, k, A.dim())
    dev = A.device
    if not (dev == R.device == C.device):
        raise ValueError("A, C and R must be on the same GPU")
    with _on_device(dev):
        h = nbutils.stream_handle(stream, dev)
        rp = R.data_ptr()
        code = _fn("nklq_quantize_f32")(A.data_ptr(), rp if add_residual else None, rp, C.data_ptr(),
                                        n, k, float(thrd), 1 if add_residual else 0, h)
        if code:
            _lib.check(code)
        _finish(stream, dev, sync)


def _dequantize(A, C, thrd, stream, sync):
    _check_f32("A", A)
    n, k = _shape2(A)
    _check_words("C", C, n, k, A.dim())
    dev = A.device
    if dev != C.device:
        raise ValueError("A and C must be on the same GPU")
    with _on_device(dev):
        h = nbutils.stream_handle(stream, dev)
        code = _fn("nklq_dequantize_f32")(A.data_ptr(), C.data_ptr(), n, k, float(thrd), h)
        if code:
            _lib.check(code)
        _finish(stream, dev, sync)


class _Kernel:
    """Stands in for a numba kernel object: ``knl[grid, block, stream](A, C, R, thrd)``.

    (necklace/cuda/quantize.py:112,134.)  Grid and block are accepted and
    ignored; the launch is asynchronous on `stream`, as a numba launch is.
    """

    def __init__(self, name, fn):
        self.__name__ = name
        self._fn = fn

    def __getitem__(self, cfg):
        if not isinstance(cfg, tuple):
            cfg = (cfg,)
        stream = cfg[2] if len(cfg) > 2 else None
        return lambda A, C, R, thrd=0.3: self._fn(A, C, R, thrd, stream)

    def __call__(self, A, C, R, thrd=0.3):
        return self._fn(A, C, R, thrd, None)


cu_knl_matrix_quantize_e = _Kernel(
    "cu_knl_matrix_quantize_e",
    lambda A, C, R, thrd, stream: _quantize(A, C, R, thrd, False, stream, False))
cu_knl_matrix_dequantize_e = _Kernel(
    "cu_knl_matrix_dequantize_e",
    lambda A, C, R, thrd, stream: _dequantize(A, C, thrd, stream, False))


def cu_fn_matrix_quantize_e(A, C, R, thrd=0.3,
                            bpg=4, tpb=128,
                            to_device=False, stream=None,
                            add_residual=False, sync=True):
    """Quantize A to 2-bit codes in C and write the residual to R.

    Signature of necklace/cuda/quantize.py:96-99.  With ``to_device=True`` the
    inputs are host arrays, copied to the GPU first; the results stay on the GPU
    (the reference does the same and drops them, :105-115) and are returned as
    ``(dA, dC, dR)``.
    """
    if to_device:
        A, R, C = _to_device(A), _to_device(R), _to_device(C)
    _quantize(A, C, R, thrd, add_residual, stream, sync)
    return (A, C, R) if to_device else None


def cu_fn_matrix_dequantize_e(A, C, R, thrd=0.3,
                              bpg=4, tpb=128,
                              to_device=False, stream=None, sync=True):
    """Decode C into A (overwrite).  Signature of necklace/cuda/quantize.py:118-121.

    R is unused, exactly as in the reference kernel (:56-87); None is accepted.
    """
    if to_device:
        A, C = _to_device(A), _to_device(C)
        R = _to_device(R) if R is not None else None
    _dequantize(A, C, thrd, stream, sync)
    return (A, C, R) if to_device else None


# ------------------------------------------------------------------ receive side

def cu_fn_dequantize_accumulate_e(acc, payloads, thrd=0.3, accumulate=False, stream=None, sync=True):
    """acc[j] = (((s0 + d_0[j]) + d_1[j]) + ...), d_p = decode of payloads[p], in list order.

    s0 is +0.0 (``accumulate=False``) or the value already in `acc`.  `acc` is a
    1-D float32 GPU tensor of n elements; `payloads` a sequence of 1-D word
    tensors of ceil(n/16) words each, or one 2-D tensor [K, ceil(n/16)].  This is
    the decompress-and-sum step the compressed gradient exchange needs
    (necklace/trainer/tnopmx.py:334-337); the decode is quantize.py:80-87.
    """
    _check_f32("acc", acc)
    if acc.dim() != 1:
        raise TypeError("acc: expected 1 dimension")
    n = acc.shape[0]
    if isinstance(payloads, torch.Tensor):
        if payloads.dim() != 2:
            raise TypeError("payloads: expected a sequence of 1-D tensors or one 2-D tensor")
        payloads = list(payloads.unbind(0))
    if len(payloads) < 1:
        raise ValueError("payloads: at least one is required")
    for i, p in enumerate(payloads):
        _check_words(f"payloads[{i}]", p, n, 1, 1)
        if p.device != acc.device:
            raise ValueError("acc and payloads must be on the same GPU")
    ptrs = (ct.c_void_p * len(payloads))(*[p.data_ptr() for p in payloads])
    with _on_device(acc.device):
        h = nbutils.stream_handle(stream, acc.device)
        _lib.check(_lib.lib().nklq_dequant_accumulate_f32(
            acc.data_ptr(), ptrs, len(payloads), n, float(thrd), 1 if accumulate else 0, h))
        _finish(stream, acc.device, sync)


# ------------------------------------------------------------------ many vectors per launch

def _ptr_array(ptrs):
    return (ct.c_void_p * len(ptrs))(*ptrs)


def cu_fn_quantize_multi_e(grads, comps, resis, thrd=0.3, add_residual=True, stream=None, sync=True):
    """Flat quantize of many vectors with one launch per 96 of them.

    ``grads[i]``, ``resis[i]``: float32 GPU tensors of the same number of elements (any shape,
    contiguous); ``comps[i]``: ceil(numel/16) words.  With ``add_residual`` the residual is read,
    added to the gradient and updated in place (error feedback); otherwise it is only written.
    The per-parameter form of necklace's buffers (grd_resi / grd_comp lists,
    necklace/trainer/tnopmx.py:140-149) maps onto this directly.
    """
    if not (len(grads) == len(comps) == len(resis)):
        raise ValueError("grads, comps and resis must have the same length")
    if not grads:
        return
    dev = grads[0].device
    ns = []
    for i, (gr, cm, rs) in enumerate(zip(grads, comps, resis)):
        _check_f32(f"grads[{i}]", gr, any_rank=True)
        _check_f32(f"resis[{i}]", rs, any_rank=True)
        n = gr.numel()
        if rs.numel() != n:
            raise ValueError(f"resis[{i}] has {rs.numel()} elements, grads[{i}] has {n}")
        _check_words(f"comps[{i}]", cm, n, 1, 1)
        if not (gr.device == cm.device == rs.device == dev):
            raise ValueError("all tensors must be on the same GPU")
        ns.append(n)
    with _on_device(dev):
        h = nbutils.stream_handle(stream, dev)
        _lib.check(_lib.lib().nklq_quantize_multi_f32(
            len(ns), _ptr_array([t.data_ptr() for t in grads]), _ptr_array([t.data_ptr() for t in resis]),
            _ptr_array([t.data_ptr() for t in comps]), (ct.c_uint64 * len(ns))(*ns), float(thrd),
            1 if add_residual else 0, h))
        _finish(stream, dev, sync)


def cu_fn_dequantize_accumulate_multi_e(accs, word_offsets, payloads, thrd=0.3, accumulate=False,
                                        divisor=1.0, stream=None, sync=True):
    """Fixed-order decode-and-sum into many vectors with one launch per 96 of them.

    ``payloads``: one 2-D tensor [K, W] (or a list of K 1-D tensors of W words): the message of
    each of the K peers.  Vector i (``accs[i]``, float32, contiguous) has its code words at
    ``word_offsets[i]`` in every message.  Same sum as `cu_fn_dequantize_accumulate_e`; the
    result is divided by `divisor` (true division) when it is not 1.
    """
    if len(accs) != len(word_offsets):
        raise ValueError("accs and word_offsets must have the same length")
    if isinstance(payloads, torch.Tensor):
        if payloads.dim() != 2:
            raise TypeError("payloads: expected a sequence of 1-D tensors or one 2-D tensor")
        payloads = list(payloads.unbind(0))
    if len(payloads) < 1:
        raise ValueError("payloads: at least one is required")
    if not accs:
        return
    dev = accs[0].device
    w_total = payloads[0].numel()
    for i, p in enumerate(payloads):
        if not isinstance(p, torch.Tensor) or p.dtype not in _WORD_DTYPES or p.dim() != 1:
            raise TypeError(f"payloads[{i}]: expected a 1-D uint32/int32 tensor")
        if not p.is_cuda or not p.is_contiguous() or p.numel() != w_total or p.device != dev:
            raise ValueError(f"payloads[{i}]: must be contiguous, on the same GPU and of equal length")
    ns = []
    for i, (a, wo) in enumerate(zip(accs, word_offsets)):
        _check_f32(f"accs[{i}]", a, any_rank=True)
        if a.device != dev:
            raise ValueError("all tensors must be on the same GPU")
        n = a.numel()
        if wo < 0 or wo + packed_rows(n) > w_total:
            raise ValueError(f"vector {i}: words [{wo}, {wo + packed_rows(n)}) exceed the payload length {w_total}")
        ns.append(n)
    with _on_device(dev):
        h = nbutils.stream_handle(stream, dev)
        _lib.check(_lib.lib().nklq_dequant_accumulate_multi_f32(
            len(ns), _ptr_array([t.data_ptr() for t in accs]), (ct.c_uint64 * len(ns))(*ns),
            (ct.c_uint64 * len(ns))(*[int(w) for w in word_offsets]),
            _ptr_array([p.data_ptr() for p in payloads]), len(payloads), float(thrd),
            1 if accumulate else 0, float(divisor), h))
        _finish(stream, dev, sync)


# ------------------------------------------------------------------ the reference's own smoke

def test_11():
    """The timing smoke of necklace/cuda/quantize.py:139-174 on this implementation: a 224 x 224
    matrix of values in [-1, 0), thrd 0.5, quantize then dequantize, wall time of each printed."""
    from timeit import default_timer as time

    n = 7 * 32
    m = packed_rows(n)
    thrd = 0.5
    A = torch.rand(n, n, device="cuda") - thrd * 2
    R = torch.empty_like(A)
    C = torch.zeros(m, n, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()

    tm = time()
    cu_fn_matrix_quantize_e(A, C, R, thrd)
    print('quantize: ', time() - tm)

    B = torch.empty_like(A)
    tm = time()
    cu_fn_matrix_dequantize_e(B, C, R, thrd)
    print('dequantize: ', time() - tm)
    return A, B, C, R


if __name__ == '__main__':
    test_11()
