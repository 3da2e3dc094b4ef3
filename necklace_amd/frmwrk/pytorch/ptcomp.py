"""Trainer-side buffers and steps for 2-bit compressed gradient exchange.

necklace's trainer prepares gradient compression with

    grd_resi, grd_recv, grd_comp, grd_cmps = mxprms.init_grads_compression(
        params, kn, grd_siz_thrd=...)                  (necklace/trainer/tnopmx.py:135-151)
    mxprms.grads_do_nccl(params, prm_recvs, nc, kn, grad_comp_cfg=cfg)   (:334-337)

but the module behind those calls is not in the reference tree, and the PyTorch
trainers only pass ``grad_comp_cfg`` along without using it
(necklace/frmwrk/pytorch/ptprms.py:319-401).  This module is that missing piece
for PyTorch-ROCm, laid out for one big GPU: ONE flat residual buffer, ONE flat
buffer of packed codes (the payload a rank sends) and ONE ``[kn, words]``
receive buffer (what an all-gather of the payloads fills), with per-parameter
views into them.  Every compressed parameter starts on a word boundary, so the
whole payload is exchanged as a single contiguous ``uint32`` message.

Steps (all on the GPU, through the kernels of libnklq.so):

    compress      a = grad + resi; codes -> comp; resi <- a - decode(codes)
    exchange      (caller's all-gather of `comp` into `recv`; not part of this module —
                   with one GPU the peers' slots are filled by the caller)
    decompress    grad <- sum over ranks, in rank order, of decode(recv[k]);  / kn

Semantics that the reference leaves open and this module fixes: error feedback
is an fp32 add before quantizing; the sum over ranks is a strict left-to-right
fp32 sum in rank order (fp32 sums of {0, +t, -t} depend on the order).
"""
import ctypes as ct
import operator

import torch

from ... import _lib
from ...cuda import nbutils as _nb
from ...cuda import quantize as _q

_data_ptr = torch.Tensor.data_ptr

CMP_RATIO = _q.CMP_RATIO
DEFAULT_SIZE_THRESHOLD = 1001  # grad_size_threshold default, necklace/trainer/tnopmx.py:137
DEFAULT_COMP_THRESHOLD = 0.5   # grad_comp_threshold default, necklace/trainer/tnopmx.py:138
DEFAULT_CHUNK = 268_435_456    # elements per launch of the chunked driver (1 GiB of fp32)


def _sync(device, stream):
    if stream is None:
        torch.cuda.current_stream(device).synchronize()
    else:
        stream.synchronize()


class _stream_ctx:
    """`with torch.cuda.stream(s)` for a torch stream; nothing for None (the current stream is the
    one) or a raw handle (torch cannot enter it: the caller orders such work itself)."""
    __slots__ = ("ctx",)

    def __init__(self, stream):
        self.ctx = None if stream is None or isinstance(stream, int) else torch.cuda.stream(stream)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


def _numel(p):
    if isinstance(p, int):
        return p
    if isinstance(p, torch.Tensor):
        return p.numel()
    return p.data.numel() if hasattr(p, "data") else int(p)


class GradCompLayout:
    """Which parameters are compressed and where their residual / code words live.

    Parameters with fewer than `size_threshold` elements are left alone (the
    reference's ``grad_size_threshold``); the others get consecutive slices of the
    flat residual (elements) and of the flat payload (words, ceil(numel/16) each).
    Slices start at multiples of 256 elements / 16 words: the kernels move 256-element
    chunks (1 KiB of fp32, 64 B of codes) and run 5-7 % faster when chunks do not straddle
    1 KiB address boundaries.  The padding words stay zero.
    """
    ELEM_ALIGN = 256
    WORD_ALIGN = 16

    def __init__(self, numels, size_threshold=DEFAULT_SIZE_THRESHOLD):
        self.numels = [int(n) for n in numels]
        self.size_threshold = int(size_threshold)
        self.compressed = [n >= self.size_threshold and n > 0 for n in self.numels]
        self.elem_offset, self.word_offset, self.words = [], [], []
        eo = wo = 0
        for n, c in zip(self.numels, self.compressed):
            w = _q.packed_rows(n) if c else 0
            self.elem_offset.append(eo if c else None)
            self.word_offset.append(wo if c else None)
            self.words.append(w)
            if c:
                eo = -(-(eo + n) // self.ELEM_ALIGN) * self.ELEM_ALIGN
                wo = -(-(wo + w) // self.WORD_ALIGN) * self.WORD_ALIGN
        self.total_elems, self.total_words = eo, wo

    def __len__(self):
        return len(self.numels)


class GradCompressor:
    """Flat buffers + the compress / decompress steps for one model replica."""

    def __init__(self, params, kn, thrd=DEFAULT_COMP_THRESHOLD, size_threshold=DEFAULT_SIZE_THRESHOLD,
                 device="cuda", rank=None):
        """`rank`: this worker's index among the kn.  Known, this rank's payload is written straight
        into its own slot of the receive buffer (the all-gather can then run in place).  None with
        several workers (the reference's set-up call, necklace/trainer/tnopmx.py:140-143, does not
        pass one): the payload gets a buffer of its own, and whatever needs to know who this worker
        is (a reduce onto a root) raises instead of assuming worker 0."""
        if kn < 1:
            raise ValueError("kn (number of workers) must be >= 1")
        if rank is None and kn == 1:
            rank = 0
        if rank is not None and not 0 <= rank < kn:
            raise ValueError("rank must be in [0, kn)")
        self.kn, self.rank, self.thrd = int(kn), (None if rank is None else int(rank)), float(thrd)
        self.layout = GradCompLayout([_numel(p) for p in params], size_threshold)
        lay = self.layout
        self.device = torch.device(device)
        self.resi = torch.zeros(lay.total_elems, dtype=torch.float32, device=self.device)
        # slot k of `recv` holds rank k's payload; this rank's own slot doubles as `comp`
        self.recv = torch.zeros(self.kn, max(lay.total_words, 1), dtype=torch.int32, device=self.device)
        if self.rank is None:
            self.comp = torch.zeros(max(lay.total_words, 1), dtype=torch.int32, device=self.device)[:lay.total_words]
        else:
            self.comp = self.recv[self.rank, :lay.total_words]
        self.grd_cmps = list(lay.compressed)
        self.grd_resi, self.grd_comp, self.grd_recv = [], [], []
        for i in range(len(lay)):
            if lay.compressed[i]:
                eo, wo, n, w = lay.elem_offset[i], lay.word_offset[i], lay.numels[i], lay.words[i]
                self.grd_resi.append(self.resi[eo:eo + n])
                self.grd_comp.append(self.comp[wo:wo + w])
                self.grd_recv.append(self.recv[:, wo:wo + w])
            else:
                self.grd_resi.append(None)
                self.grd_comp.append(None)
                self.grd_recv.append(None)
        # argument tables of the many-vectors entry points: everything but the gradients' own
        # addresses is fixed for the life of the buffers (built on first use, per subset of
        # parameters that have a gradient)
        self._idx = [i for i, c in enumerate(self.grd_cmps) if c]
        self._pick = (operator.itemgetter(*self._idx) if len(self._idx) > 1
                      else (lambda seq, idx=tuple(self._idx): tuple(seq[i] for i in idx)))
        self._live_key, self._live_tabs = None, None
        self._addr_cache = {}
        # what Tensor.get_device() returns for tensors that live where the buffers do; host tensors
        # (-1) never match: there is no CPU path
        self._dev_index = self.resi.get_device() if self.resi.is_cuda else -2
        self._pl_arr = (ct.c_void_p * self.kn)(*[self.recv[k].data_ptr() for k in range(self.kn)])

    def _tables(self, tensors, what, stream=None):
        """Argument tables for the compressed parameters whose tensor is present (not None) in this
        call.  Returns (count, ptrs, r, c, n, word_offset, staged); `staged` lists (tensor,
        contiguous temporary) pairs for tensors that are not contiguous (their temporary is what the
        kernels see).

        Gradients normally keep their storage from step to step (also when `.grad` is a new tensor
        object every step: the allocator hands out the same blocks), so the tables are cached on the
        tuple of their addresses: a steady-state call costs one pass that reads the addresses and
        nothing else (no ctypes arrays are rebuilt, no tensor is examined again).  Sizes and types
        are looked at when an address changes, not on a hit: they belong to the parameter, not to
        the step, and a tensor of another size at the very address its predecessor had is taken
        for the predecessor."""
        if len(tensors) != len(self.layout):
            raise ValueError(f"expected {len(self.layout)} {what}s, got {len(tensors)}")
        try:
            key = tuple(map(_data_ptr, self._pick(tensors)))
        except TypeError:  # a parameter without a tensor this step
            key = tuple([0 if tensors[i] is None else tensors[i].data_ptr() for i in self._idx])
        hit = self._addr_cache.get(what)
        if hit is not None and hit[0] == key:
            return hit[1]
        # something moved (or this is the first call): look at every tensor; what exactly is wrong is
        # worked out only when something is
        live, addrs, staged = [], [], []
        numels, f32, dev_index = self.layout.numels, torch.float32, self._dev_index
        for i in self._idx:
            t = tensors[i]
            if t is None:
                continue
            if t.numel() != numels[i] or t.dtype is not f32 or t.get_device() != dev_index:
                self._refuse(tensors, what)
            if not t.is_contiguous():
                # e.g. a channels_last gradient: the kernels take flat memory, so it goes through a
                # contiguous copy (and back, for an output)
                with _stream_ctx(stream):
                    tmp = t.contiguous()
                staged.append((t, tmp))
                t = tmp
            live.append(i)
            addrs.append(t.data_ptr())
        lkey = tuple(live)
        if lkey != self._live_key:
            m = len(live)
            self._live_key = lkey
            self._live_tabs = (
                (ct.c_void_p * m)(*[self.grd_resi[i].data_ptr() for i in live]),
                (ct.c_void_p * m)(*[self.grd_comp[i].data_ptr() for i in live]),
                (ct.c_uint64 * m)(*[self.layout.numels[i] for i in live]),
                (ct.c_uint64 * m)(*[self.layout.word_offset[i] for i in live]))
        tabs = (len(live), (ct.c_void_p * len(live))(*addrs)) + self._live_tabs + (staged,)
        # temporaries are new memory every call: only tables without them can be kept (one set for the
        # gradients, one for the outputs, which may be other tensors)
        self._addr_cache[what] = (key, tabs) if not staged else None
        return tabs

    def _refuse(self, tensors, what):
        """Raise for the first tensor that does not fit: sizes first, then type, layout, device."""
        live = [i for i in self._idx if tensors[i] is not None]
        for i in live:
            if tensors[i].numel() != self.layout.numels[i]:
                raise ValueError(
                    f"{what} {i}: {tensors[i].numel()} elements, layout has {self.layout.numels[i]}")
        for i in live:
            t = tensors[i]
            if t.dtype != torch.float32 or not t.is_cuda:
                raise TypeError(f"{what} {i}: expected a float32 GPU tensor, got {t.dtype} on {t.device}")
            if t.device != self.resi.device:
                raise ValueError(f"{what} {i} is on {t.device}, the buffers are on {self.resi.device}")
        raise AssertionError("unreachable: the quick check and the detailed one disagree")

    # ---- send side

    def compress(self, grads, stream=None, sync=False):
        """Quantize every compressed parameter's gradient with error feedback.

        `grads[i]` is parameter i's gradient (any shape, fp32 on the GPU; one that is not contiguous,
        such as a channels_last gradient, goes through a contiguous copy), or None when
        the parameter has no gradient this step (its residual and code words are left as they
        are); entries of uncompressed parameters are ignored.  One launch per 96 parameters.
        """
        m, g_arr, r_arr, c_arr, n_arr, _, _staged = self._tables(grads, "gradient", stream)
        if not m:
            return
        with _q._on_device(self.resi.device):
            _lib.check(_lib.lib().nklq_quantize_multi_f32(
                m, g_arr, r_arr, c_arr, n_arr, self.thrd, 1, _nb.stream_handle(stream, self.resi.device)))
        if sync:
            _sync(self.device, stream)

    def compress_flat(self, flat_grad, stream=None, sync=False, chunk=DEFAULT_CHUNK):
        """Quantize one flat gradient buffer that holds exactly the compressed parameters back to
        back (e.g. a flattened bucket): a single launch, or one per `chunk` elements.

        The packing is then that of ONE flat vector (words do not restart at parameter
        boundaries); use it with a layout of a single entry per bucket.
        """
        idx = [i for i, c in enumerate(self.grd_cmps) if c]
        if len(idx) != 1:
            raise ValueError("compress_flat needs a layout with exactly one compressed entry (the bucket)")
        if flat_grad.numel() != self.layout.numels[idx[0]]:
            raise ValueError("flat gradient length does not match the layout")
        quantize_chunked(flat_grad.reshape(-1), self.grd_comp[idx[0]], self.grd_resi[idx[0]], self.thrd,
                         chunk=chunk, stream=stream, add_residual=True, sync=sync)

    # ---- receive side

    def decompress_sum(self, outs, average=True, stream=None, sync=False):
        """outs[i] <- sum over ranks k = 0..kn-1 (in that order) of decode(recv[k] of parameter i),
        divided by kn when `average` (the `/ kn` of necklace/frmwrk/pytorch/ptprms.py:294).
        Entries that are None are skipped, as in `compress`."""
        m, o_arr, _, _, n_arr, wo_arr, staged = self._tables(outs, "output", stream)
        if not m:
            return
        with _q._on_device(self.resi.device):
            _lib.check(_lib.lib().nklq_dequant_accumulate_multi_f32(
                m, o_arr, n_arr, wo_arr, self._pl_arr, self.kn, self.thrd, 0,
                float(self.kn) if average else 1.0, _nb.stream_handle(stream, self.resi.device)))
            for t, tmp in staged:  # a non-contiguous output: the sums were written to its temporary
                with _stream_ctx(stream):
                    t.copy_(tmp)
        if sync:
            _sync(self.device, stream)

    def state_dict(self):
        """Error-feedback state that has to survive a restart."""
        return {"resi": self.resi, "thrd": self.thrd, "numels": list(self.layout.numels),
                "size_threshold": self.layout.size_threshold}

    def load_state_dict(self, state):
        if list(state["numels"]) != self.layout.numels or state["size_threshold"] != self.layout.size_threshold:
            raise ValueError("residual state belongs to a different parameter layout")
        self.resi.copy_(state["resi"])
        self.thrd = float(state["thrd"])


def quantize_chunked(g, c, r, thrd, chunk=DEFAULT_CHUNK, stream=None, add_residual=True, sync=True):
    """Quantize a long flat vector in launches of `chunk` elements (a multiple of 16, so the
    words of consecutive chunks abut and the result equals a single launch over the whole vector)."""
    if chunk <= 0 or chunk % CMP_RATIO:
        raise ValueError("chunk must be a positive multiple of 16")
    if g.dim() != 1 or r.shape != g.shape:
        raise ValueError("g and r must be flat vectors of the same length")
    n = g.shape[0]
    if c.dim() != 1 or c.shape[0] != _q.packed_rows(n):
        raise ValueError(f"c must hold {_q.packed_rows(n)} words")
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        _q.cu_fn_matrix_quantize_e(g[lo:hi], c[lo // CMP_RATIO:_q.packed_rows(hi)], r[lo:hi], thrd,
                                   stream=stream, add_residual=add_residual, sync=False)
    if sync and n:
        _sync(g.device, stream)


# --------------------------------------------------------------------------- functional surface

def init_grads_compression(params, kn, grd_siz_thrd=DEFAULT_SIZE_THRESHOLD, device="cuda", rank=None,
                           thrd=DEFAULT_COMP_THRESHOLD):
    """Counterpart of the call at necklace/trainer/tnopmx.py:140-143.

    Returns ``(grd_resi, grd_recv, grd_comp, grd_cmps)``: per-parameter residuals,
    ``[kn, words]`` receive slots, local packed codes (views of this rank's receive slot when `rank`
    is given, of a buffer of their own otherwise), and which parameters are compressed.  The views keep the flat buffers alive; use
    `init_grad_comp_cfg` to also get the `GradCompressor` that owns them.
    """
    gc = GradCompressor(params, kn, thrd=thrd, size_threshold=grd_siz_thrd, device=device, rank=rank)
    return gc.grd_resi, gc.grd_recv, gc.grd_comp, gc.grd_cmps


def init_grad_comp_cfg(params, kn, grad_comp_cfg=None, device="cuda", rank=None):
    """Fill a ``grad_comp_cfg`` dict the way TrainerOPMxnet.init_grads_comp does
    (necklace/trainer/tnopmx.py:135-151): keys grd_resi, grd_recv, grd_comp, grd_cmps,
    grad_size_threshold, grad_comp_threshold; plus 'compressor', the object that owns the buffers.
    `rank` (or ``grad_comp_cfg['rank']``): see GradCompressor; it is recorded in the dict."""
    cfg = dict(grad_comp_cfg or {})
    if "rank" in cfg:
        if rank is not None and int(rank) != int(cfg["rank"]):
            raise ValueError(f"rank = {rank} but grad_comp_cfg['rank'] = {cfg['rank']}")
        rank = int(cfg["rank"])
    siz = cfg.get("grad_size_threshold", DEFAULT_SIZE_THRESHOLD)
    thr = cfg.get("grad_comp_threshold", DEFAULT_COMP_THRESHOLD)
    gc = GradCompressor(params, kn, thrd=thr, size_threshold=siz, device=device, rank=rank)
    cfg.update(grd_resi=gc.grd_resi, grd_recv=gc.grd_recv, grd_comp=gc.grd_comp, grd_cmps=gc.grd_cmps,
               grad_size_threshold=siz, grad_comp_threshold=thr, compressor=gc)
    if gc.rank is not None:
        cfg["rank"] = gc.rank
    return cfg


def _run_exchange(exchange, gc, kn, stream):
    """Calls the caller's all-gather of the payloads in stream order with the kernels around it.

    The kernels run on `stream` (None: torch's current stream); `exchange(comp, recv)` is called
    with torch's current stream as it is, which is where a collective issued through torch runs.
    When the two differ, the current stream first waits for the compress, and `stream` then waits
    for what the exchange put on the current stream."""
    if exchange is None:
        if kn != 1:
            raise ValueError("an exchange callable is required when kn > 1")
        return
    cur = torch.cuda.current_stream(gc.device)
    other = stream is not None and not isinstance(stream, int) and stream != cur
    if isinstance(stream, int) and stream != cur.cuda_stream:
        raise ValueError("with a raw stream handle the exchange cannot be ordered: pass a torch.cuda.Stream")
    if other:
        cur.wait_stream(stream)
    exchange(gc.comp, gc.recv)
    if other:
        stream.wait_stream(cur)


def grads_do_compressed_exchange(grads, kn, grad_comp_cfg, exchange=None, average=True, stream=None):
    """The compressed form of the gradient all-reduce (what ``grads_do_nccl(..., grad_comp_cfg=)``
    stands for at necklace/trainer/tnopmx.py:334-337): compress, exchange, decompress-sum in place.

    `exchange(comp, recv)` must fill ``recv[k]`` with rank k's payload for all k (an all-gather of
    `comp`); it is the caller's, since collectives are not part of this module.  With ``kn == 1``
    it may be omitted.  Entries of `grads` may be None (no gradient this step).  Returns the
    indices of the parameters that were NOT compressed (below the size threshold) and still need
    the ordinary fp32 all-reduce.
    """
    gc = grad_comp_cfg["compressor"]
    if gc.kn != kn:
        raise ValueError(f"grad_comp_cfg was built for kn={gc.kn}, got kn={kn}")
    gc.compress(grads, stream=stream)
    _run_exchange(exchange, gc, kn, stream)
    gc.decompress_sum(grads, average=average, stream=stream)
    return [i for i, c in enumerate(gc.grd_cmps) if not c and grads[i] is not None]


# --------------------------------------------------------------------------- flat gradient buffer

def init_flat_grad_comp_cfg(total_size, kn, grad_comp_cfg=None, device="cuda", rank=None):
    """`grad_comp_cfg` for ONE flat gradient buffer of `total_size` floats — the `grd_fltn_gpu` of
    PtCudaFltnMemManager (necklace/frmwrk/pytorch/tsmem.py:157-180), which the flat ZeRO trainer
    reduces as a whole (necklace/trainer/zroppf.py:957-965).  Residual, payload and receive slots
    are allocated once, next to it; the buffer itself is never copied."""
    cfg = dict(grad_comp_cfg or {})
    cfg["grad_size_threshold"] = 1  # a flat buffer is always compressed
    return init_grad_comp_cfg([int(total_size)], kn, cfg, device=device, rank=rank)


def _flat_view(d_arr_send, sz):
    if not d_arr_send.is_contiguous():
        raise ValueError("the flat gradient buffer must be contiguous (the result is written in place)")
    return d_arr_send.view(-1)[:sz]


def opt_grads_fltn_do_compressed_reduce(kn, d_arr_send, sz, grad_comp_cfg, exchange=None, average=False,
                                        stream=None, decode=True):
    """Compressed form of ``opt_grads_fltn_do_nccl_reduce(nc, kn, root, d_arr_send, sz, grad_comp_cfg)``
    (necklace/frmwrk/pytorch/ptprms.py:396-401): the first `sz` floats of the flat buffer
    `d_arr_send` are quantized with error feedback (one launch per 2^28 elements), `exchange(comp,
    recv)` gathers every rank's payload, and (with `decode`) the decoded sum over ranks, in rank
    order, replaces them.  The reference's reduce does not average; pass ``average=True`` for ``/ kn``."""
    gc = grad_comp_cfg["compressor"]
    if gc.kn != kn:
        raise ValueError(f"grad_comp_cfg was built for kn={gc.kn}, got kn={kn}")
    flat = _flat_view(d_arr_send, sz)
    gc.compress_flat(flat, stream=stream)
    _run_exchange(exchange, gc, kn, stream)
    if decode:
        gc.decompress_sum([flat], average=average, stream=stream)


# --------------------------------------------------------------------------- checkpoint

def grad_comp_state(grad_comp_cfg):
    """What has to go into the `state` dict handed to save_checkpoint
    (necklace/frmwrk/pytorch/callback.py:16-19) for the error feedback to survive a restart:
    the residual and the layout it belongs to.  Plain tensors and numbers only, so the file
    loads with ``torch.load(..., weights_only=True)``.

    The bucket form lays its residuals out per bucket, and the buckets depend on which parameters
    have a gradient; its state is therefore saved per PARAMETER (``param_resi``: position in the
    optimizer's parameter list -> what that parameter is still owed, including the ones set aside
    while a parameter sits a step out), which any later bucketing can take up again."""
    st = grad_comp_cfg["compressor"].state_dict()
    out = {"resi": st["resi"].detach().clone(), "thrd": float(st["thrd"]),
           "numels": [int(n) for n in st["numels"]], "size_threshold": int(st["size_threshold"])}
    places = grad_comp_cfg.get("_places")
    if grad_comp_cfg.get("_signature", ("",))[0] == "buckets" and places is not None:
        gc = grad_comp_cfg["compressor"]
        per = {int(pos): gc.grd_resi[bi][off:off + n].detach().clone() for pos, (bi, off, n) in places.items()}
        for pos, r in grad_comp_cfg.get("_parked", {}).items():
            per[int(pos)] = r.detach().clone()
        out["form"] = "buckets"
        out["param_resi"] = per
    return out


def load_grad_comp_state(grad_comp_cfg, state):
    """Restore what `grad_comp_state` saved into a `grad_comp_cfg` for the same parameters.  When the
    buffers are not laid out yet (a dict that has only been configured: the drop-ins below lay them
    out on their first call), the state is kept in the dict and applied at that first call."""
    gc = grad_comp_cfg.get("compressor")
    grad_comp_cfg["grad_comp_threshold"] = float(state["thrd"])
    if gc is None or state.get("form") == "buckets":
        grad_comp_cfg["_pending_state"] = state
        if gc is not None:
            gc.thrd = float(state["thrd"])
        return
    gc.load_state_dict(state)


def _apply_pending_state(cfg, gc, places=None):
    """Residuals loaded before the buffers existed: put them where the layout now has them."""
    state = cfg.pop("_pending_state", None)
    if state is None:
        return
    gc.thrd = float(state["thrd"])
    per = state.get("param_resi")
    if places is not None:  # bucket form: per-parameter residuals into their bucket slices
        if per is None:
            raise ValueError("the residual state was saved by the per-parameter form; it cannot be split over buckets")
        parked = cfg.setdefault("_parked", {})
        for pos, r in per.items():
            where = places.get(int(pos))
            if where is not None and where[2] == r.numel():
                bi, off, n = where
                gc.grd_resi[bi][off:off + n].copy_(r)
            else:
                parked[int(pos)] = r.to(gc.device).clone()
    elif per is not None:   # saved by the bucket form, taken up by the per-parameter form
        for pos, r in per.items():
            pos = int(pos)
            if pos < len(gc.grd_resi) and gc.grd_resi[pos] is not None and gc.grd_resi[pos].numel() == r.numel():
                gc.grd_resi[pos].copy_(r)
    else:
        gc.load_state_dict(state)


# --------------------------------------------------------------------------- ptprms call surface
#
# Same names, argument order and return value (None) as necklace/frmwrk/pytorch/ptprms.py:300-401, so
# that a trainer can import them from here instead.  What differs is what travels:
#
#   nc             where necklace passes its NCCL communicator.  Collectives are not part of this
#                  package, so `nc` is whatever moves the data: a callable ``nc(comp, recv)`` that
#                  all-gathers the packed words, or an object with ``all_gather_words(comp, recv)``
#                  and, for the gradients that stay fp32, ``all_reduce_f32(flat)`` /
#                  ``reduce_f32(flat, root)`` (sum, in place).  None is allowed for kn == 1.
#   grad_comp_cfg  the dict of necklace/trainer/tnopmx.py:135-151 (grad_size_threshold,
#                  grad_comp_threshold) plus: 'rank' (this worker), 'form' ("params": every gradient
#                  of at least grad_size_threshold elements is packed on its own, the smaller ones
#                  are flattened into one fp32 message, the default; "buckets": all gradients are
#                  flattened into buckets of at most 'bucket_bytes' = 256 MB and each bucket is packed
#                  as one vector, the shape of nccl_allreduce_by_buckets, ptprms.py:256-299),
#                  'small_allreduce' / 'small_reduce' (callables that override nc's fp32 methods).
#                  The buffers are laid out on the first call and kept in the dict.
#   prm_revs       accepted and unused, as in the reference.

NCCL_REDUCE_BUCKET_BYTES = 256 * 1024 * 1024  # nccl_reduce_bucket_size, necklace/frmwrk/pytorch/ptprms.py:253


def _opt_params(opt):
    """Every parameter an optimizer owns, in the order necklace walks them
    (necklace/frmwrk/pytorch/ptprms.py:331-336)."""
    return [p for group in opt.param_groups for p in group["params"]]


def _exchange_of(nc):
    if nc is None or (callable(nc) and not hasattr(nc, "all_gather_words")):
        return nc
    return nc.all_gather_words


def _small_fn(nc, cfg, root):
    """The fp32 collective for what is not compressed: sums `flat` over the workers in place."""
    key, meth = ("small_allreduce", "all_reduce_f32") if root is None else ("small_reduce", "reduce_f32")
    fn = cfg.get(key) or getattr(nc, meth, None)
    if fn is None:
        return None
    return fn if root is None else (lambda flat: fn(flat, root))


def _take_buckets(tensors, limit_bytes):
    """Consecutive groups of tensors of at most `limit_bytes` each (a tensor larger than that is a
    group of its own): the bucketing of ptprms.py:258 for tensors of one type (the callers have
    checked that all are float32)."""
    buckets, cur, size = [], [], 0
    for t in tensors:
        b = t.numel() * t.element_size()
        if cur and size + b > limit_bytes:
            buckets.append(cur)
            cur, size = [], 0
        cur.append(t)
        size += b
    if cur:
        buckets.append(cur)
    return buckets


def _rank_of(nc, cfg, kn):
    """This worker's index among the kn: grad_comp_cfg['rank'], else nc.rank.  With several workers it
    decides which receive slot holds the own payload and who decodes a reduce: a silent default of 0
    on every worker would give wrong sums without any error."""
    if "rank" in cfg:
        return int(cfg["rank"])
    r = getattr(nc, "rank", None)
    if r is not None and not callable(r):
        return int(r)
    if kn > 1:
        raise ValueError("grad_comp_cfg['rank'] (this worker's index, 0 .. kn-1) is required when kn > 1")
    return 0


def _decodes(gc, root):
    """Whether this worker decodes the sum: every worker of an all-reduce (root None), the root of a
    reduce.  A compressor that was set up without a rank cannot tell and says so."""
    if root is None:
        return True
    if gc.rank is None:
        raise ValueError("a reduce onto a root needs this worker's rank: set grad_comp_cfg['rank'] "
                         "(or pass rank= where the buffers are set up)")
    return gc.rank == root


def _check_fp32(grads):
    """The compressed path packs fp32 gradients.  The reference buckets per tensor type
    (_take_tensors, necklace/frmwrk/pytorch/ptprms.py:258) and all-reduces every type; here any other
    type is refused before anything is launched (such gradients belong on the uncompressed path)."""
    for i, g in enumerate(grads):
        if g is not None and g.dtype != torch.float32:
            raise TypeError(f"gradient {i} is {g.dtype}: the compressed exchange takes float32 gradients only")


def _carry_residuals(old_gc, old_ids, new_gc, new_ids):
    """Error feedback owed to a parameter survives a change of the layout: matched by parameter
    identity when the old layout knows its parameters, by position otherwise (a layout that was
    built or restored before the parameters were seen)."""
    if old_gc is None:
        return
    if old_ids:
        where = {pid: i for i, pid in enumerate(old_ids)}
        pairs = [(where.get(pid), j) for j, pid in enumerate(new_ids)]
    else:
        pairs = [(j, j) for j in range(min(len(old_gc.grd_resi), len(new_gc.grd_resi)))]
    for i, j in pairs:
        if i is not None and old_gc.grd_resi[i] is not None and new_gc.grd_resi[j] is not None \
                and old_gc.grd_resi[i].numel() == new_gc.grd_resi[j].numel():
            new_gc.grd_resi[j].copy_(old_gc.grd_resi[i])


def _cfg_for_params(params, kn, cfg, nc=None):
    """Lay the buffers out over ALL parameters of the optimizer (a parameter without a gradient is
    skipped per call); rebuilt, residuals carried over, when the optimizer's parameters change.  A
    compressor that is already in the dict and fits the parameters (from `init_grad_comp_cfg`,
    possibly with residuals restored from a checkpoint) is taken as it is."""
    ids = [id(p) for p in params]
    numels = [p.numel() for p in params]
    siz = int(cfg.get("grad_size_threshold", DEFAULT_SIZE_THRESHOLD))
    sig = ("params", tuple(numels), kn, siz)
    if cfg.get("_signature") != sig:
        old_gc, old_ids = cfg.get("compressor"), cfg.get("_ids", [])
        was_params = cfg.get("_signature", ("params",))[0] == "params"
        if old_gc is not None and "_signature" not in cfg and old_gc.kn == kn \
                and old_gc.layout.numels == numels and old_gc.layout.size_threshold == siz:
            gc = old_gc  # laid out beforehand for exactly these parameters
            known = int(cfg["rank"]) if "rank" in cfg else getattr(nc, "rank", None)
            if known is not None and not callable(known) and gc.rank is not None and int(known) != gc.rank:
                raise ValueError(f"this worker's rank is {known}, the buffers were laid out for rank {gc.rank}")
        else:
            dev = params[0].device if params else torch.device("cuda")
            built = init_grad_comp_cfg(params, kn, cfg, device=dev, rank=_rank_of(nc, cfg, kn))
            gc = built["compressor"]
            _carry_residuals(old_gc if was_params else None, old_ids, gc, ids)
            cfg.update(built)
        cfg["_signature"], cfg["_ids"] = sig, ids
    if "_pending_state" in cfg:  # residuals from a checkpoint, loaded before this layout existed
        _apply_pending_state(cfg, cfg["compressor"])
    return cfg["compressor"]


def _reduce_small(small, kn, fn, average):
    """The gradients below the size threshold, as ONE flattened fp32 message
    (flatten -> collective -> / kn -> copy back, ptprms.py:261-299)."""
    if not small:
        return
    if kn == 1:
        return  # the sum over one worker, divided by one
    if fn is None:
        raise ValueError(
            f"{len(small)} gradients are below grad_size_threshold and kn > 1: give nc an all_reduce_f32 / "
            "reduce_f32 method or put 'small_allreduce' / 'small_reduce' into grad_comp_cfg")
    flat = torch.cat([g.reshape(-1) for g in small])
    fn(flat)
    if average:
        flat /= float(kn)
    pos = 0
    for g in small:
        g.copy_(flat[pos:pos + g.numel()].view_as(g))
        pos += g.numel()


def _reduce_params_form(nc, kn, root, params, cfg):
    grads = [p.grad.data if p.grad is not None else None for p in params]
    _check_fp32(grads)
    gc = _cfg_for_params(params, kn, cfg, nc)
    if all(g is None for g in grads):
        return
    average = root is None  # the reference's reduce leaves `/ kn` commented out (ptprms.py:385)
    gc.compress(grads)
    _run_exchange(_exchange_of(nc), gc, kn, None)
    if _decodes(gc, root):
        gc.decompress_sum(grads, average=average)
    small = [g for g, c in zip(grads, gc.grd_cmps) if g is not None and not c]
    _reduce_small(small, kn, _small_fn(nc, cfg, root), average)


def _bucket_places(owners, buckets):
    """{position of the parameter: (bucket, offset, numel)} for a bucketing of the parameters' gradients."""
    places, it = {}, iter(owners)
    for bi, bucket in enumerate(buckets):
        pos = 0
        for g in bucket:
            places[next(it)] = (bi, pos, g.numel())
            pos += g.numel()
    return places


def _reduce_buckets_form(nc, kn, root, params, cfg):
    live = [(i, p) for i, p in enumerate(params) if p.grad is not None]
    grads = [p.grad.data for _, p in live]
    if not grads:
        return
    _check_fp32(grads)
    buckets = _take_buckets(grads, int(cfg.get("bucket_bytes", NCCL_REDUCE_BUCKET_BYTES)))
    sizes = [sum(g.numel() for g in b) for b in buckets]
    sig = ("buckets", tuple(tuple(g.numel() for g in b) for b in buckets), kn)
    # a parameter is known by its position in the optimizer's list: the same in every process and
    # after a restart, which an id() is not
    places = _bucket_places([i for i, _ in live], buckets)
    if cfg.get("_signature") != sig or cfg.get("_places") != places:
        old_gc, old_places = cfg.get("compressor"), cfg.get("_places")
        was_buckets = cfg.get("_signature", ("",))[0] == "buckets"
        sub = dict(cfg)
        sub["grad_size_threshold"] = 1  # a bucket is always packed
        built = init_grad_comp_cfg(sizes, kn, sub, device=grads[0].device, rank=_rank_of(nc, cfg, kn))
        if was_buckets and old_places:
            # the set of gradients changed: what a parameter is still owed moves to its new place;
            # a parameter that sits this step out has its residual set aside until it comes back
            parked = cfg.setdefault("_parked", {})
            for pos, was in old_places.items():
                if pos not in places:
                    parked[pos] = old_gc.grd_resi[was[0]][was[1]:was[1] + was[2]].clone()
            for pos, (bi, off, n) in places.items():
                was = old_places.get(pos)
                if was is not None and was[2] == n:
                    built["grd_resi"][bi][off:off + n].copy_(old_gc.grd_resi[was[0]][was[1]:was[1] + n])
                elif was is None and pos in parked and parked[pos].numel() == n:
                    built["grd_resi"][bi][off:off + n].copy_(parked.pop(pos))
        for key in ("grd_resi", "grd_recv", "grd_comp", "grd_cmps", "compressor"):
            cfg[key] = built[key]
        cfg["_signature"], cfg["_places"] = sig, places
        cfg["_flat"] = [torch.empty(n, dtype=torch.float32, device=grads[0].device) for n in sizes]
    if "_pending_state" in cfg:  # residuals from a checkpoint, loaded before this layout existed (or over it)
        _apply_pending_state(cfg, cfg["compressor"], places)
    gc, flats = cfg["compressor"], cfg["_flat"]
    for flat, bucket in zip(flats, buckets):  # grads_batch_coalesced, ptprms.py:262
        torch.cat([g.reshape(-1) for g in bucket], out=flat)
    gc.compress(flats)
    _run_exchange(_exchange_of(nc), gc, kn, None)
    if _decodes(gc, root):
        gc.decompress_sum(flats, average=root is None)
        for flat, bucket in zip(flats, buckets):  # unflatten and copy back, ptprms.py:296-299
            pos = 0
            for g in bucket:
                g.copy_(flat[pos:pos + g.numel()].view_as(g))
                pos += g.numel()


def _reduce_opt(nc, kn, root, opt, grad_comp_cfg):
    _reduce_params(nc, kn, root, _opt_params(opt), grad_comp_cfg)


def _reduce_params(nc, kn, root, params, grad_comp_cfg):
    if grad_comp_cfg is None:
        raise ValueError("grad_comp_cfg is required: this is the compressed path")
    form = grad_comp_cfg.get("form", "params")
    if form == "params":
        _reduce_params_form(nc, kn, root, params, grad_comp_cfg)
    elif form == "buckets":
        _reduce_buckets_form(nc, kn, root, params, grad_comp_cfg)
    else:
        raise ValueError(f"grad_comp_cfg['form'] must be 'params' or 'buckets', got {form!r}")


def _per_optimizer(opt, grad_comp_cfg):
    if not isinstance(opt, (list, tuple)):
        return [(opt, grad_comp_cfg)]
    if len(opt) > 1 and not isinstance(grad_comp_cfg, (list, tuple)):
        raise ValueError("several optimizers need one grad_comp_cfg each (their residuals differ)")
    cfgs = grad_comp_cfg if isinstance(grad_comp_cfg, (list, tuple)) else [grad_comp_cfg] * len(opt)
    return list(zip(opt, cfgs))


def grads_do_nccl_allreduce(nc, kn, model, prm_revs=None, grad_comp_cfg=None):
    """Compressed counterpart of ptprms.grads_do_nccl_allreduce
    (necklace/frmwrk/pytorch/ptprms.py:300-315): the same step over a model's trainable parameters
    instead of an optimizer's.  Returns None."""
    params = [p for p in model.parameters() if p.requires_grad]
    for p in params:
        if p.grad is not None and p.grad.requires_grad:
            # the reference's wording (ptprms.py:307-310)
            raise RuntimeError("DistributedDataParallel only works with gradients that don't require grad")
    _reduce_params(nc, kn, None, params, grad_comp_cfg)


def grads_do_nccl(params, prm_recvs, nc, kn, grad_comp_cfg=None):
    """The call the MXNet trainer makes, ``mxprms.grads_do_nccl(net.collect_params(), prm_recvs,
    nc, kn, grad_comp_cfg=...)`` (necklace/trainer/tnopmx.py:334-337), with its argument order:
    `params` is a sequence of parameters or a dict of them (the values are taken, in order), each
    with a ``.grad``; `prm_recvs` (the fp32 receive buffers of the uncompressed path) is not needed
    here.  Every gradient ends as the average over the `kn` workers.  Returns None."""
    plist = list(params.values()) if hasattr(params, "values") else list(params)
    _reduce_params(nc, kn, None, plist, grad_comp_cfg)


def opt_one_grads_do_nccl_allreduce(nc, kn, opt, prm_revs=None, grad_comp_cfg=None):
    """Compressed counterpart of ptprms.opt_one_grads_do_nccl_allreduce
    (necklace/frmwrk/pytorch/ptprms.py:329-338): afterwards EVERY gradient of the optimizer holds
    the average over the `kn` workers — of its 2-bit decode where it was packed, of its fp32 values
    where it was too small to pack.  Returns None, like the reference."""
    _reduce_opt(nc, kn, None, opt, grad_comp_cfg)


def opt_grads_do_nccl_allreduce(nc, kn, opt, prm_revs=None, grad_comp_cfg=None):
    """ptprms.opt_grads_do_nccl_allreduce (ptprms.py:319-326): one optimizer or a list of them, each
    with its own ``grad_comp_cfg`` when a list of configs is given."""
    for o, c in _per_optimizer(opt, grad_comp_cfg):
        opt_one_grads_do_nccl_allreduce(nc, kn, o, prm_revs=prm_revs, grad_comp_cfg=c)


def opt_one_grads_do_nccl_reduce(nc, kn, root, opt, prm_revs=None, grad_comp_cfg=None):
    """Compressed counterpart of ptprms.opt_one_grads_do_nccl_reduce (ptprms.py:354-363): like the
    all-reduce but only worker `root` ends up with the sums, and they are not averaged (the
    reference's reduce leaves the `/ kn` commented out, ptprms.py:385).  Returns None."""
    _reduce_opt(nc, kn, root, opt, grad_comp_cfg)


def opt_grads_do_nccl_reduce(nc, kn, root, opt, prm_revs=None, grad_comp_cfg=None):
    """ptprms.opt_grads_do_nccl_reduce (ptprms.py:344-351)."""
    for o, c in _per_optimizer(opt, grad_comp_cfg):
        opt_one_grads_do_nccl_reduce(nc, kn, root, o, prm_revs=prm_revs, grad_comp_cfg=c)


def opt_grads_fltn_do_nccl_reduce(nc, kn, root, d_arr_send, sz, grad_comp_cfg=None):
    """Compressed counterpart of ptprms.opt_grads_fltn_do_nccl_reduce (ptprms.py:396-401) on the
    flat gradient buffer; see `opt_grads_fltn_do_compressed_reduce`.  Only `root` decodes.  The
    buffers are laid out on the first call (or by `init_flat_grad_comp_cfg` beforehand) and kept in
    `grad_comp_cfg`."""
    if grad_comp_cfg is None:
        raise ValueError("grad_comp_cfg is required: this is the compressed path")
    gc = grad_comp_cfg.get("compressor")
    if gc is None or gc.kn != kn or list(gc.layout.numels) != [int(sz)]:
        # first call (or another buffer length): lay the buffers out next to the flat gradient;
        # a residual from before belongs to another layout and does not carry over
        grad_comp_cfg.update(init_flat_grad_comp_cfg(sz, kn, grad_comp_cfg, device=d_arr_send.device,
                                                     rank=_rank_of(nc, grad_comp_cfg, kn)))
        gc = grad_comp_cfg["compressor"]
        _apply_pending_state(grad_comp_cfg, gc)
    opt_grads_fltn_do_compressed_reduce(kn, d_arr_send, sz, grad_comp_cfg, exchange=_exchange_of(nc),
                                        average=False, decode=_decodes(gc, root))
