"""Trainer-side compression buffers on the GPU: per-parameter compress with error feedback,
synthetic peers, fixed-order decompress-sum, chunked driver — all against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal, assert_words_equal
from gpu_util import dev, host_words, random_payloads_gpu, resnet50_segment_sizes
from necklace_amd.frmwrk.pytorch import ptcomp

pytestmark = pytest.mark.gpu


def test_per_parameter_compress_exchange_decompress_three_steps():
    """A ResNet-50-shaped set of 161 gradients, kn = 4 (this rank is 1, three synthetic peers),
    grad_size_threshold 1001: small tensors are skipped, the others go through
    compress -> exchange -> decompress-sum, three steps with the residual carried."""
    sizes = resnet50_segment_sizes()
    kn, rank, thrd = 4, 1, 1e-3
    cfg = ptcomp.init_grad_comp_cfg(sizes, kn, {"grad_comp_threshold": thrd}, rank=rank)
    gc = cfg["compressor"]
    lay = gc.layout
    assert sum(cfg["grd_cmps"]) == sum(1 for s in sizes if s >= 1001)
    resid_host = [np.zeros(s, np.float32) for s in sizes]
    rng = np.random.default_rng(8)
    sig = 10.0 ** rng.uniform(-4, -2, len(sizes))
    for step in range(3):
        grads_host = [(rng.standard_normal(s, dtype=np.float32) * np.float32(sig[i])) for i, s in enumerate(sizes)]
        grads = [dev(g) for g in grads_host]
        peers = random_payloads_gpu(kn, 16 * lay.total_words, 900 + step)  # [kn, total_words]

        def exchange(comp, recv, peers=peers):
            mine = comp.clone()
            recv.copy_(peers)
            recv[rank].copy_(mine)

        left = ptcomp.grads_do_compressed_exchange(grads, kn, cfg, exchange=exchange, average=True)
        assert left == [i for i, s in enumerate(sizes) if s < 1001]
        torch.cuda.synchronize()
        peers_host = host_words(peers)
        for i, s in enumerate(sizes):
            if s < 1001:
                assert_bits_equal(grads[i].cpu().numpy(), grads_host[i], f"uncompressed {i} must be untouched")
                continue
            want_c, want_r = oracle.c.quantize(grads_host[i], thrd, R_in=resid_host[i])
            resid_host[i] = want_r
            wo, w = lay.word_offset[i], lay.words[i]
            assert_words_equal(host_words(gc.grd_comp[i]), want_c, f"step {step} param {i} codes")
            assert_bits_equal(gc.grd_resi[i].cpu().numpy(), want_r, f"step {step} param {i} residual")
            pl = [peers_host[k, wo:wo + w].copy() for k in range(kn)]
            pl[rank] = want_c
            want = (oracle.c.dequant_accumulate(pl, s, thrd) / np.float32(kn)).astype(np.float32)
            assert_bits_equal(grads[i].cpu().numpy(), want, f"step {step} param {i} sum")


def test_bucket_compress_flat_and_chunked_driver():
    n, thrd = 3_000_000 + 7, 5e-3
    rng = np.random.default_rng(17)
    g = rng.normal(0, 5e-3, n).astype(np.float32)
    gc = ptcomp.GradCompressor([n], kn=1, thrd=thrd)
    r0 = rng.normal(0, 1e-3, n).astype(np.float32)
    gc.grd_resi[0].copy_(dev(r0))
    want_c, want_r = oracle.c.quantize(g, thrd, R_in=r0)
    gc.compress_flat(dev(g), chunk=1 << 20, sync=True)  # three chunks, the last one ragged
    assert_words_equal(host_words(gc.grd_comp[0]), want_c)
    assert_bits_equal(gc.grd_resi[0].cpu().numpy(), want_r)
    out = torch.empty(n, device="cuda")
    gc.decompress_sum([out], sync=True)
    assert_bits_equal(out.cpu().numpy(), oracle.c.dequant_accumulate([want_c], n, thrd))
    # chunked driver on its own buffers equals one launch
    c1 = torch.full(((n + 15) // 16,), -1, dtype=torch.int32, device="cuda")
    r1 = dev(r0)
    ptcomp.quantize_chunked(dev(g), c1, r1, thrd, chunk=4096)
    assert_words_equal(host_words(c1), want_c)
    assert_bits_equal(r1.cpu().numpy(), want_r)


def test_residual_state_survives_a_restart():
    n, thrd = 50_000, 1e-3
    rng = np.random.default_rng(23)
    gs = [rng.normal(0, 1e-3, n).astype(np.float32) for _ in range(4)]
    a = ptcomp.GradCompressor([n], kn=1, thrd=thrd)
    for g in gs[:2]:
        a.compress([dev(g)])
    state = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in a.state_dict().items()}
    b = ptcomp.GradCompressor([n], kn=1, thrd=thrd)
    b.load_state_dict(state)
    for g in gs[2:]:
        a.compress([dev(g)])
        b.compress([dev(g)], sync=True)
    torch.cuda.synchronize()
    assert torch.equal(a.resi.view(torch.int32), b.resi.view(torch.int32))
    assert torch.equal(a.comp, b.comp)


def test_flat_zero_style_buffer_reduce_in_place():
    """One flat gradient buffer (the grd_fltn_gpu of the flat ZeRO trainer): compress in place,
    two synthetic peers, decoded sum written back over the gradient; nothing is copied."""
    total, kn, rank, thrd = 1_500_000 + 9, 3, 2, 2e-3
    cfg = ptcomp.init_flat_grad_comp_cfg(total, kn, {"grad_comp_threshold": thrd}, rank=rank)
    gc = cfg["compressor"]
    rng = np.random.default_rng(31)
    resid = np.zeros(total, np.float32)
    for step in range(2):
        g = rng.normal(0, 2e-3, total).astype(np.float32)
        buf = dev(g)
        peers = random_payloads_gpu(kn, 16 * gc.layout.total_words, 40 + step)

        def exchange(comp, recv, peers=peers):
            mine = comp.clone()
            recv.copy_(peers)
            recv[rank].copy_(mine)

        ptr = buf.data_ptr()
        ptcomp.opt_grads_fltn_do_compressed_reduce(kn, buf, total, cfg, exchange=exchange)
        torch.cuda.synchronize()
        assert buf.data_ptr() == ptr
        want_c, resid = oracle.c.quantize(g, thrd, R_in=resid)
        ph = host_words(peers)
        w = gc.layout.words[0]
        pl = [ph[k, :w].copy() for k in range(kn)]
        pl[rank] = want_c
        assert_words_equal(host_words(gc.grd_comp[0]), want_c, f"step {step}")
        assert_bits_equal(gc.grd_resi[0].cpu().numpy(), resid, f"step {step}")
        assert_bits_equal(buf.cpu().numpy(), oracle.c.dequant_accumulate(pl, total, thrd), f"step {step}")


def test_flat_buffer_drop_in_under_the_reference_name():
    """ptprms.opt_grads_fltn_do_nccl_reduce(nc, kn, root, d_arr_send, sz, grad_comp_cfg=...)
    (necklace/frmwrk/pytorch/ptprms.py:396-401) with nothing but the trainer's own dict: the
    buffers are laid out on the first call; the root ends with the decoded sum (not averaged, as
    the reference's reduce), the other worker keeps its gradient; two steps of error feedback."""
    n, kn, thrd = 300_000 + 7, 2, 1e-3
    rng = np.random.default_rng(8)
    for rank, root in ((0, 0), (1, 0)):
        cfg = {"grad_comp_threshold": thrd, "rank": rank}
        nc = TwoWorkersWithEqualData(rank=rank)
        resid = np.zeros(n, np.float32)
        for step in range(2):
            g = rng.normal(0, 1e-3, n + 5).astype(np.float32)
            buf = dev(g)                                   # the flat buffer is longer than what is sent
            assert ptcomp.opt_grads_fltn_do_nccl_reduce(nc, kn, root, buf, n, grad_comp_cfg=cfg) is None
            torch.cuda.synchronize()
            c, resid = oracle.c.quantize(g[:n], thrd, R_in=resid)
            assert_bits_equal(cfg["compressor"].grd_resi[0].cpu().numpy(), resid, f"rank {rank} step {step}")
            got = buf.cpu().numpy()
            assert_bits_equal(got[n:], g[n:], "past sz")
            if rank == root:
                assert_bits_equal(got[:n], oracle.c.dequant_accumulate([c, c], n, thrd), f"root, step {step}")
            else:
                assert_bits_equal(got[:n], g[:n], f"not the root, step {step}")
    with pytest.raises(ValueError):
        ptcomp.opt_grads_fltn_do_nccl_reduce(None, 1, 0, dev(np.zeros(64, np.float32)), 64, grad_comp_cfg=None)


def test_checkpoint_file_round_trip(tmp_path):
    n, thrd = 20_000, 1e-3
    cfg = ptcomp.init_flat_grad_comp_cfg(n, 1, {"grad_comp_threshold": thrd})
    g = dev(np.random.default_rng(2).normal(0, 1e-3, n).astype(np.float32))
    cfg["compressor"].compress_flat(g, sync=True)
    path = tmp_path / "checkpoint.pth.tar"
    torch.save({"epoch": 3, "grad_comp": ptcomp.grad_comp_state(cfg)}, path)
    state = torch.load(path, weights_only=True)
    cfg2 = ptcomp.init_flat_grad_comp_cfg(n, 1, {"grad_comp_threshold": 0.5})
    ptcomp.load_grad_comp_state(cfg2, state["grad_comp"])
    assert cfg2["compressor"].thrd == thrd
    assert torch.equal(cfg2["compressor"].resi.view(torch.int32), cfg["compressor"].resi.view(torch.int32))
    assert state["epoch"] == 3


class TwoWorkersWithEqualData:
    """Stands where necklace passes its NCCL communicator: a second worker that holds exactly what
    this one holds (so every sum is x + x), with the three collectives the compressed path needs."""
    def __init__(self, rank=0):
        self.calls, self.rank = [], rank

    def all_gather_words(self, comp, recv):
        self.calls.append(("gather", comp.numel()))
        recv[1 - self.rank].copy_(recv[self.rank])

    def all_reduce_f32(self, flat):
        self.calls.append(("allreduce", flat.numel()))
        flat.mul_(2.0)

    def reduce_f32(self, flat, root):
        self.calls.append(("reduce", flat.numel(), root))
        flat.mul_(2.0)


def _mlp_with_grads(seed=0):
    torch.manual_seed(seed)
    model = torch.nn.Sequential(torch.nn.Linear(784, 256), torch.nn.ReLU(), torch.nn.Linear(256, 64),
                                torch.nn.ReLU(), torch.nn.Linear(64, 10)).cuda()
    opt = torch.optim.SGD(model.parameters(), lr=0.1)
    x = torch.randn(32, 784, device="cuda")
    y = torch.randint(0, 10, (32,), device="cuda")
    torch.nn.functional.cross_entropy(model(x), y).backward()
    return model, opt, x, y


def test_ptprms_call_surface_on_a_real_optimizer():
    """opt_grads_do_nccl_allreduce / _reduce with necklace's argument order on the gradients of a
    small MLP (the shape of the reference's MNIST example).  Like the reference functions
    (necklace/frmwrk/pytorch/ptprms.py:319-363) they return None and leave EVERY gradient reduced:
    the large ones through the 2-bit codes, the small ones as one flattened fp32 message."""
    model, opt, x, y = _mlp_with_grads()
    thrd, kn = 1e-3, 2
    before = [p.grad.detach().cpu().numpy().copy() for p in model.parameters()]
    nc = TwoWorkersWithEqualData()
    cfg = {"grad_comp_threshold": thrd, "grad_size_threshold": 1001}
    assert ptcomp.opt_grads_do_nccl_allreduce(nc, kn, opt, None, grad_comp_cfg=cfg) is None
    torch.cuda.synchronize()
    assert "compressor" in cfg
    n_small = sum(g.size for g in before if g.size < 1001)
    assert ("allreduce", n_small) in nc.calls and nc.calls[0][0] == "gather"
    for p, g in zip(model.parameters(), before):
        got = p.grad.detach().cpu().numpy()
        if g.size < 1001:
            want = ((g + g) / np.float32(kn)).astype(np.float32)  # fp32 sum of two equal workers, averaged
            assert_bits_equal(got, want, "small gradients are averaged in fp32")
            continue
        c, _ = oracle.c.quantize(g.reshape(-1), thrd, R_in=np.zeros(g.size, np.float32))
        want = (oracle.c.dequant_accumulate([c, c], g.size, thrd) / np.float32(kn)).astype(np.float32)
        assert_bits_equal(got.reshape(-1), want, f"gradient of {g.shape}")
    # without a way to reduce the small gradients the call refuses instead of skipping them
    with pytest.raises(ValueError):
        ptcomp.opt_grads_do_nccl_allreduce(lambda comp, recv: None, kn, opt, None,
                                           grad_comp_cfg={"grad_comp_threshold": thrd})
    # reduce-to-root: the non-root worker compresses and sends but keeps its large gradients
    cfg1 = {"grad_comp_threshold": thrd, "rank": 1}
    opt.zero_grad(set_to_none=False)
    torch.nn.functional.cross_entropy(model(x), y).backward()
    keep = [p.grad.detach().clone() for p in model.parameters()]
    nc1 = TwoWorkersWithEqualData(rank=1)
    assert ptcomp.opt_grads_do_nccl_reduce(nc1, kn, 0, opt, None, grad_comp_cfg=cfg1) is None
    torch.cuda.synchronize()
    for p, k in zip(model.parameters(), keep):
        if p.numel() >= 1001:
            assert torch.equal(p.grad, k)
        else:
            assert torch.equal(p.grad, k * 2.0)  # summed by nc.reduce_f32, not averaged (ptprms.py:385)
    assert ("reduce", n_small, 0) in nc1.calls
    assert int((cfg1["compressor"].comp != 0).sum()) > 0


def test_model_form_gives_what_the_optimizer_form_gives():
    """grads_do_nccl_allreduce(nc, kn, model, ...) (necklace/frmwrk/pytorch/ptprms.py:300-315) walks
    model.parameters() instead of an optimizer's groups; frozen parameters are left out."""
    thrd, kn = 1e-3, 2
    cfg_a = {"grad_comp_threshold": thrd, "grad_size_threshold": 1001}
    cfg_b = dict(cfg_a)
    model_a, opt_a, _, _ = _mlp_with_grads(seed=5)
    model_b, _, _, _ = _mlp_with_grads(seed=5)
    ptcomp.opt_grads_do_nccl_allreduce(TwoWorkersWithEqualData(), kn, opt_a, None, grad_comp_cfg=cfg_a)
    assert ptcomp.grads_do_nccl_allreduce(TwoWorkersWithEqualData(), kn, model_b, None, grad_comp_cfg=cfg_b) is None
    torch.cuda.synchronize()
    for pa, pb in zip(model_a.parameters(), model_b.parameters()):
        assert torch.equal(pa.grad, pb.grad)
    # the MXNet trainer's call shape: a dict of parameters, the receive buffers, nc, kn
    model_d, _, _, _ = _mlp_with_grads(seed=5)
    assert ptcomp.grads_do_nccl(dict(model_d.named_parameters()), None, TwoWorkersWithEqualData(), kn,
                                grad_comp_cfg={"grad_comp_threshold": thrd, "grad_size_threshold": 1001}) is None
    torch.cuda.synchronize()
    for pa, pd in zip(model_a.parameters(), model_d.parameters()):
        assert torch.equal(pa.grad, pd.grad)
    # a frozen parameter is not part of the layout, its stale gradient is left alone
    model_c, _, _, _ = _mlp_with_grads(seed=5)
    first = next(model_c.parameters())
    first.requires_grad_(False)
    stale = first.grad.clone()
    cfg_c = {"grad_comp_threshold": thrd, "grad_size_threshold": 1001}
    ptcomp.grads_do_nccl_allreduce(TwoWorkersWithEqualData(), kn, model_c, None, grad_comp_cfg=cfg_c)
    torch.cuda.synchronize()
    assert torch.equal(first.grad, stale)
    assert len(cfg_c["compressor"].layout) == len(list(model_c.parameters())) - 1
    for pa, pc in list(zip(model_a.parameters(), model_c.parameters()))[1:]:
        assert torch.equal(pa.grad, pc.grad)


def test_a_gradient_that_first_appears_at_step_two_and_a_parameter_added_later():
    """The layout covers all parameters of the optimizer from the start, so one whose .grad is None
    at step 1 simply joins at step 2 with a zero residual; a parameter group added later rebuilds
    the layout and carries the residuals over."""
    torch.manual_seed(3)
    thrd = 1e-3
    a = torch.nn.Parameter(torch.randn(3000, device="cuda") * 1e-3)
    b = torch.nn.Parameter(torch.randn(5000, device="cuda") * 1e-3)
    opt = torch.optim.SGD([a, b], lr=0.1)
    cfg = {"grad_comp_threshold": thrd, "grad_size_threshold": 1}
    rng = np.random.default_rng(12)
    ra, rb = np.zeros(3000, np.float32), np.zeros(5000, np.float32)

    def step(ga, gb, gc_=None):
        a.grad = None if ga is None else dev(ga)
        b.grad = None if gb is None else dev(gb)
        ptcomp.opt_grads_do_nccl_allreduce(None, 1, opt, None, grad_comp_cfg=cfg)
        torch.cuda.synchronize()

    g1 = rng.normal(0, 2e-3, 3000).astype(np.float32)
    step(g1, None)                                   # step 1: b has no gradient yet
    c, ra = oracle.c.quantize(g1, thrd, R_in=ra)
    assert_bits_equal(a.grad.cpu().numpy(), oracle.c.dequantize(c, 3000, thrd), "step 1 a")
    g2a, g2b = rng.normal(0, 2e-3, 3000).astype(np.float32), rng.normal(0, 2e-3, 5000).astype(np.float32)
    step(g2a, g2b)                                   # step 2: b joins
    c, ra = oracle.c.quantize(g2a, thrd, R_in=ra)
    assert_bits_equal(a.grad.cpu().numpy(), oracle.c.dequantize(c, 3000, thrd), "step 2 a")
    c, rb = oracle.c.quantize(g2b, thrd, R_in=rb)
    assert_bits_equal(b.grad.cpu().numpy(), oracle.c.dequantize(c, 5000, thrd), "step 2 b")
    # step 3: a third parameter enters the optimizer; a and b keep what they are owed
    d = torch.nn.Parameter(torch.zeros(2000, device="cuda"))
    opt.add_param_group({"params": [d]})
    g3a, g3b, g3d = (rng.normal(0, 2e-3, k).astype(np.float32) for k in (3000, 5000, 2000))
    d.grad = dev(g3d)
    step(g3a, g3b)
    c, ra = oracle.c.quantize(g3a, thrd, R_in=ra)
    assert_bits_equal(a.grad.cpu().numpy(), oracle.c.dequantize(c, 3000, thrd), "step 3 a")
    c, rb = oracle.c.quantize(g3b, thrd, R_in=rb)
    assert_bits_equal(b.grad.cpu().numpy(), oracle.c.dequantize(c, 5000, thrd), "step 3 b")
    c, _ = oracle.c.quantize(g3d, thrd, R_in=np.zeros(2000, np.float32))
    assert_bits_equal(d.grad.cpu().numpy(), oracle.c.dequantize(c, 2000, thrd), "step 3 d")


def test_bucket_form_packs_flattened_buckets_like_nccl_allreduce_by_buckets():
    """grad_comp_cfg['form'] = 'buckets': gradients are flattened into buckets (here of at most
    512 KB so that the MLP gives several), every bucket is packed as ONE flat vector, exchanged,
    decoded, averaged and copied back (necklace/frmwrk/pytorch/ptprms.py:256-299); two steps with
    the residual carried per bucket."""
    model, opt, x, y = _mlp_with_grads(seed=5)
    thrd, kn = 1e-3, 2
    cfg = {"grad_comp_threshold": thrd, "form": "buckets", "bucket_bytes": 1 << 19}
    nc = TwoWorkersWithEqualData()
    resid = None
    for step in range(2):
        if step:
            opt.zero_grad(set_to_none=False)
            torch.nn.functional.cross_entropy(model(x), y).backward()
        grads = [p.grad.detach().cpu().numpy().reshape(-1).copy() for p in model.parameters()]
        assert ptcomp.opt_grads_do_nccl_allreduce(nc, kn, opt, None, grad_comp_cfg=cfg) is None
        torch.cuda.synchronize()
        # the same bucketing on the host: consecutive tensors, at most 512 KB per bucket
        buckets, cur, size = [], [], 0
        for g in grads:
            if cur and size + 4 * g.size > (1 << 19):
                buckets.append(cur)
                cur, size = [], 0
            cur.append(g)
            size += 4 * g.size
        buckets.append(cur)
        assert len(buckets) >= 2
        if resid is None:
            resid = [np.zeros(sum(g.size for g in b), np.float32) for b in buckets]
        got = [p.grad.detach().cpu().numpy().reshape(-1) for p in model.parameters()]
        k = 0
        for bi, b in enumerate(buckets):
            flat = np.concatenate(b)
            c, resid[bi] = oracle.c.quantize(flat, thrd, R_in=resid[bi])
            want = (oracle.c.dequant_accumulate([c, c], flat.size, thrd) / np.float32(kn)).astype(np.float32)
            pos = 0
            for g in b:
                assert_bits_equal(got[k], want[pos:pos + g.size], f"step {step} bucket {bi} tensor {k}")
                pos += g.size
                k += 1
    assert all(c[0] == "gather" for c in nc.calls)  # nothing stays fp32 in this form


def test_bucket_form_keeps_what_is_owed_when_the_set_of_gradients_changes():
    """Bucket form, three steps; at step 2 one parameter has no gradient, at step 3 it is back: the
    buckets are laid out anew both times and every parameter's residual moves to its new place
    (the one that sat out keeps what it was owed at step 1... which a fresh layout would drop)."""
    model, opt, x, y = _mlp_with_grads(seed=9)
    params = list(model.parameters())
    thrd, kn, limit = 1e-3, 2, 1 << 19
    cfg = {"grad_comp_threshold": thrd, "form": "buckets", "bucket_bytes": limit}
    nc = TwoWorkersWithEqualData()
    owed = {i: np.zeros(p.numel(), np.float32) for i, p in enumerate(params)}
    absent = 2  # the second layer's weight
    for step in range(3):
        if step:
            opt.zero_grad(set_to_none=False)
            torch.nn.functional.cross_entropy(model(x), y).backward()
        if step == 1:
            params[absent].grad = None
        live = [i for i, p in enumerate(params) if p.grad is not None]
        grads = {i: params[i].grad.detach().cpu().numpy().reshape(-1).copy() for i in live}
        ptcomp.opt_grads_do_nccl_allreduce(nc, kn, opt, None, grad_comp_cfg=cfg)
        torch.cuda.synchronize()
        buckets, cur, size = [], [], 0
        for i in live:
            if cur and size + 4 * grads[i].size > limit:
                buckets.append(cur)
                cur, size = [], 0
            cur.append(i)
            size += 4 * grads[i].size
        buckets.append(cur)
        for b in buckets:
            flat = np.concatenate([grads[i] for i in b])
            c, r = oracle.c.quantize(flat, thrd, R_in=np.concatenate([owed[i] for i in b]))
            want = (oracle.c.dequant_accumulate([c, c], flat.size, thrd) / np.float32(kn)).astype(np.float32)
            pos = 0
            for i in b:
                n = grads[i].size
                owed[i] = r[pos:pos + n].copy()
                assert_bits_equal(params[i].grad.detach().cpu().numpy().reshape(-1), want[pos:pos + n],
                                  f"step {step} parameter {i}")
                pos += n
    assert float(np.abs(owed[absent]).sum()) > 0


def test_sgd_with_compressed_gradients_still_learns():
    """End to end on one worker: every step's gradients go through compress -> decompress (2 bits
    per element plus error feedback) before the optimizer sees them, and the model still fits."""
    torch.manual_seed(1)
    x = torch.randn(512, 64, device="cuda")
    w_true = torch.randn(64, 10, device="cuda")
    y = (x @ w_true).argmax(1)
    model = torch.nn.Sequential(torch.nn.Linear(64, 128), torch.nn.ReLU(), torch.nn.Linear(128, 10)).cuda()
    opt = torch.optim.SGD(model.parameters(), lr=0.2)
    cfg = {"grad_comp_threshold": 2e-3, "grad_size_threshold": 1}
    losses = []
    for step in range(150):
        opt.zero_grad(set_to_none=False)
        loss = torch.nn.functional.cross_entropy(model(x), y)
        loss.backward()
        ptcomp.opt_grads_do_nccl_allreduce(None, 1, opt, None, grad_comp_cfg=cfg)
        opt.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < 0.5 * losses[0], (losses[0], losses[-1])
    assert bool(torch.isfinite(cfg["compressor"].resi).all())


def test_checkpoint_round_trip_through_the_drop_in_surface(tmp_path):
    """Residual checkpointing as a trainer would use it (necklace/frmwrk/pytorch/callback.py:16-19):
    step 1, save, "restart" (new model objects, a new grad_comp_cfg, load), step 2 through
    opt_grads_do_nccl_allreduce must give exactly what two uninterrupted steps give — in both forms.
    The layout step of the first call after the restart must not replace the restored residuals."""
    for form in ("params", "buckets"):
        thrd, kn = 1e-3, 2
        base = {"grad_comp_threshold": thrd, "form": form, "bucket_bytes": 1 << 19}
        # uninterrupted: two steps with one dict
        model, opt, x, y = _mlp_with_grads(seed=11)
        g1 = [p.grad.detach().clone() for p in model.parameters()]
        cfg = dict(base)
        ptcomp.opt_grads_do_nccl_allreduce(TwoWorkersWithEqualData(), kn, opt, None, grad_comp_cfg=cfg)
        path = tmp_path / f"ckpt_{form}.pth.tar"
        torch.save({"grad_comp": ptcomp.grad_comp_state(cfg)}, path)
        g2 = [torch.randn_like(g) * 1e-3 for g in g1]   # the second step's gradients
        for p, g in zip(model.parameters(), g2):
            p.grad = g.clone()
        ptcomp.opt_grads_do_nccl_allreduce(TwoWorkersWithEqualData(), kn, opt, None, grad_comp_cfg=cfg)
        want = [p.grad.detach().clone() for p in model.parameters()]
        # restart: other parameter objects, a dict that has only been configured, the state loaded into it
        model2, opt2, _, _ = _mlp_with_grads(seed=11)
        cfg2 = dict(base)
        ptcomp.load_grad_comp_state(cfg2, torch.load(path, weights_only=True)["grad_comp"])
        for p, g in zip(model2.parameters(), g2):
            p.grad = g.clone()
        ptcomp.opt_grads_do_nccl_allreduce(TwoWorkersWithEqualData(), kn, opt2, None, grad_comp_cfg=cfg2)
        torch.cuda.synchronize()
        for i, (p, w) in enumerate(zip(model2.parameters(), want)):
            assert_bits_equal(p.grad.cpu().numpy(), w.cpu().numpy(), f"form {form}: parameter {i} after the restart")
        assert torch.equal(cfg2["compressor"].resi.view(torch.int32), cfg["compressor"].resi.view(torch.int32)), form
        assert float(cfg["compressor"].resi.abs().sum()) > 0
        # without the state the second step differs (the test would pass trivially otherwise)
        model3, opt3, _, _ = _mlp_with_grads(seed=11)
        for p, g in zip(model3.parameters(), g2):
            p.grad = g.clone()
        ptcomp.opt_grads_do_nccl_allreduce(TwoWorkersWithEqualData(), kn, opt3, None, grad_comp_cfg=dict(base))
        assert any(not torch.equal(p.grad, w) for p, w in zip(model3.parameters(), want))


def test_a_gradient_that_is_not_contiguous_goes_through_a_copy():
    """A channels_last gradient (what _flatten_dense_tensors accepts at ptprms.py:262) in the
    per-parameter form: compressed from, and decoded into, a contiguous copy; the residual is laid
    out in the gradient's logical (row-major) order."""
    thrd, kn = 1e-3, 2
    rng = np.random.default_rng(31)
    w = torch.nn.Parameter(torch.zeros(16, 8, 5, 5, device="cuda"))
    b = torch.nn.Parameter(torch.zeros(2000, device="cuda"))
    gw = rng.normal(0, 1e-3, (16, 8, 5, 5)).astype(np.float32)
    gb = rng.normal(0, 1e-3, 2000).astype(np.float32)
    w.grad = dev(gw).contiguous(memory_format=torch.channels_last)
    b.grad = dev(gb)
    assert not w.grad.is_contiguous()
    opt = torch.optim.SGD([w, b], lr=0.1)
    cfg = {"grad_comp_threshold": thrd}
    resid = [np.zeros(3200, np.float32), np.zeros(2000, np.float32)]
    for step in range(2):   # twice: the tables are rebuilt every call while a temporary is involved
        ptcomp.opt_grads_do_nccl_allreduce(TwoWorkersWithEqualData(), kn, opt, None, grad_comp_cfg=cfg)
        torch.cuda.synchronize()
        assert not w.grad.is_contiguous()
        for i, (p, g) in enumerate(((w, gw), (b, gb))):
            c, resid[i] = oracle.c.quantize(g.reshape(-1), thrd, R_in=resid[i])
            want = (oracle.c.dequant_accumulate([c, c], g.size, thrd) / np.float32(kn)).astype(np.float32)
            assert_bits_equal(p.grad.cpu().numpy().reshape(-1), want, f"step {step} parameter {i}")
            assert_bits_equal(cfg["compressor"].grd_resi[i].cpu().numpy(), resid[i], f"step {step} residual {i}")
        w.grad = dev(gw).contiguous(memory_format=torch.channels_last)
        b.grad = dev(gb)


def test_steady_state_calls_reuse_the_argument_tables():
    """Gradients that keep their storage: the second call finds its tables by the gradients'
    addresses; a gradient that moved is noticed and gives the right result."""
    thrd = 1e-3
    sizes = [3000, 10, 5000, 70000]
    gc = ptcomp.GradCompressor(sizes, 1, thrd=thrd)
    rng = np.random.default_rng(41)
    hosts = [rng.normal(0, 1e-3, n).astype(np.float32) for n in sizes]
    grads = [dev(h) for h in hosts]
    gc.compress(grads, sync=True)
    tabs = gc._addr_cache["gradient"][1]
    for g, h in zip(grads, hosts):
        g.copy_(torch.from_numpy(h))
    gc.compress(grads, sync=True)
    assert gc._addr_cache["gradient"][1] is tabs
    resid = [None] * len(sizes)
    for i, n in enumerate(sizes):
        if gc.grd_cmps[i]:
            _, r1 = oracle.c.quantize(hosts[i], thrd, R_in=np.zeros(n, np.float32))
            c2, resid[i] = oracle.c.quantize(hosts[i], thrd, R_in=r1)
            assert_words_equal(host_words(gc.grd_comp[i]), c2, f"parameter {i}")
    moved = dev(hosts[2] * np.float32(2.0))     # parameter 2's gradient now lives elsewhere
    grads[2] = moved
    gc.compress(grads, sync=True)
    assert gc._addr_cache["gradient"][1] is not tabs
    c3, _ = oracle.c.quantize(hosts[2] * np.float32(2.0), thrd, R_in=resid[2])
    assert_words_equal(host_words(gc.grd_comp[2]), c3, "the moved gradient")
