"""Layout arithmetic and argument checking of the trainer-side compression buffers (no GPU)."""
import pytest
import torch

from necklace_amd.frmwrk.pytorch import ptcomp


def test_layout_thresholds_offsets_and_alignment():
    numels = [9408, 64, 1000, 1001, 16, 4097, 0]
    lay = ptcomp.GradCompLayout(numels, size_threshold=1001)
    # necklace/trainer/tnopmx.py:137: parameters below grad_size_threshold are not compressed
    assert lay.compressed == [True, False, False, True, False, True, False]
    assert lay.words == [588, 0, 0, 63, 0, 257, 0]
    assert lay.elem_offset == [0, None, None, 9472, None, 9472 + 1024, None]
    assert lay.word_offset == [0, None, None, 592, None, 592 + 64, None]
    assert all(o % 256 == 0 for o in lay.elem_offset if o is not None)
    assert all(o % 16 == 0 for o in lay.word_offset if o is not None)
    assert lay.total_elems == 9472 + 1024 + 4352 and lay.total_words == 592 + 64 + 272


def test_cfg_has_the_keys_the_trainer_stores():
    params = [torch.zeros(2000), torch.zeros(10), torch.zeros(50, 40)]
    cfg = ptcomp.init_grad_comp_cfg(params, kn=4, grad_comp_cfg={"grad_comp_threshold": 0.25}, device="cpu",
                                    rank=2)
    # necklace/trainer/tnopmx.py:145-151
    for key in ("grd_resi", "grd_recv", "grd_comp", "grd_cmps", "grad_size_threshold", "grad_comp_threshold"):
        assert key in cfg
    assert cfg["grad_size_threshold"] == 1001 and cfg["grad_comp_threshold"] == 0.25
    assert cfg["grd_cmps"] == [True, False, True]
    assert cfg["grd_resi"][1] is None and cfg["grd_resi"][0].shape == (2000,)
    assert cfg["grd_recv"][0].shape == (4, 125) and cfg["grd_comp"][2].shape == (125,)
    gc = cfg["compressor"]
    # this rank's payload lives in its own receive slot: no copy before the exchange
    assert gc.comp.data_ptr() == gc.recv[2].data_ptr()
    resi, recv, comp, cmps = ptcomp.init_grads_compression(params, 4, device="cpu")
    assert cmps == [True, False, True] and len(resi) == len(recv) == len(comp) == 3


def test_argument_errors():
    with pytest.raises(ValueError):
        ptcomp.GradCompressor([100], kn=0, device="cpu")
    with pytest.raises(ValueError):
        ptcomp.GradCompressor([100], kn=2, rank=2, device="cpu")
    gc = ptcomp.GradCompressor([2000, 3000], kn=2, device="cpu")
    with pytest.raises(ValueError):
        gc.compress([torch.zeros(2000)])
    with pytest.raises(ValueError):
        gc.compress([torch.zeros(2000), torch.zeros(2999)])
    with pytest.raises(TypeError):  # host tensors never reach a CPU path: there is none
        gc.compress([torch.zeros(2000), torch.zeros(3000)])
    with pytest.raises(ValueError):
        gc.compress_flat(torch.zeros(5000))
    with pytest.raises(ValueError):
        ptcomp.quantize_chunked(torch.zeros(64), torch.zeros(4, dtype=torch.int32), torch.zeros(64), 0.5, chunk=24)
    with pytest.raises(ValueError):
        ptcomp.grads_do_compressed_exchange([torch.zeros(2000), torch.zeros(3000)], 3, {"compressor": gc})


def test_state_round_trip():
    gc = ptcomp.GradCompressor([2000], kn=1, device="cpu")
    gc.resi.normal_()
    st = {k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in gc.state_dict().items()}
    gc2 = ptcomp.GradCompressor([2000], kn=1, device="cpu")
    gc2.load_state_dict(st)
    assert torch.equal(gc2.resi, gc.resi)
    with pytest.raises(ValueError):
        ptcomp.GradCompressor([2001], kn=1, device="cpu").load_state_dict(st)


def test_bucketing_follows_the_reference_rule():
    """Consecutive tensors, a new bucket when the next one would pass the limit, an oversized tensor
    alone (the shape of _take_tensors at necklace/frmwrk/pytorch/ptprms.py:258)."""
    ts = [torch.zeros(n) for n in (100, 200, 300, 1000, 50, 60)]
    sizes = lambda bs: [[t.numel() for t in b] for b in bs]
    assert sizes(ptcomp._take_buckets(ts, 4 * 600)) == [[100, 200, 300], [1000], [50, 60]]
    assert sizes(ptcomp._take_buckets(ts, 4 * 10 ** 6)) == [[100, 200, 300, 1000, 50, 60]]
    assert sizes(ptcomp._take_buckets(ts, 1)) == [[100], [200], [300], [1000], [50], [60]]
    assert ptcomp._take_buckets([], 1024) == []


def test_layout_is_rebuilt_when_the_optimizer_changes_and_residuals_move_along():
    a, b = torch.nn.Parameter(torch.zeros(3000)), torch.nn.Parameter(torch.zeros(500))
    cfg = {"grad_comp_threshold": 0.25, "grad_size_threshold": 1001, "rank": 0}
    gc1 = ptcomp._cfg_for_params([a, b], 2, cfg)
    assert gc1.grd_cmps == [True, False] and ptcomp._cfg_for_params([a, b], 2, cfg) is gc1  # kept while nothing changes
    gc1.grd_resi[0].copy_(torch.arange(3000, dtype=torch.float32))
    d = torch.nn.Parameter(torch.zeros(2000))
    gc2 = ptcomp._cfg_for_params([a, b, d], 2, cfg)
    assert gc2 is not gc1 and gc2.grd_cmps == [True, False, True]
    assert torch.equal(gc2.grd_resi[0], torch.arange(3000, dtype=torch.float32))  # what a is owed survives
    assert float(gc2.grd_resi[2].abs().sum()) == 0.0
    assert cfg["compressor"] is gc2 and cfg["grad_comp_threshold"] == 0.25


def test_small_gradients_need_a_collective_when_there_are_several_workers():
    g = [torch.ones(10), torch.ones(20)]
    ptcomp._reduce_small(g, 1, None, True)            # one worker: nothing to do
    with pytest.raises(ValueError):
        ptcomp._reduce_small(g, 2, None, True)
    seen = []

    def allreduce(flat):
        seen.append(flat.numel())
        flat.mul_(2.0)                                # a second worker with the same values

    ptcomp._reduce_small(g, 2, allreduce, True)
    assert seen == [30] and all(float(t.sum()) == t.numel() for t in g)   # (1 + 1) / 2
    ptcomp._reduce_small(g, 2, allreduce, False)
    assert all(float(t.sum()) == 2 * t.numel() for t in g)                # the reduce form: summed, not averaged


def test_model_form_refuses_a_gradient_that_requires_grad():
    """As necklace/frmwrk/pytorch/ptprms.py:307-310 does, before anything is laid out."""
    model = torch.nn.Linear(4, 3)
    model.weight.grad = torch.zeros(3, 4, requires_grad=True)
    with pytest.raises(RuntimeError):
        ptcomp.grads_do_nccl_allreduce(None, 1, model, None, grad_comp_cfg={})
    model.weight.grad = torch.zeros(3, 4)
    with pytest.raises(ValueError):  # the compressed path needs its configuration
        ptcomp.grads_do_nccl_allreduce(None, 1, model, None, grad_comp_cfg=None)


def _params(*numels):
    return [torch.nn.Parameter(torch.zeros(n)) for n in numels]


def test_residuals_from_a_checkpoint_survive_the_first_drop_in_call():
    """save -> new process -> init_grad_comp_cfg -> load -> first opt_*_do_nccl_* call: the layout step of
    that call must take the restored compressor as it is, not build a zeroed one over it."""
    params = _params(3000, 10, 5000)
    cfg = ptcomp.init_grad_comp_cfg(params, 2, {"grad_comp_threshold": 0.25}, device="cpu", rank=1)
    cfg["compressor"].resi.normal_()
    state = ptcomp.grad_comp_state(cfg)
    # a restart: same shapes, new parameter objects (other id()s), a fresh dict
    params2 = _params(3000, 10, 5000)
    cfg2 = ptcomp.init_grad_comp_cfg(params2, 2, {"grad_comp_threshold": 0.5}, device="cpu", rank=1)
    ptcomp.load_grad_comp_state(cfg2, state)
    want = state["resi"].clone()
    gc = ptcomp._cfg_for_params(params2, 2, cfg2)
    assert gc is cfg2["compressor"] and gc.rank == 1 and gc.thrd == 0.25
    assert torch.equal(gc.resi, want) and float(want.abs().sum()) > 0
    assert ptcomp._cfg_for_params(params2, 2, cfg2) is gc  # and it stays
    # restored into a dict that has only been configured: kept until the first call lays the buffers out
    cfg3 = {"grad_comp_threshold": 0.5, "rank": 1}
    ptcomp.load_grad_comp_state(cfg3, state)
    gc3 = ptcomp._cfg_for_params(_params(3000, 10, 5000), 2, cfg3)
    assert torch.equal(gc3.resi, want) and gc3.thrd == 0.25 and "_pending_state" not in cfg3
    # a state that belongs to other parameters is refused, not dropped
    cfg4 = {"rank": 0}
    ptcomp.load_grad_comp_state(cfg4, state)
    with pytest.raises(ValueError):
        ptcomp._cfg_for_params(_params(3000, 10, 5001), 2, cfg4)


def test_bucket_state_is_kept_per_parameter_position():
    """What the bucket form saves can be taken up by another bucketing (other bucket limits, a
    parameter that sits out) and by the per-parameter form: it is keyed by the parameter's position."""
    gc = ptcomp.GradCompressor([5000, 7000], kn=1, size_threshold=1, device="cpu")
    gc.resi.normal_()
    cfg = {"compressor": gc, "_signature": ("buckets", ((3000, 2000), (7000,)), 1),
           "_places": {0: (0, 0, 3000), 2: (0, 3000, 2000), 3: (1, 0, 7000)},
           "_parked": {1: torch.full((40,), 3.0)}}
    state = ptcomp.grad_comp_state(cfg)
    assert state["form"] == "buckets" and sorted(state["param_resi"]) == [0, 1, 2, 3]
    assert torch.equal(state["param_resi"][2], gc.grd_resi[0][3000:5000])
    assert torch.equal(state["param_resi"][1], torch.full((40,), 3.0))
    # into one bucket of three of the parameters (position 2 has no gradient this step)
    gc2 = ptcomp.GradCompressor([10040], kn=1, size_threshold=1, device="cpu")
    cfg2 = {"_pending_state": state}
    ptcomp._apply_pending_state(cfg2, gc2, {0: (0, 0, 3000), 1: (0, 3000, 40), 3: (0, 3040, 7000)})
    assert torch.equal(gc2.grd_resi[0][:3000], state["param_resi"][0])
    assert torch.equal(gc2.grd_resi[0][3000:3040], torch.full((40,), 3.0))
    assert torch.equal(gc2.grd_resi[0][3040:], state["param_resi"][3])
    assert torch.equal(cfg2["_parked"][2], state["param_resi"][2])   # set aside until it has a gradient again
    # into the per-parameter form
    gc3 = ptcomp.GradCompressor([3000, 40, 2000, 7000], kn=1, size_threshold=1001, device="cpu")
    ptcomp._apply_pending_state({"_pending_state": state}, gc3)
    assert torch.equal(gc3.grd_resi[0], state["param_resi"][0]) and gc3.grd_resi[1] is None
    assert torch.equal(gc3.grd_resi[3], state["param_resi"][3])


def test_rank_is_required_with_several_workers():
    class Comm:
        rank = 3
    assert ptcomp._rank_of(None, {}, 1) == 0
    assert ptcomp._rank_of(None, {"rank": 2}, 4) == 2
    assert ptcomp._rank_of(Comm(), {}, 4) == 3          # taken from the communicator object
    with pytest.raises(ValueError):
        ptcomp._rank_of(None, {}, 2)
    with pytest.raises(ValueError):
        ptcomp._rank_of(lambda comp, recv: None, {}, 2)  # a bare exchange callable knows no rank
    params = _params(3000)
    with pytest.raises(ValueError):
        ptcomp._cfg_for_params(params, 2, {})
    with pytest.raises(ValueError):
        ptcomp.opt_grads_fltn_do_nccl_reduce(None, 2, 0, torch.zeros(64), 64, grad_comp_cfg={})
    with pytest.raises(ValueError):                      # the dict says 1, the argument 0
        ptcomp.init_grad_comp_cfg(params, 2, {"rank": 1}, device="cpu", rank=0)
    cfg = ptcomp.init_grad_comp_cfg(params, 2, {}, device="cpu", rank=0)
    assert cfg["rank"] == 0
    rankless = {k: v for k, v in cfg.items() if k != "rank"}

    class Other:
        rank = 1
    with pytest.raises(ValueError):                      # the communicator says 1, the buffers were laid out for 0
        ptcomp._cfg_for_params(params, 2, rankless, Other())


def test_buffers_set_up_without_a_rank_assume_none():
    """The reference's set-up call passes no rank (necklace/trainer/tnopmx.py:140-143).  The payload then
    has a buffer of its own instead of a slot of the receive buffer, and a reduce onto a root, which has
    to know who this worker is, raises; nothing ever assumes worker 0."""
    params = _params(3000, 5000)
    resi, recv, comp, cmps = ptcomp.init_grads_compression(params, 4, device="cpu")
    gc_rankless = ptcomp.GradCompressor([3000, 5000], kn=4, device="cpu")
    assert gc_rankless.rank is None
    lo, hi = gc_rankless.recv.data_ptr(), gc_rankless.recv.data_ptr() + 4 * gc_rankless.recv.numel()
    assert not lo <= gc_rankless.comp.data_ptr() < hi          # not a slot of the receive buffer
    assert all(not lo <= c.data_ptr() < hi for c in gc_rankless.grd_comp if c is not None)
    gc1 = ptcomp.GradCompressor([3000], kn=1, device="cpu")
    assert gc1.rank == 0 and gc1.comp.data_ptr() == gc1.recv.data_ptr()
    gc2 = ptcomp.GradCompressor([3000], kn=4, device="cpu", rank=2)
    assert gc2.comp.data_ptr() == gc2.recv[2].data_ptr()
    with pytest.raises(ValueError, match="rank"):
        ptcomp._decodes(gc_rankless, 0)
    assert ptcomp._decodes(gc_rankless, None) and ptcomp._decodes(gc2, 2) and not ptcomp._decodes(gc2, 1)
    cfg = ptcomp.init_grad_comp_cfg(params, 4, {}, device="cpu")
    assert "rank" not in cfg and cfg["compressor"].rank is None


def test_gradients_that_are_not_float32_are_refused_up_front():
    """The reference buckets per tensor type (ptprms.py:258); the compressed path takes fp32 only and
    says so before anything is laid out or launched."""
    for form in ("params", "buckets"):
        a, b = torch.nn.Parameter(torch.zeros(3000)), torch.nn.Parameter(torch.zeros(2000, dtype=torch.bfloat16))
        a.grad, b.grad = torch.zeros(3000), torch.zeros(2000, dtype=torch.bfloat16)
        opt = torch.optim.SGD([a, b], lr=0.1)
        cfg = {"form": form}
        with pytest.raises(TypeError, match="float32"):
            ptcomp.opt_grads_do_nccl_allreduce(None, 1, opt, None, grad_comp_cfg=cfg)
        assert "compressor" not in cfg
