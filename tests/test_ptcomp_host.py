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
    cfg = {"grad_comp_threshold": 0.25, "grad_size_threshold": 1001}
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
