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
