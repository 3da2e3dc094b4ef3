"""The entry points allocate nothing and touch only the stream they are given, so a training
step's compress / decompress can be captured in a HIP graph and replayed."""
import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal, assert_words_equal
from gpu_util import dev, host_words, random_payloads_gpu
from necklace_amd.frmwrk.pytorch import ptcomp

pytestmark = pytest.mark.gpu


def test_compress_and_decompress_replayed_from_a_hip_graph():
    sizes = [5000, 100, 70001, 4096, 1, 33333]
    kn, rank, thrd = 3, 0, 1e-3
    gc = ptcomp.GradCompressor(sizes, kn, thrd=thrd, rank=rank)
    lay = gc.layout
    grads = [torch.zeros(s, device="cuda") for s in sizes]      # static input buffers of the graph
    outs = [torch.zeros(s, device="cuda") for s in sizes]
    peers = random_payloads_gpu(kn, 16 * lay.total_words, 5)
    gc.recv.copy_(peers)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                                # warm-up outside the capture
        gc.compress(grads)
        gc.decompress_sum(outs)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    gc.resi.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gc.compress(grads)
        gc.decompress_sum(outs, average=True)
    gc.resi.zero_()                                              # capture does not execute
    rng = np.random.default_rng(12)
    resid = [np.zeros(s, np.float32) for s in sizes]
    peers_host = host_words(peers)
    for step in range(4):
        gh = [rng.normal(0, 1e-3, s).astype(np.float32) for s in sizes]
        for t, a in zip(grads, gh):
            t.copy_(dev(a))                                      # eager work between the replays
        graph.replay()
        torch.cuda.synchronize()
        for i, s in enumerate(sizes):
            if s < 1001:
                continue
            want_c, want_r = oracle.c.quantize(gh[i], thrd, R_in=resid[i])
            resid[i] = want_r
            assert_words_equal(host_words(gc.grd_comp[i]), want_c, f"replay {step} param {i}")
            assert_bits_equal(gc.grd_resi[i].cpu().numpy(), want_r, f"replay {step} param {i}")
            wo, w = lay.word_offset[i], lay.words[i]
            pl = [peers_host[k, wo:wo + w].copy() for k in range(kn)]
            pl[rank] = want_c
            want = (oracle.c.dequant_accumulate(pl, s, thrd) / np.float32(kn)).astype(np.float32)
            assert_bits_equal(outs[i].cpu().numpy(), want, f"replay {step} param {i} sum")
