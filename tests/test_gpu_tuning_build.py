"""The two entry points only the measurement build exports (include/nklq_tuning.h), on the GPU:
the copy used to calibrate the HBM counters, and the fixed-order sum over payloads that alternate
inside one array, bit for bit against the CPU oracle's sum over the same payloads."""
import numpy as np
import pytest
import torch

import oracle
from conftest import assert_bits_equal
from gpu_util import dev
from necklace_amd import _lib

pytestmark = pytest.mark.gpu


def test_copy_moves_every_element():
    T = _lib.tuning_lib()
    stream = torch.cuda.current_stream().cuda_stream
    for n in (1, 255, 256, 1024 * 37 + 5, 3_000_001):
        src = torch.randn(n, device="cuda")
        dst = torch.zeros(n, device="cuda")
        _lib.check(T.nklq_copy_f32(dst.data_ptr(), src.data_ptr(), n, stream))
        assert torch.equal(dst, src), n


@pytest.mark.parametrize("k_payloads", [1, 3, 8, 9, 16])
@pytest.mark.parametrize("run_log2", [6, 7, 10, 14, 20])
def test_sum_over_interleaved_payloads(k_payloads, run_log2):
    T = _lib.tuning_lib()
    stream = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(1000 * k_payloads + run_log2)
    run = 1 << run_log2
    for n in (1024, 1024 * 3, 1024 * 257):
        wl = n // 16
        pl = [rng.integers(0, 2 ** 32, size=wl, dtype=np.uint64).astype(np.uint32) for _ in range(k_payloads)]
        want = oracle.c.dequant_accumulate(pl, n, 2e-3)
        runs = (wl + run - 1) // run
        # (runs, k, run) words: run j of payload p starts at word (j * k + p) * run
        d = torch.zeros((runs, k_payloads, run), dtype=torch.int32, device="cuda")
        for p in range(k_payloads):
            padded = torch.zeros(runs * run, dtype=torch.int32, device="cuda")
            padded[:wl] = dev(pl[p])
            d[:, p, :] = padded.view(runs, run)
        acc = torch.full((n,), 7.0, device="cuda")
        _lib.check(T.nklq_tuning_sum_interleaved_f32(acc.data_ptr(), d.data_ptr(), k_payloads, n, run_log2,
                                                     2e-3, stream))
        assert_bits_equal(acc.cpu().numpy(), want, f"n={n} k={k_payloads} run=2^{run_log2}")
