"""Host-side behaviour of the Python surface that mirrors necklace/cuda/quantize.py
(names, keyword arguments, argument errors).  Runs without a GPU."""
import inspect

import numpy as np
import pytest
import torch

from necklace_amd.cuda import nbutils, quantize as q


def test_constants_match_reference_module():
    # necklace/cuda/quantize.py:8-13
    assert (q.CMP_RATIO, q.g, q.e, q.l, q.msk) == (16, 0b01, 0b00, 0b10, 0b11)


@pytest.mark.parametrize("fn", [q.cu_fn_matrix_quantize_e, q.cu_fn_matrix_dequantize_e])
def test_wrapper_signature_matches_reference(fn):
    # necklace/cuda/quantize.py:96-99 and :118-121
    p = inspect.signature(fn).parameters
    assert list(p)[:8] == ["A", "C", "R", "thrd", "bpg", "tpb", "to_device", "stream"]
    assert p["thrd"].default == 0.3 and p["bpg"].default == 4 and p["tpb"].default == 128
    assert p["to_device"].default is False and p["stream"].default is None


def test_kernel_objects_take_launch_configuration():
    # necklace/cuda/quantize.py:112: knl[(bpg, bpg), (tpb // 16, tpb), stream](dA, dC, dR, thrd)
    launch = q.cu_knl_matrix_quantize_e[(4, 4), (8, 128), None]
    assert callable(launch)
    assert callable(q.cu_knl_matrix_dequantize_e[(4, 4), (8, 128)])


def test_wrong_dtype_and_rank_raise_type_error_like_numba_signature_mismatch():
    A = torch.zeros(4, 4)
    C = torch.zeros(1, 4, dtype=torch.int32)
    with pytest.raises(TypeError):
        q.cu_fn_matrix_quantize_e(A.double(), C, A)
    with pytest.raises(TypeError):
        q.cu_fn_matrix_quantize_e(A.reshape(2, 2, 4), C, A)
    with pytest.raises(TypeError):  # host tensors need to_device=True
        q.cu_fn_matrix_quantize_e(A, C, A.clone())
    with pytest.raises(TypeError):
        q.cu_fn_matrix_quantize_e(np.zeros((4, 4), np.float32), C, A)


def test_packed_rows():
    assert [q.packed_rows(n) for n in (1, 15, 16, 17, 224)] == [1, 1, 1, 2, 14]


def test_nbutils_names_exist():
    for name in ("cuda_select_device", "cuda_current_context", "cuda_stream", "cuda_to_device",
                 "cuda_devarr_c_void_p"):
        assert callable(getattr(nbutils, name))  # necklace/cuda/nbutils.py:11-39
