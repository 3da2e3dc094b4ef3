"""MI355X-native 2-bit gradient quantizer with the call surface of necklace.cuda.quantize.

Only the quantization hot path of necklace is provided here:

* ``necklace_amd.cuda.quantize`` — same names as necklace/cuda/quantize.py
  (``cu_fn_matrix_quantize_e``, ``cu_fn_matrix_dequantize_e``, the constants), running
  hand-written HIP kernels for gfx950 through a ctypes C-ABI (include/nklq.h);
* ``necklace_amd.cuda.nbutils`` — the device helpers of necklace/cuda/nbutils.py on
  PyTorch-ROCm instead of numba;
* ``necklace_amd.frmwrk.pytorch.ptcomp`` — trainer-side buffers for compressed
  gradient exchange (what necklace/trainer/tnopmx.py:135-151 expects of the
  ``mxprms`` module missing from the reference tree).
"""

__version__ = "1.0.0"


def init(gpu=None):
    """Counterpart of necklace.init (necklace/__init__.py:8-38): pick the GPU before anything else."""
    if gpu is not None:
        from .cuda import nbutils
        nbutils.cuda_select_device(int(gpu))
