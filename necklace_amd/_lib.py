"""ctypes binding of libnklq.so (declarations: include/nklq.h).

There is no fallback: if the library is missing or a call fails, an exception
is raised.  Nothing here computes on the CPU.

`tuning_lib()` binds libnklq_tuning.so, the measurement build of the same source
(include/nklq_tuning.h): every geometry nklq_tune can name, a copy kernel and the
sum over interleaved payloads.  The package never loads it by itself; sweeps and
tests that want it either call it directly or make it the bound library for a
while with `use_tuning_library()`.
"""
import contextlib
import ctypes as ct
import os

# torch first: it carries its own copy of the HIP runtime (soname libamdhip64.so.7).  Loaded
# before libnklq.so, that copy also satisfies libnklq's dependency, so tensors and kernels
# share one runtime; the other way round the process ends up with two runtimes and the second
# one finds no device.
import torch  # noqa: F401

_PKG = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_PKG, "libnklq.so")
TUNING_SO_PATH = os.path.join(_PKG, "libnklq_tuning.so")

NKLQ_MAX_PAYLOADS_PER_LAUNCH = 16

SYMBOLS = (
    "nklq_quantize_f32", "nklq_dequantize_f32", "nklq_dequant_accumulate_f32",
    "nklq_quantize_multi_f32", "nklq_dequant_accumulate_multi_f32",
    "nklq_packed_words", "nklq_strerror", "nklq_version", "nklq_tune",
)
TUNING_SYMBOLS = ("nklq_copy_f32", "nklq_tuning_sum_interleaved_f32")

_lib = None
_tuning = None


class NklqError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"libnklq error {code}: {text}")
        self.code = code


def _bind(path, tuning):
    L = ct.CDLL(path)
    vp, u64, f32, i32 = ct.c_void_p, ct.c_uint64, ct.c_float, ct.c_int
    L.nklq_quantize_f32.argtypes = [vp, vp, vp, vp, u64, u64, f32, i32, vp]
    L.nklq_quantize_f32.restype = i32
    L.nklq_dequantize_f32.argtypes = [vp, vp, u64, u64, f32, vp]
    L.nklq_dequantize_f32.restype = i32
    L.nklq_dequant_accumulate_f32.argtypes = [vp, ct.POINTER(vp), i32, u64, f32, i32, vp]
    L.nklq_dequant_accumulate_f32.restype = i32
    L.nklq_quantize_multi_f32.argtypes = [i32, ct.POINTER(vp), ct.POINTER(vp), ct.POINTER(vp),
                                          ct.POINTER(u64), f32, i32, vp]
    L.nklq_quantize_multi_f32.restype = i32
    L.nklq_dequant_accumulate_multi_f32.argtypes = [i32, ct.POINTER(vp), ct.POINTER(u64), ct.POINTER(u64),
                                                    ct.POINTER(vp), i32, f32, i32, f32, vp]
    L.nklq_dequant_accumulate_multi_f32.restype = i32
    L.nklq_packed_words.argtypes = [u64, u64]
    L.nklq_packed_words.restype = u64
    L.nklq_strerror.argtypes = [i32]
    L.nklq_strerror.restype = ct.c_char_p
    L.nklq_version.argtypes = []
    L.nklq_version.restype = i32
    L.nklq_tune.argtypes = [i32, i32]
    L.nklq_tune.restype = i32
    if tuning:
        L.nklq_copy_f32.argtypes = [vp, vp, u64, vp]
        L.nklq_copy_f32.restype = i32
        L.nklq_tuning_sum_interleaved_f32.argtypes = [vp, vp, i32, u64, i32, f32, vp]
        L.nklq_tuning_sum_interleaved_f32.restype = i32
    return L


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(SO_PATH):
        raise ImportError(
            f"{SO_PATH} is missing: build it with `python -m necklace_amd.csrc.build` "
            "(needs hipcc; there is no CPU fallback)")
    _lib = _bind(SO_PATH, tuning=False)
    return _lib


def tuning_lib():
    """The measurement build (every launch geometry, copy kernel, interleaved sum); raises if not built."""
    global _tuning
    if _tuning is not None:
        return _tuning
    if not os.path.exists(TUNING_SO_PATH):
        raise ImportError(
            f"{TUNING_SO_PATH} is missing: build it with `python -m necklace_amd.csrc.build --tuning`")
    _tuning = _bind(TUNING_SO_PATH, tuning=True)
    return _tuning


@contextlib.contextmanager
def use_tuning_library():
    """Inside the block `lib()`, and with it every wrapper of the package, is the measurement build."""
    global _lib
    before = _lib
    _lib = tuning_lib()
    try:
        yield _lib
    finally:
        _lib = before


def check(code):
    if code != 0:
        raise NklqError(code, lib().nklq_strerror(code).decode())


def packed_words(n_rows, n_cols=1):
    return int(lib().nklq_packed_words(n_rows, n_cols))


TUNE_CHUNKS_PER_WAVE, TUNE_WORKGROUP_SIZE, TUNE_NONTEMPORAL = 0, 1, 2
TUNE_XCD_INTERLEAVE_LOG2, TUNE_XCD_INTERLEAVE_LOG2_DECODE, TUNE_XCD_INTERLEAVE_LOG2_ACCUMULATE = 3, 4, 5
TUNE_DECODE_PREFETCH = 6
N_TUNE = 7


def tune(which, value=-1):
    r = lib().nklq_tune(which, value)
    if r < 0:
        raise ValueError(f"nklq_tune({which}, {value}) rejected")
    return r
