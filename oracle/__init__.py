"""CPU checker for the 2-bit gradient quantizer — TEST INFRASTRUCTURE ONLY.

Only the tests, ``__graft_entry__.smoke()`` and the CPU-baseline leg of
``bench.py`` may import this package; the shipped package never does.

Two independent restatements of necklace/cuda/quantize.py:16-87 live here:

* ``oracle.c``   — ctypes view of ``nklq_oracle.c`` (scalar loops in the order
  one reference thread walks them; OpenMP over word rows for large inputs);
* ``oracle.vec`` — ``oracle_np.py``, whole-array numpy arithmetic.

They share no code, so a slip in one (a wrong shift, a swapped branch, a
dropped tail guard) shows up as a disagreement between them as well as
against the hand-worked known-answer vectors in ``tests/golden``.
"""
from . import oracle_np as vec  # noqa: F401
from . import oracle_c as c  # noqa: F401
from .oracle_c import build  # noqa: F401
