"""Compiles csrc/nklq.hip for gfx950 (MI355X).

    python -m necklace_amd.csrc.build            # necklace_amd/libnklq.so, the product library
    python -m necklace_amd.csrc.build --tuning   # necklace_amd/libnklq_tuning.so as well

The tuning library is the same source with -DNKLQ_TUNING_BUILD=1: every launch geometry nklq_tune
can name, a copy kernel and the sum over interleaved payloads (include/nklq_tuning.h).  Only the
geometry sweeps of bench.py and the parity tests that run every geometry load it.

hipcc cross-compiles without a GPU present.  The libraries are kept inside the
package directory so that they are found next to the Python sources.
"""
import os
import subprocess
import sys

CSRC = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(CSRC)
ROOT = os.path.dirname(PKG)
SO_PATH = os.path.join(PKG, "libnklq.so")
TUNING_SO_PATH = os.path.join(PKG, "libnklq_tuning.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-shared", "-fPIC", "-std=c++17",
    # IEEE fp32: no contraction, no fast-math, denormals kept (hipcc's default)
    "-ffp-contract=off", "-fno-fast-math",
    # keep the compiler from forming packed-fp32 VALU ops out of the float4 arithmetic
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def build(verbose=False, tuning=False):
    """Compile the product library, or with tuning=True the measurement build of the same source."""
    target = TUNING_SO_PATH if tuning else SO_PATH
    cmd = [HIPCC, *FLAGS, *(["-DNKLQ_TUNING_BUILD=1"] if tuning else []), "-I", os.path.join(ROOT, "include"),
           os.path.join(CSRC, "nklq.hip"), "-o", target]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only feature flag and says so; that is harmless
    noise = ("packed-fp32-ops", "is not a recognized feature")
    out = "\n".join(l for l in res.stdout.splitlines() if not any(s in l for s in noise))
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{out}")
    if verbose and out.strip():
        print(out)
    return target


def ensure_built(tuning=False):
    """Build only when no library is there yet (a fresh checkout: the .so is not in version control)."""
    target = TUNING_SO_PATH if tuning else SO_PATH
    if not os.path.exists(target):
        build(tuning=tuning)
    return target


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
    if "--tuning" in sys.argv:
        print(build(verbose="-q" not in sys.argv, tuning=True))
