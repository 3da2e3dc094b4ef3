"""Compiles csrc/nklq.hip into necklace_amd/libnklq.so for gfx950 (MI355X).

    python -m necklace_amd.csrc.build

hipcc cross-compiles without a GPU present.  The library is kept inside the
package directory so that it is found next to the Python sources.
"""
import os
import subprocess
import sys

CSRC = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(CSRC)
ROOT = os.path.dirname(PKG)
SO_PATH = os.path.join(PKG, "libnklq.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-shared", "-fPIC", "-std=c++17",
    # IEEE fp32: no contraction, no fast-math, denormals kept (hipcc's default)
    "-ffp-contract=off", "-fno-fast-math",
    # keep the compiler from forming packed-fp32 VALU ops out of the float4 arithmetic
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def build(verbose=False):
    cmd = [HIPCC, *FLAGS, "-I", os.path.join(ROOT, "include"),
           os.path.join(CSRC, "nklq.hip"), "-o", SO_PATH]
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
    return SO_PATH


def ensure_built():
    """Build only when no library is there yet (a fresh checkout: the .so is not in version control)."""
    if not os.path.exists(SO_PATH):
        build()
    return SO_PATH


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
