"""The C-ABI from a caller with no Python and no torch in it: tests/c/abi_client.c."""
import os
import subprocess

import pytest

from conftest import ROOT

CDIR = os.path.join(ROOT, "tests", "c")
EXE = os.path.join(CDIR, "abi_client")


def _client():
    if not os.path.exists(EXE):
        subprocess.run(["make", "-s", "-C", CDIR], check=True)
    return EXE


def test_plain_c_caller_host_checks():
    out = subprocess.run([_client(), "host"], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr
    assert "ok" in out.stdout


@pytest.mark.gpu
def test_plain_c_caller_on_the_gpu():
    out = subprocess.run([_client(), "gpu"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "abi_client gpu: ok" in out.stdout
