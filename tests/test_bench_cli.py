"""bench.py's command line, as far as it can be checked without a GPU."""
import os
import subprocess
import sys

from conftest import ROOT


def _run(*args):
    env = dict(os.environ)
    env.pop("WORLD_SIZE", None)
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True,
                          text=True, timeout=300, env=env)


def test_more_than_one_gpu_is_refused_with_a_message():
    out = _run("--gpus", "2")
    assert out.returncode == 2
    assert "ONE GPU" in out.stderr
    assert out.stdout.strip() == ""


def test_bad_chunk_is_refused():
    out = _run("--chunk", "24", "--elems", "4096")
    assert out.returncode == 2
    assert "--chunk" in out.stderr
    assert out.stdout.strip() == ""
