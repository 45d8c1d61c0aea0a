"""bench.py's command line where no GPU is needed: more than one GPU is refused with a message, and without a GPU
the script fails instead of printing a number."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300, cwd=ROOT)


def test_more_than_one_gpu_is_refused():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "--gpus 1" in (r.stdout + r.stderr)
    assert "{" not in r.stdout                      # no result line


def test_no_gpu_no_number():
    import torch
    if torch.cuda.is_available():
        return                                      # (covered by the GPU run of bench.py itself)
    r = _run("--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "{" not in r.stdout
