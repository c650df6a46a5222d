"""bench.py's command line on a machine without a GPU: the refusals are explicit and nothing falls back to the CPU."""
import os
import subprocess
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*flags):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], capture_output=True, text=True,
                          timeout=300, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and not r.stdout.strip()


@pytest.mark.skipif(torch.cuda.is_available(), reason="this is the behaviour without a GPU")
def test_without_a_gpu_there_is_no_cpu_fallback():
    r = _run("--steps", "1", "--warmup", "0")
    assert r.returncode != 0
    assert "no CPU fallback" in r.stderr and not r.stdout.strip()
