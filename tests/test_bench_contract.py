"""bench.py's command-line contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args, env=None):
    e = dict(os.environ)
    e.update(env or {})
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          env=e, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode == 2
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""
    r = _run(env={"WORLD_SIZE": "8"})
    assert r.returncode == 2 and "ONE GPU" in r.stderr


def test_without_a_gpu_it_fails_loudly_instead_of_falling_back():
    import torch
    if torch.cuda.is_available():
        return
    r = _run("--steps", "1", "--warmup", "0")
    assert r.returncode == 3
    assert "no GPU" in r.stderr and r.stdout.strip() == ""
