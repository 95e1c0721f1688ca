"""bench.py's command line, as far as it can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    p = _run("--gpus", "2")
    assert p.returncode != 0 and "one GPU" in p.stderr and p.stdout.strip() == ""


def test_help_names_the_contract_flags():
    p = _run("--help")
    assert p.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup"):
        assert flag in p.stdout
