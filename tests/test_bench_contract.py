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


def test_counter_traffic_and_kernel_name_are_read_from_the_committed_profile():
    # roofline.traffic and roofline.kernel come from two lines of the committed counter summary; a refresh of that file
    # that drops them would silently turn both into null in the bench line
    import importlib.util

    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    traffic, kernel = mod.profile_figures()
    assert isinstance(traffic, int) and 33_095_680 <= traffic < 1.05 * 33_095_680  # at least the algorithmic bytes
    assert kernel and kernel.startswith("gemv_i4g32_mfma_kernel<")
