"""bench.py's command-line contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    res = _run("--gpus", "2")
    assert res.returncode == 2
    assert "ONE GPU" in res.stderr and res.stdout == ""


def test_without_a_device_it_fails_loudly_instead_of_falling_back():
    from vtl_amd import capi
    if capi.device_count() > 0:
        return      # on a GPU box the benchmark itself is the check
    res = _run("--steps", "1", "--warmup", "0")
    assert res.returncode == 1 and "no HIP device" in res.stderr and res.stdout == ""
