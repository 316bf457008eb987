"""Runs the C++ host-mirror test program (tests/host_cpp/test_host_mirror.cpp),
the stand-in for the V callers: HipStorage / HipTensor / the Linear hook over
the C ABI, checked against the CPU oracle."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "host_cpp", "test_host_mirror")


def _binary():
    if not os.path.exists(BIN):   # built by __graft_entry__.build(); this is the CPU-side fallback
        subprocess.run(["make", "-C", os.path.join(HERE, "host_cpp")], check=True,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    return BIN


def test_host_mirror_error_paths_without_device():
    res = subprocess.run([_binary(), "--no-device"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                         text=True, timeout=60)
    assert res.returncode == 0, res.stdout
    assert "ok" in res.stdout


@pytest.mark.gpu
def test_host_mirror_on_device(hip):
    assert os.path.exists(BIN), "tests/host_cpp/test_host_mirror is not built"
    res = subprocess.run([BIN], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert res.returncode == 0, res.stdout
    assert "host mirror: ok" in res.stdout


def test_plain_c_consumer_of_the_abi():
    """tests/host_c/abi_check.c is C99 -pedantic -Werror: the header is valid C, the
    exports have C linkage, argument checks answer without a device."""
    cdir = os.path.join(HERE, "host_c")
    exe = os.path.join(cdir, "abi_check")
    if not os.path.exists(exe):   # built by __graft_entry__.build(); this is the CPU-side fallback
        subprocess.run(["make", "-C", cdir], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    res = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert res.returncode == 0 and "C ABI check: ok" in res.stdout, res.stdout
