"""Host-side sanitizer runs (AddressSanitizer + UndefinedBehaviorSanitizer, CPU only).

The reference's failure contract for a device call is a status code and a CPU
fallback (storage/cuda_d_cuda.v:39-42,69-77, nn/layers/linear_forward_f32.v:8-11);
what it cannot survive is host code that reads or writes out of bounds.  Two
programs are built with -fsanitize=address,undefined and run:
  * tests/sanitize/oracle_sanitized.c walks every function of the CPU oracle over
    ragged shapes (empty, single element, odd lengths, the longest K) with
    exactly sized heap buffers;
  * the C++ host mirror's test program in its --no-device mode (argument checks,
    error paths and object lifetimes of HipStorage / HipTensor / HipSession).
GPU code is not instrumented: device sanitizers do not run on this pool, so the
device side is covered by guard bands around every buffer of the ragged-shape
parity tests instead (conftest.py: guard_bands).
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SAN = os.path.join(HERE, "sanitize")


def _build(target):
    res = subprocess.run(["make", "-C", SAN, "-B", target], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                         text=True, timeout=300)
    assert res.returncode == 0, res.stdout[-3000:]
    return os.path.join(SAN, target)


def _run(exe, *args):
    env = dict(os.environ, UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1",
               # the HIP runtime that libvtlhip.so links keeps allocations until exit: leaks are not the question
               ASAN_OPTIONS="detect_leaks=0:abort_on_error=0:verify_asan_link_order=0")
    return subprocess.run([exe, *args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300,
                          env=env)


def test_oracle_under_asan_and_ubsan():
    res = _run(_build("oracle_sanitized"))
    assert res.returncode == 0 and "oracle under sanitizers: ok" in res.stdout, res.stdout[-3000:]
    assert "runtime error" not in res.stdout and "AddressSanitizer" not in res.stdout, res.stdout[-3000:]


def test_host_mirror_error_paths_under_asan_and_ubsan():
    res = _run(_build("host_mirror_sanitized"), "--no-device")
    assert res.returncode == 0 and "ok" in res.stdout, res.stdout[-3000:]
    assert "runtime error" not in res.stdout and "AddressSanitizer" not in res.stdout, res.stdout[-3000:]
