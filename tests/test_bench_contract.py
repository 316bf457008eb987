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


def test_traffic_records_go_stale_with_their_source(tmp_path, monkeypatch):
    """roofline.traffic comes from the committed counter summary only while the kernel's source
    file still has the digest recorded there; otherwise the bench line says null."""
    import hashlib
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    src = tmp_path / "kernel.hip"
    src.write_text("__global__ void k() {}\n")
    digest = hashlib.sha256(src.read_bytes()).hexdigest()[:16]
    records = tmp_path / "traffic.md"
    records.write_text("# summary\n\n"
                       f"record: name=linear source={src} sha256={digest} bytes=168088496\n"
                       f"record: name=quantize source={tmp_path / 'missing.hip'} sha256={digest} bytes=1\n")
    monkeypatch.setattr(bench, "TRAFFIC_RECORDS", str(records))
    assert bench.measured_traffic("linear") == 168088496.0
    assert bench.measured_traffic("quantize") is None          # source file gone
    assert bench.measured_traffic("dequantize") is None        # no record
    src.write_text("__global__ void k() { }\n")                 # the kernel changed after the counter run
    assert bench.measured_traffic("linear") is None



def test_decode_and_chain_legs_time_the_configs_own_tensors():
    """The timed tensors of configs[3] and configs[4] are the seeded ones of vtl_amd.workloads
    (seeds 3 and 4), the same the parity tests and the golden fixtures use - no generator of
    the benchmark's own."""
    import importlib.util
    import inspect
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    dec = inspect.getsource(bench._bench_decode)
    chain = inspect.getsource(bench._bench_chain)
    assert "workloads.decode_linear(" in dec and "workloads.decode_linear_activations(" in dec
    assert "workloads.mlp_chain(" in chain
    for src in (dec, chain, inspect.getsource(bench._other_decode_chain)):
        assert "Philox" not in src and "default_rng" not in src and "rng." not in src
    # and the activations bench.py draws for a given M are the ones decode_linear(M) returns
    import numpy as np
    from vtl_amd import workloads
    x, _ = workloads.decode_linear(8, k=64, n=4)
    assert np.array_equal(x, workloads.decode_linear_activations(8, k=64))
