#!/usr/bin/env python3
"""Benchmark of the INT8 quantized-linear path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the int8 Linear at M=N=K=4096 (int8 MFMA GEMM with the
fused f32 scale/bias epilogue) over device-resident synthetic inputs.  The
same run also times the per-row quantize and dequantize of a [16384,16384]
f32 tensor (the bandwidth half of the metric) and the CPU oracle on a bounded
sample of each workload.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from vtl_amd import capi, workloads  # noqa: E402
from vtl_amd.tensor import HipTensor  # noqa: E402

METRIC = "int8 Linear TOPS @M=N=K=4096 + quant/dequant GB/s, % of MI355X roofline"
PEAK_INT8_TOPS = 5000.0      # dense int8 MFMA, MI355X published
PEAK_HBM_GBPS = 8000.0       # HBM3E, MI355X published
PEAK_FP64_TFLOPS = 78.6      # dense f64 MFMA, MI355X published

TRAFFIC_RECORDS = os.path.join(ROOT, "profiles", "bench_pmc_traffic.md")


def measured_traffic(name: str):
    """HBM-side bytes per launch of the kernel behind `name`, from the committed summary of
    the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script (each counter scaled by
    its reading for the 1 GiB copy kernel).  A record names the kernel's source file and the
    SHA-256 of that file when the counters were read; if the file has changed since, the
    figure is stale and None is reported instead."""
    import hashlib
    try:
        lines = open(TRAFFIC_RECORDS).read().splitlines()
    except OSError:
        return None
    for line in lines:
        if not line.startswith("record:"):
            continue
        rec = dict(kv.split("=", 1) for kv in line[len("record:"):].split())
        if rec.get("name") != name:
            continue
        try:
            digest = hashlib.sha256(open(os.path.join(ROOT, rec["source"]), "rb").read()).hexdigest()
        except OSError:
            return None
        return float(rec["bytes"]) if digest.startswith(rec["sha256"]) else None
    return None


class Timer:
    """hipEvent pair recorded on the stream the kernels are launched on."""

    def __init__(self):
        self.e0, self.e1 = C.c_void_p(), C.c_void_p()
        capi.call("vtl_hip_event_create", C.byref(self.e0))
        capi.call("vtl_hip_event_create", C.byref(self.e1))

    def run(self, fn, steps: int):
        """Returns (wall seconds, device milliseconds) for `steps` calls of fn."""
        capi.call("vtl_hip_sync")
        t0 = time.perf_counter()
        capi.call("vtl_hip_event_record", self.e0)
        for _ in range(steps):
            fn()
        capi.call("vtl_hip_event_record", self.e1)
        capi.call("vtl_hip_sync")
        wall = time.perf_counter() - t0
        ms = C.c_float()
        capi.call("vtl_hip_event_elapsed_ms", self.e0, self.e1, C.byref(ms))
        return wall, float(ms.value)

    def each(self, fn, steps: int):
        """Median and minimum over `steps` launches timed one by one, in microseconds
        (an event before every launch and one after the last; untimed by run())."""
        steps = max(1, min(steps, 50))
        evs = [C.c_void_p() for _ in range(steps + 1)]
        for e in evs:
            capi.call("vtl_hip_event_create", C.byref(e))
        capi.call("vtl_hip_sync")
        for i in range(steps):
            capi.call("vtl_hip_event_record", evs[i])
            fn()
        capi.call("vtl_hip_event_record", evs[steps])
        capi.call("vtl_hip_sync")
        out = []
        ms = C.c_float()
        for i in range(steps):
            capi.call("vtl_hip_event_elapsed_ms", evs[i], evs[i + 1], C.byref(ms))
            out.append(float(ms.value) * 1e3)
        for e in evs:
            capi.call("vtl_hip_event_destroy", e)
        return {"median_us": float(np.median(out)), "min_us": float(np.min(out)),
                "note": "launches separated by an event record each: includes that gap, unlike kernel_us"}


class PowerClockSampler:
    """Samples the card's shader clock (one reading per XCD), socket power and the
    power-throttle residency counter from a thread while the main thread keeps the GPU busy.
    Readings come from the amdsmi Python binding of the ROCm image (the driver's gpu_metrics
    table, which the firmware refreshes ONCE A SECOND: a load has to last a few seconds for
    two or three fresh readings), or, when that is not importable, from the amdgpu hwmon /
    pp_dpm_sclk sysfs files.  Measurement aid of this script only."""

    def __init__(self, hz: float = 20.0):
        import threading
        self.period = 1.0 / hz
        self.samples = []
        self._stop = threading.Event()
        self._thread = None
        self._handle = None
        self._smi = None
        self.source = None
        try:
            import amdsmi
            if not PowerClockSampler._smi_ready:
                amdsmi.amdsmi_init()
                PowerClockSampler._smi_ready = True
            self._handle = amdsmi.amdsmi_get_processor_handles()[0]
            amdsmi.amdsmi_get_gpu_metrics_info(self._handle)
            self._smi = amdsmi
            self.source = "amdsmi gpu_metrics (refreshed once a second)"
        except Exception:                      # noqa: BLE001 - any failure means: use sysfs
            self._smi = None
            import glob
            hw = glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")
            self._power_file = hw[0] if hw else None
            dpm = glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")
            self._sclk_file = dpm[0] if dpm else None
            self.source = "sysfs hwmon power1_input + pp_dpm_sclk" if hw or dpm else None

    _smi_ready = False

    def _read(self):
        if self._smi is not None:
            m = self._smi.amdsmi_get_gpu_metrics_info(self._handle)
            clks = [c for c in m.get("current_gfxclks", []) if isinstance(c, int) and 0 < c < 10000]
            return {"t": time.perf_counter(), "sclk": clks, "power_w": m.get("current_socket_power"),
                    "energy": m.get("energy_accumulator"), "ppt_acc": m.get("ppt_residency_acc"),
                    "acc": m.get("accumulation_counter"), "fw_t": m.get("firmware_timestamp")}
        rec = {"t": time.perf_counter(), "sclk": [], "power_w": None}
        try:
            if self._power_file:
                rec["power_w"] = int(open(self._power_file).read()) / 1e6
            if self._sclk_file:
                for line in open(self._sclk_file).read().splitlines():
                    if line.rstrip().endswith("*"):
                        rec["sclk"] = [int(line.split(":")[1].strip().split("M")[0])]
        except (OSError, ValueError):
            pass
        return rec

    def __enter__(self):
        import threading
        self.samples = []
        self._stop.clear()
        if self.source is None:
            return self

        def loop():
            while not self._stop.is_set():
                try:
                    self.samples.append(self._read())
                except Exception:              # noqa: BLE001
                    pass
                self._stop.wait(self.period)
        self._thread = threading.Thread(target=loop, daemon=True)
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        if self._thread:
            self._thread.join()
        return False

    def summary(self, skip_s: float = 1.05):
        """Means over the distinct readings taken later than skip_s after the start (a reading
        describes the second before it, and the clock settles over the first tens of
        milliseconds of load)."""
        if not self.samples:
            return {"source": self.source, "readings": 0}
        t0 = self.samples[0]["t"]
        distinct, seen = [], None
        for x in self.samples:
            key = (x.get("fw_t"), x.get("energy"), tuple(x["sclk"]), x.get("power_w"))
            if key != seen:
                distinct.append(x)
                seen = key
        if self._smi is not None:
            distinct = distinct[1:]            # the first one was refreshed before the load began
        ss = [x for x in distinct if x["t"] - t0 >= skip_s]
        if not ss:
            return {"source": self.source, "readings": 0,
                    "note": "load too short for a fresh reading (raise --load-seconds)"}
        clk = [np.mean(x["sclk"]) for x in ss if x["sclk"]]
        per_xcd = [x["sclk"] for x in ss if x["sclk"]]
        pw = [x["power_w"] for x in ss if isinstance(x.get("power_w"), (int, float))]
        out = {"source": self.source, "readings": len(ss),
               "sclk_mhz_mean": float(np.mean(clk)) if clk else None,
               "sclk_mhz_per_xcd_min": float(np.min(per_xcd)) if per_xcd else None,
               "sclk_mhz_per_xcd_max": float(np.max(per_xcd)) if per_xcd else None,
               "power_w_mean": float(np.mean(pw)) if pw else None}
        a, b = ss[0], ss[-1]
        ints = lambda k: isinstance(a.get(k), int) and isinstance(b.get(k), int)   # noqa: E731
        if len(ss) >= 2 and ints("energy") and ints("fw_t") and b["fw_t"] > a["fw_t"]:
            # energy accumulator in units of 2^-16 J, firmware timestamp in units of 10 ns
            out["power_w_from_energy_counter"] = ((b["energy"] - a["energy"]) * 15.259e-6 /
                                                  ((b["fw_t"] - a["fw_t"]) * 1e-8))
        if len(ss) >= 2 and ints("ppt_acc") and ints("acc") and b["acc"] > a["acc"]:
            out["power_throttle_residency"] = (b["ppt_acc"] - a["ppt_acc"]) / (b["acc"] - a["acc"])
        return out

    def idle(self):
        try:
            r = self._read() if self.source else None
        except Exception:                      # noqa: BLE001
            r = None
        return None if r is None else {"sclk_mhz": float(np.mean(r["sclk"])) if r["sclk"] else None,
                                       "power_w": r.get("power_w")}


def bench_linear(timer: Timer, steps: int, warmup: int, cpu: bool, load_s: float = 3.2, operands: str = "config"):
    m = n = k = 4096
    a, bt, sa, sb, bias = workloads.square_int8_gemm(m, n, k)
    if operands == "zeros":       # diagnostic: the same launch without the data-dependent power draw
        a, bt = np.zeros_like(a), np.zeros_like(bt)
    A, B = HipTensor.from_host(a), HipTensor.from_host(bt)
    SA, SB, BIAS = HipTensor.from_host(sa), HipTensor.from_host(sb), HipTensor.from_host(bias)
    Y = HipTensor.empty([m, n], np.float32)

    def step():
        capi.call("vtl_hip_linear_i8_f32", A.ptr, SA.ptr, 1, B.ptr, SB.ptr, 1, BIAS.ptr, Y.ptr, m, n, k, 0)

    for _ in range(warmup):
        step()
    wall, dev_ms = timer.run(step, steps)
    ops = 2.0 * m * n * k
    kernel_ms = dev_ms / steps
    per_launch = timer.each(step, steps)
    # shader clock and socket power while the same launch runs back to back for about load_s
    # seconds (timed by its own event pair; not part of `value`)
    under_load = None
    if load_s > 0:
        sampler = PowerClockSampler()
        idle = sampler.idle()
        n_load = max(steps, int(load_s / (kernel_ms * 1e-3)))
        with sampler:
            _, load_ms = timer.run(step, n_load)
        under_load = sampler.summary()
        under_load.update({"launches": n_load, "kernel_us": load_ms / n_load * 1e3, "idle_before": idle})
    res = {
        "per_launch": per_launch,
        "under_load": under_load,
        "ms_per_step": wall * 1e3 / steps,
        "tops": ops / (wall / steps) / 1e12,
        "roofline": {"kernel": "gemm_i8_dma_kernel<256,256,128,2,2,4,f32 epilogue>", "bound": "mfma",
                     "achieved": ops / (kernel_ms * 1e-3) / 1e12, "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": ops / (kernel_ms * 1e-3) / 1e12 / PEAK_INT8_TOPS,
                     "kernel_us": kernel_ms * 1e3, "algorithmic_ops": ops,
                     "traffic": measured_traffic("linear")},
    }
    if cpu:
        import oracle  # CPU baseline leg only
        flags = oracle.use_native_build()
        rows = m       # the whole workload, repeated for about ten seconds of CPU work: median pass

        def passes(threads, budget_s):
            ts, ref_, t_all = [], None, time.perf_counter()
            while not ts or (time.perf_counter() - t_all < budget_s and len(ts) < 50):
                t0 = time.perf_counter()
                ref_ = oracle.linear_i8_f32(a[:rows], sa[:rows], bt, sb, bias, threads=threads)
                ts.append(time.perf_counter() - t0)
            return float(np.median(ts)), len(ts), ref_
        dt1, n1, ref = passes(1, 10.0)
        threads = oracle.max_threads()
        rows_mt = m
        dtn, nn, _ = passes(threads, 3.0)
        got = Y.cpu()[:rows]
        res["parity_sample_bit_exact"] = bool(np.array_equal(got, ref))
        res["cpu_baseline"] = {"value": 2.0 * rows * n * k / dt1 / 1e12, "unit": "TOPS", "cores": 1,
                               "kind": "port", "build": flags,
                               "sample": f"the whole workload ({rows} rows of A against all of Bt), median of {n1} "
                                         f"passes of {dt1:.2f} s, 1 thread"}
        res["cpu_baseline_all_cores"] = {"value": 2.0 * rows_mt * n * k / dtn / 1e12, "unit": "TOPS",
                                         "cores": threads, "kind": "port",
                                         "build": flags,
                                         "sample": f"the whole workload, median of {nn} passes of {dtn:.2f} s, OpenMP"}
    for h in (A, B, SA, SB, BIAS, Y):
        h.release()
    return res


def bench_quant(timer: Timer, steps: int, warmup: int, cpu: bool):
    rows = cols = 16384
    x = workloads.outlier_matrix(rows, cols)
    X = HipTensor.from_host(x)
    Q = HipTensor.empty([rows, cols], np.int8)
    S = HipTensor.empty([rows], np.float32)
    D = HipTensor.empty([rows, cols], np.float32)
    algo_bytes = rows * cols * 5.0 + rows * 4.0     # 4 B in + 1 B out (or 1 + 4) per element + scales
    out = {}

    def q_step():
        capi.call("vtl_hip_quantize_f32_i8", X.ptr, rows, cols, 1, Q.ptr, S.ptr)

    def d_step():
        capi.call("vtl_hip_dequantize_i8_f32", Q.ptr, S.ptr, rows, cols, 1, D.ptr)

    for name, fn, kern in (("quantize", q_step, "quantize_rows_reg_kernel<1024,4,true>"),
                           ("dequantize", d_step, "dequantize_kernel<512,2,4>")):
        for _ in range(warmup):
            fn()
        wall, dev_ms = timer.run(fn, steps)
        kernel_ms = dev_ms / steps
        per_launch = timer.each(fn, steps)
        gbps = algo_bytes / (kernel_ms * 1e-3) / 1e9
        out[name] = {
            "value": algo_bytes / (wall / steps) / 1e9, "unit": "GB/s", "ms_per_step": wall * 1e3 / steps,
            "per_launch": per_launch,
            "config": {"workload": f"configs[1]: per-row {name} of f32 [16384,16384], seed 1"},
            "roofline": {"kernel": kern, "bound": "hbm", "achieved": gbps, "peak": PEAK_HBM_GBPS,
                         "unit": "GB/s", "frac": gbps / PEAK_HBM_GBPS, "kernel_us": kernel_ms * 1e3,
                         "algorithmic_bytes": algo_bytes, "traffic": measured_traffic(name)},
        }
    if cpu:
        import oracle  # CPU baseline leg only
        oracle.use_native_build()
        sample = rows   # the whole tensor once: under a second per pass on one host core
        threads = oracle.max_threads()
        t0 = time.perf_counter()
        qr, sr = oracle.quantize(x[:sample], True, threads=1)
        dq1 = time.perf_counter() - t0
        t0 = time.perf_counter()
        dr = oracle.dequantize(qr, sr, True, threads=1)
        dd1 = time.perf_counter() - t0
        big = rows
        t0 = time.perf_counter()
        oracle.quantize(x[:big], True, threads=threads)
        dqn = time.perf_counter() - t0
        t0 = time.perf_counter()
        oracle.dequantize(qr, sr, True, threads=threads)
        ddn = time.perf_counter() - t0
        sample_bytes = sample * cols * 5.0 + sample * 4.0
        out["quantize"]["cpu_baseline"] = {"value": sample_bytes / dq1 / 1e9, "unit": "GB/s", "cores": 1,
                                           "kind": "port", "sample": f"first {sample} rows, {dq1:.2f} s"}
        out["quantize"]["cpu_baseline_all_cores"] = {
            "value": (big * cols * 5.0 + big * 4.0) / dqn / 1e9, "unit": "GB/s", "cores": threads,
            "kind": "port", "sample": f"first {big} rows, {dqn:.2f} s, OpenMP"}
        out["dequantize"]["cpu_baseline"] = {"value": sample_bytes / dd1 / 1e9, "unit": "GB/s", "cores": 1,
                                             "kind": "port", "sample": f"first {sample} rows, {dd1:.2f} s"}
        out["dequantize"]["cpu_baseline_all_cores"] = {
            "value": sample_bytes / ddn / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"first {sample} rows, {ddn:.2f} s, OpenMP"}
        out["quantize"]["parity_sample_bit_exact"] = bool(
            np.array_equal(Q.cpu()[:sample], qr) and np.array_equal(S.cpu()[:sample], sr))
        out["dequantize"]["parity_sample_bit_exact"] = bool(np.array_equal(D.cpu()[:sample], dr))
    for h in (X, Q, S, D):
        h.release()
    return out


def bench_other_configs(timer: Timer, steps: int, warmup: int, cpu: bool = False, parts=("mnist", "decode", "chain"),
                        decode_cached: bool = True, exact: bool = False):
    """Timings of the remaining configurations (parity for them is in tests/):
    configs[0] MNIST-MLP first layer, configs[3] decode-shaped linear with
    per-token quantization on the fly, configs[4] 3-layer int8 MLP chain."""
    from vtl_amd.storage import HipStorage
    # These are side figures, not `value`: launches of 4 to 60 us whose first few dozen after an idle
    # spell run 5-15 % slow while the card's clocks settle, so they are timed over at least 100
    # launches after at least 100 warm-up launches whatever --steps / --warmup say (the headline
    # and the quantize / dequantize legs use --steps / --warmup exactly).
    if not exact:
        warmup, steps = max(warmup, 100), max(steps, 100)
    out = {"note": f"every figure in here: {steps} timed launches after {warmup} warm-up launches "
                   "(at least 100 of each unless --other-exact; see bench.py)"}

    def timed(fn):
        for _ in range(warmup):
            fn()
        _, dev_ms = timer.run(fn, steps)
        return dev_ms / steps * 1e3   # microseconds

    if "mnist" not in parts:
        return _other_decode_chain(timer, timed, out, parts, decode_cached)
    # configs[0]: per-tensor quantize of x, int8 linear (weights quantized once, untimed)
    x, w, b = workloads.mnist_mlp_first_layer()
    X, W, B = HipTensor.from_host(x), HipTensor.from_host(w), HipTensor.from_host(b.reshape(-1))
    Wq, Sw = W.quantize_i8(-1)
    Xq, Sx = HipTensor.empty([64, 784], np.int8), HipTensor.empty([1], np.float32)
    Y = HipTensor.empty([64, 256], np.float32)

    def c1():
        capi.call("vtl_hip_quantize_f32_i8", X.ptr, 64, 784, 0, Xq.ptr, Sx.ptr)
        capi.call("vtl_hip_linear_i8_f32", Xq.ptr, Sx.ptr, 0, Wq.ptr, Sw.ptr, 0, B.ptr, Y.ptr, 64, 256, 784, 0)
    c0 = {"us": timed(c1), "ops": 2.0 * 64 * 784 * 256}
    if cpu:
        # The reference's own CPU-runnable case, timed on the host beside it: (i) the reference's
        # existing f32 Linear restated (operands widened to f64, f64 product, one rounding to
        # f32, bias added in f32: la/la.v:44-53, nn/layers/linear_forward_f32.v:16-18) and (ii) the
        # int8 path of this build on the CPU oracle (per-tensor quantize of x, int8 linear).
        import oracle  # CPU baseline leg only
        oracle.use_native_build()
        wq_h, sw_h = oracle.quantize(w, False)

        def best_of(fn, reps=20):
            ts = []
            for _ in range(reps):
                t0 = time.perf_counter()
                fn()
                ts.append(time.perf_counter() - t0)
            return float(np.median(ts)) * 1e6

        def int8_cpu():
            xq_h, sx_h = oracle.quantize(x, False)
            return oracle.linear_i8_f32(xq_h, sx_h, wq_h, sw_h, b.reshape(-1), threads=1)
        c0["cpu_f32_linear_via_f64_us"] = best_of(lambda: oracle.linear_f32_via_f64(x, w, b.reshape(-1)))
        c0["cpu_int8_path_us"] = best_of(int8_cpu)
        c0["cpu_note"] = "one host thread, median of 20; " + oracle.build_flags()
        c0["parity_bit_exact"] = bool(np.array_equal(Y.cpu(), int8_cpu()))
    out["configs[0] mnist first layer [64,784]x[256,784]^T"] = c0
    for h in (X, W, B, Wq, Sw, Xq, Sx, Y):
        h.release()

    return _other_decode_chain(timer, timed, out, parts, decode_cached)


def _other_decode_chain(timer: Timer, timed, out, parts, decode_cached: bool):
    if "decode" in parts:
        _bench_decode(timed, out, decode_cached)
    if "chain" in parts:
        _bench_chain(timed, out)
    return out


def _bench_decode(timed, out, decode_cached: bool):
    from vtl_amd.storage import HipStorage
    # configs[3]: K=4096, N=14336, M in {1,8,32,128}; the tensors of workloads.decode_linear
    # (seed 3), the ones the parity tests and the golden fixtures use
    k, n = 4096, 14336
    W = HipTensor.from_host(workloads.decode_linear(1, k, n)[1])
    Wq, Sw = W.quantize_i8(0)                      # one scale per output channel
    W.release()
    # The 58.7 MB of codes stay in the 256 MB last-level cache from one launch to the next.
    # A model's decode step walks through many such matrices, so the same call is also timed
    # over 12 copies taken in turn (705 MB): every launch then streams its weights from HBM.
    copies = [Wq] + [HipTensor.empty([n, k], np.int8) for _ in range(11)]
    for c in copies[1:]:
        capi.call("vtl_hip_memcpy_d2d", c.ptr, Wq.ptr, n * k)
    dec = {}
    for m in (1, 8, 32, 128):
        X = HipTensor.from_host(workloads.decode_linear_activations(m, k))
        Y = HipTensor.empty([m, n], np.float32)
        need = int(capi.lib().vtl_hip_linear_f32_dynquant_workspace(m, k))
        ws = HipStorage.empty(need, np.uint8)

        def c4():
            capi.call("vtl_hip_linear_f32_dynquant", X.ptr, Wq.ptr, Sw.ptr, None, Y.ptr, m, n, k, 0, ws.ptr, ws.size)
        us = timed(c4) if decode_cached else None
        turn = [0]

        def c4_streaming():
            w = copies[turn[0] % len(copies)]
            turn[0] += 1
            capi.call("vtl_hip_linear_f32_dynquant", X.ptr, w.ptr, Sw.ptr, None, Y.ptr, m, n, k, 0, ws.ptr, ws.size)
        us_hbm = timed(c4_streaming)
        algo = n * k + 16384.0 * m + 57344.0 * m + 57344.0     # Wq + X f32 + Y f32 + sw
        # the roofline fraction is the one with the weights streaming from HBM; the figure with
        # the 58.7 MB of weights resident in the last-level cache is kept beside it as a footnote
        dec[f"M={m}"] = {"us": us_hbm, "GB/s": algo / us_hbm / 1e3,
                         "roofline": {"bound": "hbm", "achieved": algo / us_hbm / 1e3, "peak": PEAK_HBM_GBPS,
                                      "unit": "GB/s", "frac": algo / us_hbm / 1e3 / PEAK_HBM_GBPS},
                         "TOPS": 2.0 * m * n * k / us_hbm / 1e6, "algorithmic_bytes": algo,
                         "weights_in_last_level_cache": None if us is None else {
                             "us": us, "GB/s": algo / us / 1e3, "note": "same weights every launch: not an HBM figure"}}
        capi.call("vtl_hip_sync")
        for h in (X, Y):
            h.release()
        ws.release()
    out["configs[3] decode linear K=4096 N=14336 (quantize on the fly + int8 linear)"] = dec
    for c in copies:
        c.release()
    Sw.release()



def _bench_chain(timed, out):
    # configs[4]: 256x4096 -> 11008 -> ReLU -> 4096 -> ReLU -> 1024, device-resident chain; the
    # tensors of workloads.mlp_chain (seed 4), the ones the parity tests and the golden fixtures use
    dims, m = (4096, 11008, 4096, 1024), 256
    x_host, ws_host = workloads.mlp_chain(m, dims)
    Ws, Ss = [], []
    for i in range(3):                             # Xavier-uniform f32 weights, one scale per output channel
        W = HipTensor.from_host(ws_host[i])
        wq, sw = W.quantize_i8(0)
        W.release()
        Ws.append(wq)
        Ss.append(sw)
    del ws_host
    X = HipTensor.from_host(x_host)
    # activations travel as per-token int8 codes + row scales: the first layer's input is
    # quantized, every hidden layer hands codes to the next (epilogue, ReLU and requantization
    # in one pass over the int32 sums), the last one writes f32
    Qs = [HipTensor.empty([m, dims[i]], np.int8) for i in range(3)]
    Sx = [HipTensor.empty([m], np.float32) for i in range(3)]
    Y = HipTensor.empty([m, dims[3]], np.float32)

    # The 94 MB of weights stay in the 256 MB last-level cache from one step to the next; a model
    # with many such blocks streams them from HBM, so the step is also timed over 6 copies of the
    # three matrices taken in turn (564 MB).
    sets = [Ws]
    for _ in range(5):
        cp = [HipTensor.empty([dims[i + 1], dims[i]], np.int8) for i in range(3)]
        for i in range(3):
            capi.call("vtl_hip_memcpy_d2d", cp[i].ptr, Ws[i].ptr, dims[i + 1] * dims[i])
        sets.append(cp)

    def layer(i, w=None):
        w = Ws[i] if w is None else w
        if i == 0:
            capi.call("vtl_hip_quantize_f32_i8", X.ptr, m, dims[0], 1, Qs[0].ptr, Sx[0].ptr)
        if i < 2:
            capi.call("vtl_hip_linear_i8_requant", Qs[i].ptr, Sx[i].ptr, 1, w.ptr, Ss[i].ptr, 1, None, 1,
                      Qs[i + 1].ptr, Sx[i + 1].ptr, None, m, dims[i + 1], dims[i])
        else:
            capi.call("vtl_hip_linear_i8_f32", Qs[i].ptr, Sx[i].ptr, 1, w.ptr, Ss[i].ptr, 1, None, Y.ptr,
                      m, dims[i + 1], dims[i], 0)

    def c5():
        for i in range(3):
            layer(i)
    us = timed(c5)
    turn = [0]

    def c5_streaming():
        ws = sets[turn[0] % len(sets)]
        turn[0] += 1
        for i in range(3):
            layer(i, ws[i])
    us_hbm = timed(c5_streaming)
    ops = 2.0 * m * sum(dims[i] * dims[i + 1] for i in range(3))
    wbytes = float(sum(dims[i] * dims[i + 1] for i in range(3)))
    layers = {}
    for i in range(3):
        lus = timed(lambda i=i: layer(i))
        layers[f"{dims[i]}->{dims[i + 1]}"] = {"us": lus, "TOPS": 2.0 * m * dims[i] * dims[i + 1] / lus / 1e6,
                                               "weight_GB/s": dims[i] * dims[i + 1] / lus / 1e3}
    out["configs[4] int8 MLP chain 256x4096->11008->4096->1024"] = {
        "us": us, "TOPS": ops / us / 1e6, "weight_GB/s": wbytes / us / 1e3, "ops": ops,
        "note": "same weights every step: the 94 MB stay in the last-level cache",
        "weights_from_hbm": {"us": us_hbm, "TOPS": ops / us_hbm / 1e6, "weight_GB/s": wbytes / us_hbm / 1e3,
                             "note": "6 copies of the three matrices in turn (564 MB)"},
        "per_layer (input quantize + linear/ReLU/requantize, same, linear to f32)": layers}
    # The same three layers with a few tokens: the layers hand f32 rows on and each quantizes its
    # input inside its own launch (what Sequential.forward and mlp_forward_i8 do up to 32 rows).
    few = {}
    for mt in (1, 8, 32):
        Xs = HipTensor.from_host(x_host[:mt])
        Hs = [HipTensor.empty([mt, dims[i + 1]], np.float32) for i in range(3)]
        need = int(capi.lib().vtl_hip_linear_f32_dynquant_workspace(mt, max(dims[:3])))
        Wk = HipTensor.empty([need], np.uint8)

        def few_chain(ws_=None, mt=mt, Xs=Xs, Hs=Hs, Wk=Wk):
            ws_ = Ws if ws_ is None else ws_
            src = Xs
            for i in range(3):
                capi.call("vtl_hip_linear_f32_dynquant", src.ptr, ws_[i].ptr, Ss[i].ptr, None, Hs[i].ptr, mt,
                          dims[i + 1], dims[i], 1 if i < 2 else 0, Wk.ptr, Wk.size)
                src = Hs[i]

        def few_streaming(few_chain=few_chain):
            few_chain(sets[turn[0] % len(sets)])
            turn[0] += 1
        few[f"M={mt}"] = {"us": timed(few_chain), "weights_from_hbm_us": timed(few_streaming)}
        capi.call("vtl_hip_sync")
        for h in [Xs, Wk] + Hs:
            h.release()
    out["configs[4] int8 MLP chain 256x4096->11008->4096->1024"]["few_tokens (f32 rows from layer to layer, one launch a layer)"] = few
    capi.call("vtl_hip_sync")
    for h in Ss + Qs + Sx + [X, Y] + [w for st in sets for w in st]:
        h.release()
    return out


def bench_full_precision(timer: Timer, steps: int, warmup: int):
    """The f32 matmul with f64 accumulation behind la.matmul / Linear backward
    (parity in tests/): the unquantized Linear forward at M=N=K=4096 against the
    f64 matrix-core peak, and LinearGate.backward of the first MLP layer."""
    out = {}
    steps = max(3, min(steps, 10))
    warmup = max(1, min(warmup, 2))
    rng = np.random.Generator(np.random.Philox(5))

    def timed(fn):
        for _ in range(warmup):
            fn()
        _, dev_ms = timer.run(fn, steps)
        return dev_ms / steps * 1e3   # microseconds

    m = n = k = 4096
    X = HipTensor.from_host(rng.standard_normal((m, k), dtype=np.float32))
    W = HipTensor.from_host(rng.standard_normal((n, k), dtype=np.float32))
    B = HipTensor.from_host(rng.standard_normal(n, dtype=np.float32))
    Y = HipTensor.empty([m, n], np.float32)
    us = timed(lambda: capi.call("vtl_hip_linear_f32", X.ptr, W.ptr, B.ptr, Y.ptr, m, n, k, 0))
    tf = 2.0 * m * n * k / us / 1e6
    out["linear_f32 (f64 accumulate) M=N=K=4096"] = {
        "us": us, "TFLOP/s": tf,
        "roofline": {"bound": "mfma", "achieved": tf, "peak": PEAK_FP64_TFLOPS, "unit": "TFLOP/s",
                     "frac": tf / PEAK_FP64_TFLOPS, "traffic": measured_traffic("linear_f32"),
                     "kernel": "matmul_f64acc_kernel<float, 2, 4, 4, 2, false, true, false, false>"}}
    for h in (X, W, B, Y):
        h.release()

    m, n, k = 256, 11008, 4096
    G = HipTensor.from_host(rng.standard_normal((m, n), dtype=np.float32))
    X = HipTensor.from_host(rng.standard_normal((m, k), dtype=np.float32))
    W = HipTensor.from_host(rng.standard_normal((n, k), dtype=np.float32))
    dX, dW, dB = HipTensor.empty([m, k], np.float32), HipTensor.empty([n, k], np.float32), HipTensor.empty([n], np.float32)
    us = timed(lambda: capi.call("vtl_hip_linear_backward_f32", G.ptr, X.ptr, W.ptr, dX.ptr, dW.ptr, dB.ptr, m, n, k))
    out["linear_backward_f32 grad[256,11008] x[256,4096] W[11008,4096] (dx, dw, db)"] = {
        "us": us, "TFLOP/s": 4.0 * m * n * k / us / 1e6, "frac_of_fp64_mfma_peak": 4.0 * m * n * k / us / 1e6 / PEAK_FP64_TFLOPS}
    capi.call("vtl_hip_sync")
    for h in (G, X, W, dX, dW, dB):
        h.release()
    return out


def bench_copy_calibration(timer: Timer, steps: int, warmup: int):
    """Plain device-to-device copy of 1 GiB with the library's copy kernel: the
    kernel of known traffic (1 GiB read + 1 GiB written per launch) that the
    FETCH_SIZE / WRITE_SIZE hardware counters are scaled against."""
    nbytes = 1 << 30
    src = HipTensor.empty([nbytes // 4], np.float32)
    dst = HipTensor.empty([nbytes // 4], np.float32)
    capi.call("vtl_hip_memset", src.ptr, 1, nbytes)

    def step():
        capi.call("vtl_hip_memcpy_d2d", dst.ptr, src.ptr, nbytes)

    for _ in range(warmup):
        step()
    wall, dev_ms = timer.run(step, steps)
    gbps = 2.0 * nbytes / (dev_ms / steps * 1e-3) / 1e9
    for h in (src, dst):
        h.release()
    return {"kernel": "copy_kernel", "bytes_read": nbytes, "bytes_written": nbytes,
            "kernel_us": dev_ms / steps * 1e3, "GB/s": gbps}


def bench_mfma_only(timer: Timer, load_s: float = 2.3):
    """What the matrix cores alone sustain: probe kernels (a small library of its own, built
    beside the product library and loaded only here) run nothing but the int8 MFMA of the
    matmul kernels, on constant operands and on uniformly random ones (the operand
    distribution of configs[2]), each for about load_s seconds while shader clock and socket
    power are sampled.  Two loops: `fixed` re-uses 4 + 4 operand registers, `rotating` walks
    through 32 + 32 register-resident fragments so that every instruction sees fresh operands,
    like a matmul kernel's k-steps.  The random-operand figure is the ceiling that the power
    limit leaves to any int8 kernel on such data; the Linear's fraction of it is reported
    next to its fraction of the nominal peak."""
    from vtl_amd import build as vb
    if not os.path.exists(vb.BENCH_PROBE_PATH):
        vb.build_lib()
    lib = C.CDLL(vb.BENCH_PROBE_PATH)
    stream = C.c_void_p()
    capi.call("vtl_hip_get_stream", C.byref(stream))
    rng = np.random.Generator(np.random.Philox(2))
    sink = HipTensor.empty([4], np.int32)
    out = {}
    nbytes = 256 * 1024
    hosts = (("constant_operands", np.full(nbytes, 1, np.int8)),
             ("uniform_random_operands", rng.integers(-127, 128, nbytes, dtype=np.int8)))
    for loop, sym, per_iter, iters in (("fixed", "vtl_bench_probe_mfma_i8", 16, 4000),
                                       ("rotating", "vtl_bench_probe_mfma_i8_rotating", 64, 1000)):
        probe = getattr(lib, sym)
        probe.restype, probe.argtypes = C.c_int, [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        ops = 1024.0 * 4 * per_iter * iters * 65536.0
        for label, host in hosts:
            buf = HipTensor.from_host(host)

            def step():
                if probe(buf.ptr, iters, sink.ptr, stream) != 0:
                    raise RuntimeError(sym + " failed")
            for _ in range(4):
                step()
            _, dev_ms = timer.run(step, 8)
            n = max(8, int(load_s / (dev_ms / 8 * 1e-3)))
            sampler = PowerClockSampler()
            with sampler:
                _, dev_ms = timer.run(step, n)
            rec = {"TOP/s": ops / (dev_ms / n * 1e-3) / 1e12, "us_per_launch": dev_ms / n * 1e3,
                   "under_load": sampler.summary()}
            if loop == "fixed":
                out[label] = rec
            else:
                out.setdefault("rotating_operand_registers", {})[label] = rec
            buf.release()
    sink.release()
    return out


def _vendor_yardstick_child(steps: int, warmup: int) -> int:
    """Body of the child process behind bench_vendor_yardstick(): prints one JSON object."""
    try:
        import torch
        if not torch.cuda.is_available():
            print(json.dumps({"error": "torch sees no GPU"}))
            return 0
        a, bt, _, _, _ = workloads.square_int8_gemm()
        A = torch.from_numpy(a).cuda()
        Bt = torch.from_numpy(bt).cuda()
        B = Bt.t()                                   # K x N view of the weights as stored [N,K]
        for _ in range(warmup):
            c = torch._int_mm(A, B)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            c = torch._int_mm(A, B)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / steps * 1e3
        want = a[:8].astype(np.int64) @ bt.astype(np.int64).T
        ok = bool(np.array_equal(c[:8].cpu().numpy().astype(np.int64), want))
        print(json.dumps({
            "what": "torch._int_mm(A, Wq^T) -> int32 (PyTorch-ROCm hands it to hipBLASLt), the operands of "
                    "configs[2], int32 sums out (the same 64 MiB as the Linear's f32 result), no scale/bias epilogue; "
                    "a yard-stick, not part of the product and never `value`",
            "us": us, "TOP/s": 2.0 * 4096 ** 3 / us / 1e6, "frac_of_peak": 2.0 * 4096 ** 3 / us / 1e6 / PEAK_INT8_TOPS,
            "steps": steps, "warmup": warmup, "sums_match_numpy_on_8_rows": ok, "torch": torch.__version__}))
    except Exception as e:                            # noqa: BLE001 - a yard-stick must never fail the bench
        print(json.dumps({"error": repr(e)[:200]}))
    return 0


def bench_vendor_yardstick(steps: int, warmup: int):
    """The vendor library's int8 matmul on the same operands, timed in a child process (PyTorch
    brings its own HIP runtime, which is kept out of the process that loads libvtlhip.so).
    None when the child gives no answer."""
    import subprocess
    try:
        res = subprocess.run([sys.executable, os.path.abspath(__file__), "--vendor-yardstick-child",
                              "--steps", str(steps), "--warmup", str(warmup)],
                             stdout=subprocess.PIPE, stderr=subprocess.DEVNULL, text=True, timeout=240)
        lines = [l for l in res.stdout.splitlines() if l.startswith("{")]
        return json.loads(lines[-1]) if lines else None
    except Exception as e:                            # noqa: BLE001
        return {"error": repr(e)[:200]}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the shader clock settles over the first tens of milliseconds of load: the
    # defaults warm up for about that long and time a few hundred launches
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only", choices=["all", "linear", "quant", "copy", "full", "other", "mfma", "decode", "chain"],
                    default="all")
    ap.add_argument("--linear-operands", choices=["config", "zeros"], default="config",
                    help="zeros: time the Linear on all-zero int8 operands (a diagnostic, says so in the line)")
    ap.add_argument("--load-seconds", type=float, default=3.2,
                    help="length of the back-to-back loops during which clock and power are sampled (0: none)")
    ap.add_argument("--no-probe", action="store_true", help="skip the MFMA-only probe loops (profiling runs)")
    ap.add_argument("--vendor-yardstick-child", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--no-vendor-yardstick", action="store_true",
                    help="skip the torch._int_mm timing printed beside the Linear")
    ap.add_argument("--other-exact", action="store_true",
                    help="time the side figures over exactly --steps / --warmup launches (short profiling runs)")
    ap.add_argument("--decode-from-hbm-only", action="store_true",
                    help="with --only decode: skip the launches that re-read the same weights (profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 "
              "(sharding across GPUs is a design note only; nothing multi-GPU is built)", file=sys.stderr)
        return 2
    if args.vendor_yardstick_child:
        return _vendor_yardstick_child(args.steps, args.warmup)
    if capi.device_count() < 1:
        print("bench.py: no HIP device visible", file=sys.stderr)
        return 1
    capi.call("vtl_hip_set_device", 0)
    name, cus, mhz = capi.device_info()
    timer = Timer()
    cpu = not args.no_cpu_baseline
    if args.only == "copy":
        print(json.dumps({"calibration": bench_copy_calibration(timer, args.steps, args.warmup)}))
        return 0
    if args.only == "full":
        print(json.dumps({"full_precision": bench_full_precision(timer, args.steps, args.warmup)}))
        return 0
    if args.only == "other":
        print(json.dumps({"other_configs": bench_other_configs(timer, args.steps, args.warmup, cpu,
                                                               exact=args.other_exact)}))
        return 0
    if args.only in ("decode", "chain"):
        print(json.dumps({"other_configs": bench_other_configs(timer, args.steps, args.warmup, False, (args.only,),
                                                               not args.decode_from_hbm_only, args.other_exact)}))
        return 0
    if args.only == "mfma":
        print(json.dumps({"mfma_only": bench_mfma_only(timer, max(args.load_seconds, 0.05))}))
        return 0

    lin = bench_linear(timer, args.steps, args.warmup, cpu, args.load_seconds, args.linear_operands) if args.only in ("all", "linear") else None
    qd = bench_quant(timer, args.steps, args.warmup, cpu) if args.only in ("all", "quant") else None

    line = {
        "metric": METRIC,
        "value": lin["tops"] if lin else qd["quantize"]["value"],
        "unit": "TOPS" if lin else "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": lin["ms_per_step"] if lin else qd["quantize"]["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8 (i32 accumulate, f32 epilogue)", "data": "synthetic",
        "config": {"workload": ("configs[2]: int8 Linear M=N=K=4096, per-row x per-column f32 scales + bias, "
                                "seed 2; secondary: configs[1] per-row quantize/dequantize of f32 "
                                "[16384,16384], seed 1") if lin else qd["quantize"]["config"]["workload"],
                   "device": name, "compute_units": cus, "clock_mhz": mhz},
    }
    if lin and args.linear_operands != "config":
        line["diagnostic"] = "all-zero int8 operands, NOT the configs[2] workload"
    if lin:
        line["roofline"] = lin["roofline"]
        line["per_launch"] = lin["per_launch"]
        if "cpu_baseline" in lin:
            line["cpu_baseline"] = lin["cpu_baseline"]
            line["cpu_baseline_all_cores"] = lin["cpu_baseline_all_cores"]
            line["parity_sample_bit_exact"] = lin["parity_sample_bit_exact"]
    elif qd:
        line["roofline"] = qd["quantize"]["roofline"]
        if "cpu_baseline" in qd["quantize"]:
            line["cpu_baseline"] = qd["quantize"]["cpu_baseline"]
    if qd:
        line["quantize"] = qd["quantize"]
        line["dequantize"] = qd["dequantize"]
    if lin:
        ul = lin.get("under_load") or {}
        line["roofline"]["sclk_mhz_under_load"] = ul.get("sclk_mhz_mean")
        line["roofline"]["power_w"] = ul.get("power_w_mean")
        line["under_load"] = ul
        if not args.no_probe:
            line["mfma_only"] = bench_mfma_only(timer, max(args.load_seconds * 0.72, 0.05))
            ceiling = max(line["mfma_only"]["uniform_random_operands"]["TOP/s"],
                          line["mfma_only"]["rotating_operand_registers"]["uniform_random_operands"]["TOP/s"])
            line["roofline"]["frac_of_mfma_only_rate_on_these_operands"] = line["roofline"]["achieved"] / ceiling
        if not args.no_vendor_yardstick:
            line["vendor_int8_mm"] = bench_vendor_yardstick(args.steps, args.warmup)
    if args.only == "all":
        line["other_configs"] = bench_other_configs(timer, args.steps, args.warmup, cpu, exact=args.other_exact)
        line["full_precision"] = bench_full_precision(timer, args.steps, args.warmup)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
