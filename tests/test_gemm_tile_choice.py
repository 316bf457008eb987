"""The int8 tile kernels' cost model against recorded timings (no GPU needed).

tests/golden/gemm_tile_sweep.json holds, for the tile-kernel launches of the benchmark
configurations and a few other shapes, the measured time of every tile configuration and
K-split count, with the weights re-read from the last-level cache and streamed from HBM
(made on an MI355X by tests/golden/make_gemm_tile_sweep.py).  The library's choice
(vtl_hip_gemm_tile_choice, pure host arithmetic) must be the fastest entry or within 5 % of
it in both regimes: a refit of the model's constants that loses one of these shapes fails here.
"""
import ctypes as C
import json
import os

import pytest

from vtl_amd import capi

HERE = os.path.dirname(os.path.abspath(__file__))
SWEEP = json.load(open(os.path.join(HERE, "golden", "gemm_tile_sweep.json")))


def _choice(m, n, k, requant=False):
    idx, tm, tn, splits = C.c_int(), C.c_int(), C.c_int(), C.c_int()
    capi.call("vtl_hip_gemm_tile_choice", m, n, k, int(requant), C.byref(idx), C.byref(tm), C.byref(tn),
              C.byref(splits))
    return idx.value, tm.value, tn.value, splits.value


@pytest.mark.parametrize("rec", SWEEP["shapes"], ids=lambda r: f"{r['m']}x{r['n']}x{r['k']}")
def test_choice_is_within_five_percent_of_the_fastest_measured(rec):
    idx, tm, tn, splits = _choice(rec["m"], rec["n"], rec["k"], rec["entry"] == "requant")
    key = f"{idx},{splits}"
    for regime in ("cached", "from_hbm"):
        times = rec[regime]
        assert key in times, f"the model's choice {key} was not even worth timing for this shape"
        best = min(times, key=times.get)
        assert times[key] <= 1.05 * times[best], (regime, key, times[key], best, times[best])


def test_choice_reports_tile_shapes_and_rejects_bad_arguments():
    idx, tm, tn, splits = _choice(4096, 4096, 4096)
    assert (idx, tm, tn, splits) == (7, 256, 256, 1)           # the headline launch: one round of 256x256 tiles
    idx, tm, tn, splits = _choice(256, 4096, 11008, requant=True)
    assert (tm, tn) == (128, 64) and splits == 2               # few tiles, long K: K is cut
    one = C.c_int()
    assert capi.status("vtl_hip_gemm_tile_choice", 0, 4, 4, 0, C.byref(one), C.byref(one), C.byref(one),
                       C.byref(one)) == capi.ERR_INVALID_ARG
    assert capi.status("vtl_hip_gemm_tile_choice", 4, 4, 4, 0, None, C.byref(one), C.byref(one),
                       C.byref(one)) == capi.ERR_INVALID_ARG
