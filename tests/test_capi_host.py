"""CPU-only checks of the C-ABI library and the host-side mirror: the library
loads, exports every symbol include/vtl_hip.h declares, rejects bad arguments
with a status instead of aborting, and the host logic (shape rules, flags,
strides) behaves like the reference's.  No compute call reaches a device here.
"""
import ctypes as C
import os
import re

import numpy as np
import pytest

from vtl_amd import capi, layers, workloads
from vtl_amd.storage import HipStorage
from vtl_amd.tensor import HipTensor, _matmul_shapes, _per_row, _strides_from_shape

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "vtl_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vtl_hip_\w+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    L = capi.lib()
    declared = _declared_symbols()
    assert len(declared) >= 25
    for name in declared:
        assert hasattr(L, name), f"{name} declared in vtl_hip.h but not exported"
    # and the ctypes table covers exactly the header
    assert sorted(capi.SIGNATURES) == declared


def test_status_strings():
    L = capi.lib()
    assert L.vtl_hip_strerror(0) == b"success"
    for st in range(1, 6):
        assert L.vtl_hip_strerror(st) not in (b"", b"unknown status")
    assert L.vtl_hip_strerror(99) == b"unknown status"
    assert b"gfx950" in L.vtl_hip_version()


def test_bad_arguments_return_status_not_abort():
    """Null/negative arguments are rejected before any device work
    (cf. the null-pointer check at storage/cuda_d_cuda.v:69-71)."""
    S, E = capi.status, capi.ERR_INVALID_ARG
    one = C.c_void_p(16)  # never dereferenced: argument checks come first
    assert S("vtl_hip_device_count", None) == E
    assert S("vtl_hip_malloc", None, 16) == E
    p = C.c_void_p()
    assert S("vtl_hip_malloc", C.byref(p), 0) == E
    assert S("vtl_hip_free", None) == capi.OK
    assert S("vtl_hip_memcpy_h2d", None, one, 4) == E
    assert S("vtl_hip_memcpy_d2h", one, None, 4) == E
    assert S("vtl_hip_memcpy_d2h", None, None, 0) == capi.OK
    assert S("vtl_hip_absmax_f32", None, 1, 1, 1, one) == E
    assert S("vtl_hip_absmax_f32", one, -1, 1, 1, one) == E
    assert S("vtl_hip_quantize_f32_i8", one, 4, 4, 1, one, None) == E
    assert S("vtl_hip_quantize_f32_i8", one, 4, -4, 1, one, one) == E
    assert S("vtl_hip_quantize_with_scale_f32_i8", one, None, 4, 4, 1, one) == E
    assert S("vtl_hip_dequantize_i8_f32", one, None, 4, 4, 1, one) == E
    assert S("vtl_hip_dequantize_i8_f32", None, one, 4, 4, 1, one) == E
    assert S("vtl_hip_gemm_i8_i32", None, one, one, 4, 4, 16) == E
    assert S("vtl_hip_gemm_i8_i32", one, one, one, -4, 4, 16) == E
    assert S("vtl_hip_gemm_i8_i32", one, one, one, 4, 4, 1 << 20) == capi.ERR_UNSUPPORTED
    assert S("vtl_hip_linear_i8_f32", one, None, 1, one, one, 1, None, one, 4, 4, 16, 0) == E
    assert S("vtl_hip_linear_i8_requant", one, one, 1, one, one, 1, None, 0, one, None, None, 4, 4, 16) == E   # no scales out
    assert S("vtl_hip_linear_i8_requant", one, one, 1, one, one, 1, None, 0, None, one, None, 4, 4, 16) == E   # no codes out
    assert S("vtl_hip_linear_i8_requant", one, one, 1, one, one, 1, None, 0, one, one, None, 0, 4, 16) == capi.OK
    assert S("vtl_hip_linear_f32_dynquant", one, one, one, None, one, 4, 4, 16, 0, C.c_void_p(20), 4096) == E   # misaligned
    assert S("vtl_hip_linear_f32_dynquant", one, one, one, None, one, 4, 4, 16, 0, one, 8) == E
    assert S("vtl_hip_relu_f32", None, 4) == E
    assert S("vtl_hip_event_record", None) == E
    # empty problems succeed without touching the device
    assert S("vtl_hip_gemm_i8_i32", one, one, one, 0, 4, 16) == capi.OK
    assert S("vtl_hip_dequantize_i8_f32", one, one, 0, 4, 1, one) == capi.OK
    assert S("vtl_hip_relu_f32", one, 0) == capi.OK


def test_dynquant_workspace_size():
    f = capi.lib().vtl_hip_linear_f32_dynquant_workspace
    assert f(0, 16) == 0 and f(4, 0) == 0
    assert f(1, 4096) == 4096 + 256
    assert f(3, 100) == 512 + 256          # codes and scales each rounded up to 256 bytes
    assert f(256, 11008) == 256 * 11008 + 1024


def test_stream_get_set_roundtrip():
    p = C.c_void_p(123)
    capi.call("vtl_hip_get_stream", C.byref(p))
    assert p.value is None                  # the null stream by default
    assert capi.status("vtl_hip_get_stream", None) == capi.ERR_INVALID_ARG


def test_error_type_carries_status():
    with pytest.raises(capi.VtlHipError) as ei:
        capi.call("vtl_hip_relu_f32", None, 4)
    assert ei.value.status == capi.ERR_INVALID_ARG and "vtl_hip_relu_f32" in str(ei.value)


# ---- host-side mirror ---------------------------------------------------------------

def test_strides_and_axis_rules():
    assert _strides_from_shape([3, 4]) == [4, 1]          # util.v:169-184
    assert _strides_from_shape([2, 3, 4]) == [12, 4, 1]
    assert _strides_from_shape([5]) == [1]
    assert _per_row(-1) == 0 and _per_row(0) == 1
    with pytest.raises(ValueError):
        _per_row(1)


def _fake(shape, dtype):
    count = int(np.prod(shape))
    return HipTensor(HipStorage(0, count * np.dtype(dtype).itemsize, count, dtype), shape)


def test_predicates_and_matmul_shape_rule():
    a = _fake([4, 16], np.int8)
    w = _fake([7, 16], np.int8)
    assert a.is_matrix() and not a.is_vector() and not a.is_square_matrix()
    assert a.rank() == 2 and a.numel() == 64 and a.is_row_major() and not a.is_col_major()
    assert _fake([5, 5], np.float32).is_square_matrix() and _fake([5], np.float32).is_vector()
    assert a.is_row_major_contiguous() and a.is_contiguous() and not a.is_col_major_contiguous()
    t3 = _fake([2, 3, 4], np.float32)
    assert t3.strides == [12, 4, 1] and t3.is_contiguous()
    t3.strides = [12, 8, 1]                 # a strided view is not contiguous
    assert not t3.is_row_major_contiguous() and not t3.is_contiguous()
    assert _matmul_shapes(a, w) == (4, 7, 16)
    with pytest.raises(ValueError, match="Invalid shapes for matrix multiplication"):   # la/la.v:41-43
        _matmul_shapes(a, _fake([7, 32], np.int8))
    with pytest.raises(ValueError, match="Matrix expected"):
        _matmul_shapes(a, _fake([16], np.int8))
    with pytest.raises(ValueError):
        HipTensor(HipStorage(0, 4, 4, np.int8), [2, 3])
    with pytest.raises(TypeError):
        a.quantize_i8(0)                     # int8 input where f32 is expected
    with pytest.raises(TypeError):
        _fake([4, 16], np.float32).dequantize(_fake([4], np.float32), 0)


def test_env_flags(monkeypatch):
    monkeypatch.delenv("VTL_USE_HIP", raising=False)
    monkeypatch.delenv("VTL_TEST_HIP", raising=False)
    assert not layers.hip_linear_enabled() and not layers.linear_forward_f32_use_hip()
    assert not layers.hip_tests_enabled()
    with pytest.raises(RuntimeError, match="VTL_USE_HIP=1"):
        layers.linear_forward_hip_f32(np.zeros((1, 16), np.float32), np.zeros((2, 16), np.float32), None)
    monkeypatch.setenv("VTL_USE_HIP", "1")
    monkeypatch.setenv("VTL_TEST_HIP", "1")
    assert layers.hip_linear_enabled() and layers.linear_forward_f32_use_hip() and layers.hip_tests_enabled()
    monkeypatch.setenv("VTL_USE_HIP", "true")
    assert not layers.hip_linear_enabled()   # only the literal "1" opts in (vulkan_config.v:18-20)


def test_layer_shapes_without_device():
    """nn/layers/layers_test.v:16-36 checks shapes and variable counts only."""
    rng = np.random.default_rng(0)
    layer = layers.QuantLinearLayer(layers.kaiming_normal([3, 4], rng))
    assert layer.output_shape() == [3]
    w, b = layer.variables()
    assert w.shape == (3, 4) and b.shape == (1, 3) and not b.any()
    with pytest.raises(ValueError, match="Matrix expected"):
        layers.QuantLinearLayer(np.zeros(4, np.float32))
    with pytest.raises(ValueError, match="Matrix expected"):
        layer.forward(np.zeros(4, np.float32))


def test_workload_generators_are_seeded_and_shaped():
    x, w, b = workloads.mnist_mlp_first_layer()
    assert x.shape == (64, 784) and w.shape == (256, 784) and b.shape == (1, 256)
    assert x.min() >= 0 and x.max() < 1 and not b.any()
    limit = np.sqrt(3.0) * np.sqrt(2.0 / (256 * 784))
    assert np.abs(w).max() <= limit * (1 + 1e-6)
    x2, _, _ = workloads.mnist_mlp_first_layer()
    assert np.array_equal(x, x2)
    m = workloads.outlier_matrix(64, 4096)
    assert m.shape == (64, 4096) and m.dtype == np.float32
    assert np.array_equal(m, workloads.outlier_matrix(64, 4096))
    assert 0.9 < m.std() < 1.3 and np.abs(m).max() > 8      # outliers present
    a, bt, sa, sb, bias = workloads.square_int8_gemm(64, 32, 128)
    assert a.shape == (64, 128) and bt.shape == (32, 128) and a.min() >= -127
    assert sa.shape == (64,) and sb.shape == (32,) and bias.shape == (32,)
    x, w = workloads.decode_linear(8, 256, 512)
    assert x.shape == (8, 256) and w.shape == (512, 256) and abs(w.std() - 0.02) < 0.002
    x, ws = workloads.mlp_chain(4, (64, 128, 32))
    assert x.shape == (4, 64) and [t.shape for t in ws] == [(128, 64), (32, 128)]
    assert np.abs(ws[0]).max() <= np.sqrt(6.0 / (64 + 128))


def _header_arg_counts():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    out = {}
    for name, args in re.findall(r"\b(vtl_hip_\w+)\s*\(([^)]*)\)\s*;", text):
        args = args.strip()
        out[name] = 0 if args in ("", "void") else len(args.split(","))
    return out


def test_v_binding_declarations_match_the_header():
    """Every `fn C.vtl_hip_*` the V binding files declare exists in the header with the
    same number of arguments, and the ctypes table agrees on the count too."""
    counts = _header_arg_counts()
    assert set(counts) == set(capi.SIGNATURES)
    for name, (_, argtypes) in capi.SIGNATURES.items():
        assert len(argtypes) == counts[name], name
    vbind = os.path.join(ROOT, "vtl_amd", "vbind")
    seen = set()
    for dirpath, _, files in os.walk(vbind):
        for f in files:
            if not f.endswith(".v"):
                continue
            text = open(os.path.join(dirpath, f)).read()
            for name, args in re.findall(r"fn C\.(vtl_hip_\w+)\(([^)]*)\)", text):
                n = 0 if not args.strip() else len(args.split(","))
                assert name in counts, f"{f}: {name} is not in vtl_hip.h"
                assert n == counts[name], f"{f}: {name} takes {counts[name]} arguments, declared with {n}"
                seen.add(name)
    # the binding uses the compute surface of the library
    for must in ("vtl_hip_quantize_f32_i8", "vtl_hip_dequantize_i8_f32", "vtl_hip_gemm_i8_i32", "vtl_hip_linear_i8_f32",
                 "vtl_hip_linear_i8_requant", "vtl_hip_linear_f32_dynquant", "vtl_hip_matmul_f32", "vtl_hip_linear_backward_f32",
                 "vtl_hip_malloc", "vtl_hip_free", "vtl_hip_memcpy_h2d", "vtl_hip_memcpy_d2h"):
        assert must in seen, must


def _v_files():
    vbind = os.path.join(ROOT, "vtl_amd", "vbind")
    for dirpath, _, files in os.walk(vbind):
        for f in sorted(files):
            if f.endswith(".v"):
                yield os.path.join(dirpath, f)


def _strip_v_comments_and_strings(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r"'(?:\\.|[^'\\\n])*'", "''", text)
    text = re.sub(r'"(?:\\.|[^"\\\n])*"', '""', text)
    return re.sub(r"`(?:\\.|[^`\\\n])`", "``", text)


def _pub_fns(text):
    """name (with receiver type) -> normalised parameter list and return type of every `pub fn`."""
    out = {}
    code = _strip_v_comments_and_strings(text)
    for recv, name, params, ret in re.findall(
            r"^pub fn\s*(\([^)]*\)\s*)?(\w+)(?:\[[^\]]*\])?\(([^)]*)\)\s*([^{\n]*)\{", code, flags=re.M):
        recv_type = re.sub(r"^\(\s*(?:mut\s+)?\w+\s+", "", recv.strip()).rstrip(") ").strip() if recv else ""
        types = [re.sub(r"^(?:mut\s+)?\w+\s+", "", p.strip()) for p in params.split(",") if p.strip()]
        out[(recv_type, name)] = (tuple(types), ret.strip())
    return out


def test_v_binding_files_are_balanced_and_flag_pairs_define_the_same_public_functions():
    """No V compiler exists in this image, so the binding files get the checks that need none:
    every file starts with its module line and has balanced brackets outside comments and
    strings, and a `_d_hip.v` / `_notd_hip.v` pair - of which the V build compiles exactly one,
    depending on `-d hip` - defines the same public functions with the same parameter and
    return types (cf. storage/cuda_d_cuda.v against storage/cuda_notd_cuda.v)."""
    files = list(_v_files())
    assert len(files) >= 20
    for path in files:
        text = open(path).read()
        first = [l for l in text.splitlines() if l.strip() and not l.strip().startswith("//")][0]
        assert first.startswith("module "), path
        code = _strip_v_comments_and_strings(text)
        for a, b in ("()", "{}", "[]"):
            assert code.count(a) == code.count(b), f"{path}: unbalanced {a}{b}"
    pairs = 0
    for path in files:
        if not path.endswith("_d_hip.v"):
            continue
        twin = path[:-len("_d_hip.v")] + "_notd_hip.v"
        if not os.path.exists(twin):
            continue
        pairs += 1
        d, n = _pub_fns(open(path).read()), _pub_fns(open(twin).read())
        # the stub side may be a subset only where the `-d hip` side adds device-only helpers that
        # nothing outside `$if hip ? {}` calls; what both define must agree exactly
        # (the device tensor type exists only with `-d hip`: where the real function returns
        # &HipTensor[T] / &HipStorage[T] the stub returns &Tensor[T] / &CpuStorage[T], as
        # tensor_cuda_notd_cuda.v:12-15 and storage/cuda_notd_cuda.v:13-16 do)
        def device_to_host(t):
            return t.replace("HipTensor[", "Tensor[").replace("HipStorage[", "CpuStorage[")
        norm = lambda sig: (tuple(device_to_host(t) for t in sig[0]), device_to_host(sig[1]))   # noqa: E731
        for key in sorted(set(d) & set(n)):
            assert norm(d[key]) == norm(n[key]), \
                f"{os.path.basename(path)}: {key[1]} differs from its stub: {d[key]} vs {n[key]}"
        missing = sorted(k[1] for k in set(n) - set(d))
        assert not missing, f"{os.path.basename(twin)} defines {missing}, its `-d hip` twin does not"
    assert pairs >= 6
