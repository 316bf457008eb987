"""Device tensor: the Python mirror of the V file `tensor_hip_d_hip.v`.

Follows `CudaTensor[T]` (tensor_cuda_d_cuda.v:13-60): storage plus shape and
row-major strides, `Tensor.hip()` / `.cpu()` / `.release()`, shape predicates,
and the INT8 operations of the quantized-linear path.  numpy arrays stand in
for `vtl.Tensor[T]` on the host side.
"""
from __future__ import annotations

import numpy as np

from . import capi
from .storage import HipParams, HipStorage


def _strides_from_shape(shape):
    """Row-major element strides (util.v:169-184)."""
    strides = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        strides[i] = strides[i + 1] * shape[i + 1]
    return strides


class HipTensor:
    """`HipTensor[T]{data &storage.HipStorage[T]; memory; size; shape; strides}`."""

    def __init__(self, data: HipStorage, shape):
        self.data = data
        self.memory = "row_major"
        self.shape = [int(s) for s in shape]
        self.size = int(np.prod(self.shape)) if self.shape else 1
        self.strides = _strides_from_shape(self.shape)
        if self.size != data.count:
            raise ValueError(f"HipTensor: shape {self.shape} does not match {data.count} elements")

    # -- construction / transfer (tensor_cuda_d_cuda.v:23-60) ----------------
    @staticmethod
    def from_host(t: np.ndarray, params: HipParams | None = None) -> "HipTensor":
        """`(t &Tensor[T]) hip(params) !&HipTensor[T]`: row-major copy, then upload."""
        row = np.ascontiguousarray(t)
        return HipTensor(HipStorage.from_cpu(row, params), row.shape)

    @staticmethod
    def empty(shape, dtype, params: HipParams | None = None) -> "HipTensor":
        count = int(np.prod(shape)) if len(shape) else 1
        return HipTensor(HipStorage.empty(count, dtype, params), shape)

    def hip(self, params: HipParams | None = None) -> "HipTensor":
        return self

    def cpu(self) -> np.ndarray:
        return self.data.cpu().reshape(self.shape)

    def release(self) -> None:
        self.data.release()

    # -- predicates (tensor_cuda_d_cuda.v:63-120) ------------------------------
    @property
    def dtype(self):
        return self.data.dtype

    @property
    def ptr(self) -> int:
        return self.data.ptr

    def rank(self) -> int:
        return len(self.shape)

    def numel(self) -> int:
        return self.size

    def is_matrix(self) -> bool:
        return self.rank() == 2

    def is_square_matrix(self) -> bool:
        return self.rank() == 2 and self.shape[0] == self.shape[1]

    def is_vector(self) -> bool:
        return self.rank() == 1

    def is_row_major(self) -> bool:
        return self.memory == "row_major"

    def is_col_major(self) -> bool:
        return self.memory == "col_major"

    def is_row_major_contiguous(self) -> bool:
        """Strides are those of a dense row-major tensor (tensor_cuda_d_cuda.v:128-130)."""
        return self.is_row_major() and self.strides == _strides_from_shape(self.shape)

    def is_col_major_contiguous(self) -> bool:
        """tensor_cuda_d_cuda.v:138-140; a device tensor is always uploaded row-major."""
        if not self.is_col_major():
            return False
        strides, acc = [], 1
        for d in self.shape:
            strides.append(acc)
            acc *= d
        return self.strides == strides

    def is_contiguous(self) -> bool:
        """tensor_cuda_d_cuda.v:148-150."""
        return self.is_row_major_contiguous() or self.is_col_major_contiguous()

    def _assert(self, dtype, matrix=True, what="tensor"):
        if self.dtype != np.dtype(dtype):
            raise TypeError(f"{what}: expected {np.dtype(dtype)}, got {self.dtype}")
        if matrix and not self.is_matrix():
            raise ValueError(f"{what}: Matrix expected, got shape {self.shape}")

    # -- INT8 quantization vocabulary ------------------------------------------
    def absmax(self, axis: int = -1) -> "HipTensor":
        """max |x| over the tensor (axis -1) or per row (axis 0 keeps rows)."""
        self._assert(np.float32, what="absmax")
        rows, cols = self.shape
        per_row = _per_row(axis)
        out = HipTensor.empty([rows if per_row else 1], np.float32, HipParams(self.data.device_id))
        capi.call("vtl_hip_absmax_f32", self.ptr, rows, cols, per_row, out.ptr)
        return out

    def quantize_i8(self, axis: int = -1):
        """`quantize_i8(axis /*-1 tensor, 0 row*/) !(&HipTensor[i8], &HipTensor[f32])`."""
        self._assert(np.float32, what="quantize_i8")
        rows, cols = self.shape
        per_row = _per_row(axis)
        p = HipParams(self.data.device_id)
        q = HipTensor.empty([rows, cols], np.int8, p)
        s = HipTensor.empty([rows if per_row else 1], np.float32, p)
        capi.call("vtl_hip_quantize_f32_i8", self.ptr, rows, cols, per_row, q.ptr, s.ptr)
        return q, s

    def quantize_i8_with_scale(self, scales: "HipTensor", axis: int = -1) -> "HipTensor":
        self._assert(np.float32, what="quantize_i8_with_scale")
        scales._assert(np.float32, matrix=False, what="scales")
        rows, cols = self.shape
        per_row = _per_row(axis)
        if scales.size != (rows if per_row else 1):
            raise ValueError(f"scales: expected {rows if per_row else 1} entries, got {scales.size}")
        q = HipTensor.empty([rows, cols], np.int8, HipParams(self.data.device_id))
        capi.call("vtl_hip_quantize_with_scale_f32_i8", self.ptr, scales.ptr, rows, cols, per_row, q.ptr)
        return q

    def dequantize(self, scales: "HipTensor", axis: int = -1) -> "HipTensor":
        """`(q &HipTensor[i8]) dequantize(scales &HipTensor[f32], axis int) !&HipTensor[f32]`."""
        self._assert(np.int8, what="dequantize")
        scales._assert(np.float32, matrix=False, what="scales")
        rows, cols = self.shape
        per_row = _per_row(axis)
        if scales.size != (rows if per_row else 1):
            raise ValueError(f"scales: expected {rows if per_row else 1} entries, got {scales.size}")
        x = HipTensor.empty([rows, cols], np.float32, HipParams(self.data.device_id))
        capi.call("vtl_hip_dequantize_i8_f32", self.ptr, scales.ptr, rows, cols, per_row, x.ptr)
        return x

    def relu_(self) -> "HipTensor":
        """In-place ReLU (x < 0 -> 0), cf. relu_cuda tensor_cuda_d_cuda.v:205-235."""
        sfx = _float_suffix(self, "relu_")
        capi.call(f"vtl_hip_relu_{sfx}", self.ptr, self.size)
        return self

    def relu_hip(self) -> "HipTensor":
        """`relu_hip() !&HipTensor[T]`: a new tensor, as relu_cuda (tensor_cuda_d_cuda.v:205-235)."""
        out = HipTensor.empty(self.shape, self.dtype, HipParams(self.data.device_id))
        capi.call("vtl_hip_memcpy_d2d", out.ptr, self.ptr, self.data.size)
        return out.relu_()

    def sigmoid_hip(self) -> "HipTensor":
        """`sigmoid_hip() !&HipTensor[T]`: 1 / (1 + exp(-x)), as sigmoid_cuda
        (tensor_cuda_d_cuda.v:237-270) with the arithmetic of nn/internal/activation.v:35-40."""
        sfx = _float_suffix(self, "sigmoid_hip")
        out = HipTensor.empty(self.shape, self.dtype, HipParams(self.data.device_id))
        capi.call(f"vtl_hip_sigmoid_{sfx}", self.ptr, out.ptr, self.size)
        return out


def _per_row(axis: int) -> int:
    if axis == -1:
        return 0
    if axis == 0:
        return 1
    raise ValueError(f"axis {axis}: use -1 (whole tensor) or 0 (one scale per row)")


def _matmul_shapes(a: HipTensor, bt: HipTensor):
    """Shape rule of la.matmul (la/la.v:38-43) for a second operand stored [N,K]."""
    if not a.is_matrix() or not bt.is_matrix():
        raise ValueError("Matrix expected")
    if a.shape[1] != bt.shape[1]:
        raise ValueError(
            f"Invalid shapes for matrix multiplication {a.shape} and {[bt.shape[1], bt.shape[0]]}")
    return a.shape[0], bt.shape[0], a.shape[1]


def gemm_i8_hip(dst: HipTensor, a: HipTensor, bt: HipTensor) -> None:
    """`gemm_i8_hip(dst &HipTensor[int], a &HipTensor[i8], b &HipTensor[i8]) !`

    dst[M,N] = a[M,K] . bt[N,K]^T in exact int32 (style of gemm_cuda,
    tensor_cuda_d_cuda.v:155-177)."""
    a._assert(np.int8, what="gemm_i8_hip a")
    bt._assert(np.int8, what="gemm_i8_hip b")
    dst._assert(np.int32, what="gemm_i8_hip dst")
    M, N, K = _matmul_shapes(a, bt)
    if dst.shape != [M, N]:
        raise ValueError(f"gemm_i8_hip: dst shape {dst.shape}, expected {[M, N]}")
    capi.call("vtl_hip_gemm_i8_i32", a.ptr, bt.ptr, dst.ptr, M, N, K)


def linear_i8_hip(x_q: HipTensor, sx: HipTensor, w_q: HipTensor, sw: HipTensor,
                  bias: HipTensor | None, relu: bool = False) -> HipTensor:
    """`linear_i8_hip(x_q, sx, w_q, sw, bias) !&HipTensor[f32]`: y = x.W^T + b on int8 codes."""
    x_q._assert(np.int8, what="linear_i8_hip x_q")
    w_q._assert(np.int8, what="linear_i8_hip w_q")
    M, N, K = _matmul_shapes(x_q, w_q)
    if sx.size not in (1, M) or sw.size not in (1, N):
        raise ValueError("linear_i8_hip: scale sizes do not match the operands")
    if bias is not None and bias.size != N:
        raise ValueError(f"linear_i8_hip: bias has {bias.size} entries, expected {N}")
    y = HipTensor.empty([M, N], np.float32, HipParams(x_q.data.device_id))
    capi.call("vtl_hip_linear_i8_f32", x_q.ptr, sx.ptr, int(sx.size == M), w_q.ptr, sw.ptr,
              int(sw.size == N), bias.ptr if bias is not None else None, y.ptr, M, N, K, int(relu))
    return y


def linear_i8_requant_hip(x_q: HipTensor, sx: HipTensor, w_q: HipTensor, sw: HipTensor,
                          bias: HipTensor | None, relu: bool = False, keep_f32: bool = False):
    """`linear_i8_requant_hip(x_q, sx, w_q, sw, bias, relu) !(&HipTensor[i8], &HipTensor[f32])`:
    the int8 linear whose f32 rows are quantized per row for the next int8 layer in the
    same pass (the bits of linear_i8_hip followed by quantize_i8(0)).  With keep_f32 the
    f32 output is returned as a third tensor."""
    x_q._assert(np.int8, what="linear_i8_requant_hip x_q")
    w_q._assert(np.int8, what="linear_i8_requant_hip w_q")
    M, N, K = _matmul_shapes(x_q, w_q)
    if sx.size not in (1, M) or sw.size not in (1, N):
        raise ValueError("linear_i8_requant_hip: scale sizes do not match the operands")
    if bias is not None and bias.size != N:
        raise ValueError(f"linear_i8_requant_hip: bias has {bias.size} entries, expected {N}")
    params = HipParams(x_q.data.device_id)
    y_q = HipTensor.empty([M, N], np.int8, params)
    sy = HipTensor.empty([M], np.float32, params)
    y = HipTensor.empty([M, N], np.float32, params) if keep_f32 else None
    capi.call("vtl_hip_linear_i8_requant", x_q.ptr, sx.ptr, int(sx.size == M), w_q.ptr, sw.ptr,
              int(sw.size == N), bias.ptr if bias is not None else None, int(relu), y_q.ptr, sy.ptr,
              y.ptr if y is not None else None, M, N, K)
    return (y_q, sy, y) if keep_f32 else (y_q, sy)


def linear_f32_dynquant_hip(x: HipTensor, w_q: HipTensor, sw: HipTensor, bias: HipTensor | None,
                            relu: bool = False, workspace: HipStorage | None = None) -> HipTensor:
    """Per-token quantization of x on the fly, then the int8 linear."""
    x._assert(np.float32, what="linear_f32_dynquant_hip x")
    w_q._assert(np.int8, what="linear_f32_dynquant_hip w_q")
    M, N, K = _matmul_shapes(x, w_q)
    if sw.size != N:
        raise ValueError("linear_f32_dynquant_hip: one weight scale per output channel expected")
    if bias is not None and bias.size != N:
        raise ValueError(f"linear_f32_dynquant_hip: bias has {bias.size} entries, expected {N}")
    need = int(capi.lib().vtl_hip_linear_f32_dynquant_workspace(M, K))
    own = workspace is None or workspace.size < need
    ws = HipStorage.empty(need, np.uint8, HipParams(x.data.device_id)) if own else workspace
    y = HipTensor.empty([M, N], np.float32, HipParams(x.data.device_id))
    try:
        capi.call("vtl_hip_linear_f32_dynquant", x.ptr, w_q.ptr, sw.ptr,
                  bias.ptr if bias is not None else None, y.ptr, M, N, K, int(relu), ws.ptr, ws.size)
        if own:
            capi.call("vtl_hip_sync")
    finally:
        if own:
            ws.release()
    return y


def _float_suffix(t: HipTensor, what: str) -> str:
    if t.dtype == np.float32:
        return "f32"
    if t.dtype == np.float64:
        return "f64"
    raise TypeError(f"{what}: f32 or f64 tensor expected, got {t.dtype}")


def matmul_hip(a: HipTensor, b: HipTensor, trans_a: bool = False, trans_b: bool = False) -> HipTensor:
    """`matmul_hip(a, b) !&HipTensor[T]`: la.matmul (la/la.v:38-55) on the device, f64
    products and sums, one rounding to T.  trans_a / trans_b take the stored matrix
    as its transpose, which is how the gates pass `.t()` (autograd/gates_blas.v:43-48)."""
    sfx = _float_suffix(a, "matmul_hip")
    if b.dtype != a.dtype:
        raise TypeError("matmul_hip: operands of one type expected")
    if not a.is_matrix() or not b.is_matrix():
        raise ValueError("Matrix expected")
    m, k = (a.shape[1], a.shape[0]) if trans_a else a.shape
    k2, n = (b.shape[1], b.shape[0]) if trans_b else b.shape
    if k != k2:
        raise ValueError(f"Invalid shapes for matrix multiplication {[m, k]} and {[k2, n]}")
    c = HipTensor.empty([m, n], a.dtype, HipParams(a.data.device_id))
    capi.call(f"vtl_hip_matmul_{sfx}", a.ptr, b.ptr, c.ptr, m, n, k, int(trans_a), int(trans_b))
    return c


def linear_hip(x: HipTensor, w: HipTensor, bias: HipTensor | None, relu: bool = False) -> HipTensor:
    """The unquantized Linear forward y = matmul(x, W^T) + b with W as stored [N,K]
    (linear_forward_f32_cpu, nn/layers/linear_forward_f32.v:16-18)."""
    sfx = _float_suffix(x, "linear_hip")
    if w.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise TypeError("linear_hip: operands of one type expected")
    m, n, k = _matmul_shapes(x, w)
    if bias is not None and bias.size != n:
        raise ValueError(f"linear_hip: bias has {bias.size} entries, expected {n}")
    y = HipTensor.empty([m, n], x.dtype, HipParams(x.data.device_id))
    capi.call(f"vtl_hip_linear_{sfx}", x.ptr, w.ptr, bias.ptr if bias is not None else None, y.ptr,
              m, n, k, int(relu))
    return y


def colsum_hip(x: HipTensor) -> HipTensor:
    """la.matmul(ones[1,rows], x) as [1, cols] (nn/gates/layers/linear.v:75-79)."""
    sfx = _float_suffix(x, "colsum_hip")
    if not x.is_matrix():
        raise ValueError("Matrix expected")
    out = HipTensor.empty([1, x.shape[1]], x.dtype, HipParams(x.data.device_id))
    capi.call(f"vtl_hip_colsum_{sfx}", x.ptr, x.shape[0], x.shape[1], out.ptr)
    return out


def linear_backward_hip(grad: HipTensor, x: HipTensor, w: HipTensor, need_dx: bool = True,
                        need_dw: bool = True, need_db: bool = True):
    """LinearGate.backward on the device (nn/gates/layers/linear.v:57-79): returns
    [dx[M,K], dw[N,K], db[1,N]] with None where a gradient is not required."""
    sfx = _float_suffix(grad, "linear_backward_hip")
    if x.dtype != grad.dtype or w.dtype != grad.dtype:
        raise TypeError("linear_backward_hip: operands of one type expected")
    if not (grad.is_matrix() and x.is_matrix() and w.is_matrix()):
        raise ValueError("Matrix expected")
    m, n = grad.shape
    k = x.shape[1]
    if x.shape != [m, k] or w.shape != [n, k]:
        raise ValueError(f"linear_backward_hip: grad {grad.shape}, input {x.shape}, weight {w.shape}")
    params = HipParams(grad.data.device_id)
    dx = HipTensor.empty([m, k], grad.dtype, params) if need_dx else None
    dw = HipTensor.empty([n, k], grad.dtype, params) if need_dw else None
    db = HipTensor.empty([1, n], grad.dtype, params) if need_db else None
    capi.call(f"vtl_hip_linear_backward_{sfx}", grad.ptr, x.ptr, w.ptr,
              dx.ptr if dx is not None else None, dw.ptr if dw is not None else None,
              db.ptr if db is not None else None, m, n, k)
    return [dx, dw, db]


def gemv_hip(y: HipTensor, a: HipTensor, x: HipTensor) -> None:
    """`gemv_hip(y, a, x) !`: y = A . x for A [m, n], x [n], y [m] (gemv_cuda,
    tensor_cuda_d_cuda.v:182-203), f64 products and sums."""
    sfx = _float_suffix(a, "gemv_hip")
    if a.rank() != 2 or x.rank() != 1 or y.rank() != 1:
        raise ValueError("gemv_hip: A must be rank-2, x and y must be rank-1")
    if x.dtype != a.dtype or y.dtype != a.dtype:
        raise TypeError("gemv_hip: operands of one type expected")
    m, n = a.shape
    if x.size != n or y.size != m:
        raise ValueError(f"gemv_hip: A {a.shape}, x {x.shape}, y {y.shape}")
    capi.call(f"vtl_hip_gemv_{sfx}", a.ptr, x.ptr, y.ptr, m, n)
