"""MI355X (gfx950) backend of VTL's INT8 quantized-linear path.

`capi` binds the C ABI of libvtlhip.so; `storage`, `tensor`, `layers` and
`models` mirror the V files that plug it into VTL (HipStorage, HipTensor,
the linear_forward_f32 hook, Sequential.linear).
"""
from . import capi  # noqa: F401
from .layers import (PER_CHANNEL, PER_TENSOR, HipSession, QuantLinearLayer,  # noqa: F401
                     QuantizedWeights, hip_backward_enabled, hip_linear_enabled,
                     hip_tests_enabled, linear_backward_hip_f32, linear_forward_f32_use_hip,
                     linear_forward_hip_exact, linear_forward_hip_f32,
                     linear_gate_use_hip_backward, matmul_gate_backward_hip, matmul_hip_host,
                     relu_forward_hip_f32,
                     sigmoid_forward_hip_f32)
from .models import Sequential  # noqa: F401
from .storage import HipParams, HipStorage, hip_available  # noqa: F401
from .tensor import (HipTensor, colsum_hip, gemm_i8_hip, linear_backward_hip,  # noqa: F401
                     linear_f32_dynquant_hip, linear_hip, linear_i8_hip, linear_i8_requant_hip,
                     matmul_hip)
