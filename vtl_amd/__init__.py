"""MI355X (gfx950) backend of VTL's INT8 quantized-linear path.

`capi` binds the C ABI of libvtlhip.so; `storage`, `tensor`, `layers` and
`models` mirror the V files that plug it into VTL (HipStorage, HipTensor,
the linear_forward_f32 hook, Sequential.linear).
"""
from . import capi  # noqa: F401
from .layers import (PER_CHANNEL, PER_TENSOR, HipSession, QuantLinearLayer,  # noqa: F401
                     QuantizedWeights, hip_linear_enabled, hip_tests_enabled,
                     linear_forward_f32_use_hip, linear_forward_hip_f32)
from .models import Sequential  # noqa: F401
from .storage import HipParams, HipStorage, hip_available  # noqa: F401
from .tensor import (HipTensor, gemm_i8_hip, linear_f32_dynquant_hip,  # noqa: F401
                     linear_i8_hip)
