"""Inference modules that run packed quantized weights directly."""

from .backends import Backend, LinearBackend, VQBackend, is_cuda_jit_available, is_hip_backend_available  # noqa: F401
from .np_linear import NPLinear, linearize_qtensor_weights  # noqa: F401
from .np_vq_linear import NPVQLinear, VQProxy, linearize_vq_weights  # noqa: F401
