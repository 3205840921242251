"""Inference modules that run packed quantized weights directly."""

from .backends import (  # noqa: F401
    Backend,
    EmbeddingBackend,
    LinearBackend,
    NormBackend,
    VQBackend,
    is_cuda_jit_available,
    is_hip_backend_available,
)
from .np_embedding import NPEmbedding, linearize_qtensor_embeddings  # noqa: F401
from .np_linear import NPLinear, linearize_qtensor_weights  # noqa: F401
from .np_vq_linear import NPVQLinear, VQProxy, linearize_vq_weights  # noqa: F401
from .np_rms_norm import NPRMSNorm, linearize_rms_norms  # noqa: F401
from .np_vq_embedding import NPVQEmbedding, linearize_vq_embeddings  # noqa: F401
