"""Backend enumerations for the quantized inference modules.

String values are the reference's (neuropress/nn/backends.py:102-159) so that
recipes, YAML lowering configs and saved checkpoints keep working.  The names
that say "cuda" select the HIP kernels of this package:

===================  =========================================================
``cuda`` / ``cuda_wmma``  fused decode GEMV -> tile-decode MFMA GEMM -> decode + GEMM,
                          by token count
``cuda_lut``              decode + GEMM at every token count unless the LUT
                          threshold is raised (the routing the reference gives
                          large-codebook layers)
``compile`` / ``default`` gather + ``F.linear`` with torch ops (CPU or GPU)
===================  =========================================================

``is_cuda_jit_available`` keeps its name; here it answers "can the HIP kernel
library run": the shared object loads and a GPU is visible.
"""

from __future__ import annotations

import enum
import logging
import os

_log = logging.getLogger(__name__)

_hip_ok: bool | None = None


def is_hip_backend_available() -> bool:
    """True when ``libnpamd.so`` loads and torch sees a GPU.  Cached.

    ``NEUROPRESS_FORCE_CUDA_JIT=1`` skips the probe and answers True, as the
    reference's switch of the same name does (neuropress/nn/backends.py:40).
    """
    global _hip_ok
    if _hip_ok is not None:
        return _hip_ok
    if os.environ.get("NEUROPRESS_FORCE_CUDA_JIT", "").strip() in ("1", "true", "yes"):
        _hip_ok = True
        return True
    import torch

    from .. import _lib

    if not torch.cuda.is_available():
        _hip_ok = False
        return False
    _hip_ok = _lib.is_available()
    if not _hip_ok:
        _log.warning(
            "libnpamd.so could not be loaded; HIP backends disabled, falling back to torch ops"
        )
    return _hip_ok


# Name kept for drop-in compatibility with code written against the reference.
is_cuda_jit_available = is_hip_backend_available


class _StrEnum(str, enum.Enum):
    """``enum.StrEnum`` for Python < 3.11: members compare and format as their value."""

    def __str__(self) -> str:
        return str(self.value)

    def __format__(self, spec: str) -> str:
        return format(str(self.value), spec)


class LinearBackend(_StrEnum):
    """Valid backends for scalar-quantized ``nn.Linear`` (:class:`.NPLinear`)."""

    AUTO = "auto"
    DEFAULT = "default"
    COMPILE = "compile"
    CUDA = "cuda"
    GEMLITE = "gemlite"


class EmbeddingBackend(_StrEnum):
    """Valid backends for scalar-quantized ``nn.Embedding`` (:class:`.NPEmbedding`)."""

    AUTO = "auto"
    DEFAULT = "default"
    COMPILE = "compile"
    CUDA = "cuda"


class NormBackend(_StrEnum):
    """Valid backends for RMSNorm modules (:class:`.NPRMSNorm`)."""

    AUTO = "auto"
    DEFAULT = "default"
    CUDA = "cuda"


class VQBackend(_StrEnum):
    """Valid backends for vector-quantized ``nn.Linear`` (:class:`.NPVQLinear`)."""

    AUTO = "auto"
    DEFAULT = "default"
    COMPILE = "compile"
    CUDA = "cuda"
    CUDA_WMMA = "cuda_wmma"
    CUDA_LUT = "cuda_lut"
    CUDA_TIERED = "cuda_tiered"
    CUDA_NTIER = "cuda_ntier"
    CUDA_ZERO_ESCAPE = "cuda_zero_escape"


class Backend(_StrEnum):
    """Superset enum kept for backward compatibility."""

    DEFAULT = "default"
    COMPILE = "compile"
    CUDA = "cuda"
    CUDA_WMMA = "cuda_wmma"
    CUDA_LUT = "cuda_lut"
    CUDA_TIERED = "cuda_tiered"
    CUDA_NTIER = "cuda_ntier"
    CUDA_ZERO_ESCAPE = "cuda_zero_escape"
    GEMLITE = "gemlite"
    AUTO = "auto"


def tensor_version(t) -> int:
    """``t._version`` for cache keys, or -1 for tensors that keep no version counter.

    Tensors created or moved under ``torch.inference_mode()`` raise on ``_version``; they
    cannot be written in place outside inference mode either, so device and address identify them.
    """
    try:
        return t._version
    except RuntimeError:
        return -1


def tile_band_ok(
    m: int, n: int, k: int, cus: int, min_fraction: float, split_max_tokens: int, long_k: int
) -> bool:
    """Whether the tile-decode GEMM has enough workgroups for ``m`` tokens on an
    ``n x k`` layer.  Mirrors the kernel's own plan: without a split when the
    (64 columns x up to 384 rows) grid covers ``min_fraction`` of ``cus`` compute
    units; otherwise up to 16 reduction splits of at least 512 input features."""
    blocks = -(-n // 64) * -(-m // 384)
    if blocks >= min_fraction * cus:
        return True
    splits = max(1, min(cus // blocks, k // 512, 16))
    if splits * blocks < min_fraction * cus:
        return False
    return m <= split_max_tokens or k >= long_k
