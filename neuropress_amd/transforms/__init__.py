"""Wire formats consumed by the quantized-linear path."""

from .vq_packing import IndexPacking  # noqa: F401
