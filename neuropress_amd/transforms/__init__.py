"""Wire formats consumed by the quantized-linear path."""

from .vq_packing import (  # noqa: F401
    IndexPacking,
    NTieredIndexPacking,
    TieredIndexPacking,
    ZeroEscapePacking,
)
