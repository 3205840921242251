"""Byte-level storage formats of scalar-quantized weights, and checkpoint IO (``model_io``)."""

from .packing import BitPacking, BitPacking1, BitPacking2, BitPacking4, BitPacking8  # noqa: F401
