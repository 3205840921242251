"""Byte-level storage formats of scalar-quantized weights."""

from .packing import BitPacking, BitPacking1, BitPacking2, BitPacking4, BitPacking8  # noqa: F401
