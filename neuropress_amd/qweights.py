"""Quantized-weight containers the lowering pass consumes.

In the reference a quantized ``nn.Linear`` carries a QTensor subclass from the
third-party ``torch_to_nnef`` package (``QTensorTractVQ``, ``QTensorTractScaleOnly``,
``QTensorScaleZp``).  That package is not a dependency here; the lowering pass
only reads a handful of attributes from those objects, so it is written
against that attribute surface (duck typing) and these light containers
provide it:

VQ weight (reference: neuropress/transforms/vq.py, neuropress/nn/np_vq_linear.py:856-921)
    ``w.u8_blob``                       packed index stream, 1-D uint8
    ``w.qscheme.centroids``             ``[NC, VL]`` codebook
    ``w.qscheme.vector_len``
    ``w.qscheme.is_packed_indices``     bits per index
    ``w.qscheme.column_permutation``    optional int64 ``[K]``
    ``w.qscheme.use_tiered / tier_bits / zero_escape``   entropy-coded formats (not supported)

Scalar weight (reference: neuropress/nn/np_linear.py:563-607)
    ``w.u8_blob``                       ``[N, K/vpb]`` packed codes
    ``w.qscheme.n_bits / group_size / scale``  and optional ``zero_point``
    ``w.dequant_to_dtype``

Real neuropress QTensors expose the same attributes, so a model quantized by
the reference lowers through the same code.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch
from torch import nn

from .t2n.packing import BitPacking
from .transforms.vq_packing import IndexPacking


@dataclass
class VQScheme:
    """Codebook + layout of a vector-quantized weight."""

    centroids: torch.Tensor
    original_shape: torch.Size | tuple
    is_packed_indices: int = 0  # bits per index; 0 -> derive from the codebook size
    column_permutation: torch.Tensor | None = None
    use_tiered: bool = False
    tier_bits: list[int] | None = None
    zero_escape: bool = False
    # optional residual stage + per-output-row affine (no counterpart in the reference)
    residual_centroids: torch.Tensor | None = None
    residual_bits: int = 0
    row_scale: torch.Tensor | None = None
    row_bias: torch.Tensor | None = None

    def __post_init__(self) -> None:
        if not self.is_packed_indices:
            self.is_packed_indices = IndexPacking.bits_for(self.centroids.shape[0])
        if self.residual_centroids is not None and not self.residual_bits:
            self.residual_bits = IndexPacking.bits_for(self.residual_centroids.shape[0])

    @property
    def vector_len(self) -> int:
        return self.centroids.shape[1]

    @property
    def num_centroids(self) -> int:
        return self.centroids.shape[0]

    def dequantize(self, packed_indices: torch.Tensor, target_dtype: torch.dtype) -> torch.Tensor:
        """Gather decode with torch ops (reference: neuropress/transforms/vq.py:361-414)."""
        n_vec = 1
        for d in self.original_shape:
            n_vec *= d
        n_vec //= self.vector_len
        if self.zero_escape or self.tier_bits is not None or self.use_tiered:
            from .transforms.vq_entropy_packing import decode_to_flat

            idx = decode_to_flat(packed_indices, use_tiered=self.use_tiered, tier_bits=self.tier_bits,
                                 zero_escape=self.zero_escape)  # fmt: skip
        else:
            idx = IndexPacking.unpack(packed_indices, self.is_packed_indices, n_vec)
        out = self.centroids.to(packed_indices.device)[idx].to(target_dtype)
        out = out.flatten().reshape(tuple(self.original_shape))
        if self.column_permutation is not None:
            inv = torch.argsort(self.column_permutation.to(out.device))
            out = out.reshape(-1, inv.numel())[:, inv].reshape(tuple(self.original_shape))
        return out


class VQWeight:
    """A vector-quantized weight: packed index stream(s) + :class:`VQScheme`."""

    def __init__(self, u8_blob: torch.Tensor, qscheme: VQScheme,
                 residual_blob: torch.Tensor | None = None) -> None:  # fmt: skip
        self.u8_blob = u8_blob
        self.qscheme = qscheme
        self.residual_blob = residual_blob

    @classmethod
    def from_indices(
        cls,
        indices: torch.Tensor,
        centroids: torch.Tensor,
        out_features: int,
        in_features: int,
        column_permutation: torch.Tensor | None = None,
        bits: int = 0,
        use_tiered: bool = False,
        hot_bits: int = 4,
        tier_bits: list[int] | None = None,
        zero_escape: bool = False,
    ) -> VQWeight:
        """Pack *indices* in the fixed-width format, or in a prefix-coded one when a flag names it
        (the choice the reference makes in ``VQScheme.quantize_as_u8``, neuropress/transforms/vq.py:351-357)."""
        from .transforms.vq_entropy_packing import NTieredIndexPacking, TieredIndexPacking, ZeroEscapePacking

        if zero_escape:
            use_tiered, tier_bits = False, None
        elif tier_bits is not None:
            use_tiered = False
        scheme = VQScheme(
            centroids=centroids,
            original_shape=(out_features, in_features),
            is_packed_indices=bits,
            column_permutation=column_permutation,
            use_tiered=use_tiered,
            tier_bits=tier_bits,
            zero_escape=zero_escape,
        )
        if zero_escape:
            blob = ZeroEscapePacking.pack(indices, scheme.is_packed_indices)
        elif tier_bits is not None:
            blob = NTieredIndexPacking.pack(indices, tier_bits)
        elif use_tiered:
            blob = TieredIndexPacking.pack(indices, scheme.is_packed_indices, hot_bits)
        else:
            blob = IndexPacking.pack(indices, scheme.is_packed_indices)
        return cls(blob, scheme)

    @property
    def shape(self) -> tuple:
        return tuple(self.qscheme.original_shape)


@dataclass
class ScalarQScheme:
    """Group-affine n-bit scheme: ``w = (q - zp) * scale``, zp = 2**(n_bits-1) when symmetric."""

    n_bits: int
    group_size: int
    scale: torch.Tensor
    zero_point: torch.Tensor | None = None

    def per_group_zero_point(self) -> torch.Tensor | None:
        if self.zero_point is None:
            return None
        if self.zero_point.numel() == 1:
            return self.zero_point.reshape(1).expand(self.scale.numel()).clone()
        return self.zero_point


class ScalarQWeight:
    """A scalar-quantized weight: ``[N, K/vpb]`` packed codes + :class:`ScalarQScheme`."""

    def __init__(self, u8_blob: torch.Tensor, qscheme: ScalarQScheme,
                 dequant_to_dtype: torch.dtype = torch.float16,
                 u8_compressors: list | None = None) -> None:  # fmt: skip
        self.u8_blob = u8_blob
        self.qscheme = qscheme
        self.dequant_to_dtype = dequant_to_dtype
        self.u8_compressors = (
            [BitPacking(qscheme.n_bits)] if u8_compressors is None else u8_compressors
        )

    @classmethod
    def from_codes(cls, codes: torch.Tensor, scale: torch.Tensor, n_bits: int, group_size: int,
                   zero_point: torch.Tensor | None = None,
                   dequant_to_dtype: torch.dtype = torch.float16) -> ScalarQWeight:  # fmt: skip
        """*codes*: one value per byte, ``[N, K]`` uint8."""
        blob = BitPacking(n_bits).compress(codes.to(torch.uint8))
        return cls(blob, ScalarQScheme(n_bits, group_size, scale, zero_point), dequant_to_dtype)

    def decompress_to_u8(self) -> torch.Tensor:
        out = self.u8_blob
        for comp in reversed(self.u8_compressors):
            out = comp.decompress(out)
        return out


def attach_quantized_weight(linear: nn.Linear, weight) -> nn.Linear:
    """Make *weight* the ``.weight`` of *linear* without going through ``nn.Parameter``."""
    linear._parameters.pop("weight", None)
    linear.__dict__["weight"] = weight
    return linear


def is_vq_weight(w) -> bool:
    q = getattr(w, "qscheme", None)
    return q is not None and hasattr(q, "centroids") and hasattr(w, "u8_blob")


def is_scalar_qweight(w) -> bool:
    q = getattr(w, "qscheme", None)
    return q is not None and hasattr(q, "n_bits") and hasattr(q, "group_size") and hasattr(w, "u8_blob")
