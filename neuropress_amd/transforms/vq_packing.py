"""Fixed-width index packing: the wire format of VQ codebook indices.

Index ``i`` occupies bits ``[i*bits, (i+1)*bits)`` of a byte stream, LSB first;
unused high bits of the last byte are zero.  Same format and the same
``IndexPacking`` surface (``bits_for`` / ``pack`` / ``unpack``) as the
reference (neuropress/transforms/vq_packing.py:97-295).

The implementation is window-based rather than bit-by-bit: an index of up to
20 bits starting at bit offset <= 7 touches at most four consecutive bytes, so
packing adds four byte planes into the stream and unpacking reads a four-byte
window, shifts and masks.
"""

from __future__ import annotations

import math

import torch


class IndexPacking:
    """Static pack / unpack utilities; the bit width travels next to the buffer."""

    _MIN_BITS: int = 4
    _MAX_BITS: int = 20
    _MAX_CENTROIDS: int = 1 << 20

    @staticmethod
    def bits_for(num_centroids: int) -> int:
        """``max(4, ceil(log2(num_centroids)))``; raises outside ``[2, 2**20]``."""
        if num_centroids < 2:
            raise ValueError(f"num_centroids must be >= 2, got {num_centroids}.")
        if num_centroids > IndexPacking._MAX_CENTROIDS:
            raise ValueError(
                f"num_centroids={num_centroids} exceeds the maximum supported "
                f"value of {IndexPacking._MAX_CENTROIDS} (20-bit indices)."
            )
        return max(IndexPacking._MIN_BITS, (num_centroids - 1).bit_length())

    @staticmethod
    def _check_bits(bits: int) -> None:
        if not (IndexPacking._MIN_BITS <= bits <= IndexPacking._MAX_BITS):
            raise ValueError(
                f"bits must be in [{IndexPacking._MIN_BITS}, {IndexPacking._MAX_BITS}], got {bits}."
            )

    @staticmethod
    def packed_nbytes(n_indices: int, bits: int) -> int:
        return math.ceil(n_indices * bits / 8)

    @staticmethod
    def pack(indices: torch.Tensor, bits: int) -> torch.Tensor:
        """Pack a flat integer tensor (values < 2**bits) into ``ceil(n*bits/8)`` uint8 bytes."""
        IndexPacking._check_bits(bits)
        flat = indices.flatten().to(torch.int64)
        n = flat.numel()
        if bits == 8:
            return flat.to(torch.uint8)
        if bits == 4 and n % 2 != 0:
            raise ValueError(
                f"IndexPacking(bits=4): index count ({n}) must be even for 4-bit packing."
            )
        if bits == 16:
            lo = (flat & 0xFF).to(torch.uint8)
            hi = ((flat >> 8) & 0xFF).to(torch.uint8)
            return torch.stack([lo, hi], dim=1).flatten()
        n_bytes = IndexPacking.packed_nbytes(n, bits)
        bit0 = torch.arange(n, dtype=torch.int64, device=flat.device) * bits
        byte0 = bit0 >> 3
        shifted = (flat & ((1 << bits) - 1)) << (bit0 & 7)  # < 2**27
        # Four byte planes; fields of different indices never share a bit, so
        # summing the planes into the stream is the same as OR-ing them.
        out = torch.zeros(n_bytes + 4, dtype=torch.int64, device=flat.device)
        for plane in range(4):
            out.index_add_(0, byte0 + plane, (shifted >> (8 * plane)) & 0xFF)
        return out[:n_bytes].to(torch.uint8)

    @staticmethod
    def unpack(packed: torch.Tensor, bits: int, n_indices: int) -> torch.Tensor:
        """Unpack *n_indices* indices to a 1-D int64 tensor (on the buffer's device)."""
        IndexPacking._check_bits(bits)
        if bits == 8:
            return packed.to(torch.int64)[:n_indices]
        if packed.is_cuda and bits <= 16:
            from .. import kernels

            try:
                return kernels.unpack_indices(packed, n_indices, bits)
            except RuntimeError:
                pass  # library missing: the torch ops below work on any device
        p = packed.flatten().to(torch.int64)
        if bits == 16:
            pair = p[: 2 * n_indices].view(-1, 2)
            return pair[:, 0] | (pair[:, 1] << 8)
        p = torch.cat([p, p.new_zeros(4)])
        bit0 = torch.arange(n_indices, dtype=torch.int64, device=p.device) * bits
        byte0 = bit0 >> 3
        window = p[byte0] | (p[byte0 + 1] << 8) | (p[byte0 + 2] << 16) | (p[byte0 + 3] << 24)
        return (window >> (bit0 & 7)) & ((1 << bits) - 1)


# The prefix-coded storage formats live in their own module; they are importable from here as in
# the reference (neuropress/transforms/vq_packing.py:298, 612, 1037).
from .vq_entropy_packing import (  # noqa: E402, F401
    NTieredIndexPacking,
    TieredIndexPacking,
    ZeroEscapePacking,
)
