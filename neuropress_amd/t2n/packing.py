"""n-bit value packing for scalar-quantized weights (1, 2, 4 or 8 bits).

Values are packed LSB-first inside each byte; for 4 bits
``byte = (x[2i] & 0xF) | ((x[2i+1] & 0xF) << 4)``.  Same layout and the same
``compress`` / ``decompress`` surface as the reference's ``BitPacking``
(neuropress/t2n/packing.py:48-207); the third-party base class it derives from
there is not needed for the layout and is not reproduced.
"""

from __future__ import annotations

import torch


class BitPacking:
    """Pack *nbits*-wide unsigned values (one per uint8) along the last dimension."""

    def __init__(self, nbits: int) -> None:
        if nbits not in (1, 2, 4, 8):
            raise ValueError(f"nbits must be one of 1, 2, 4, 8; got {nbits}")
        self.nbits = nbits
        self.vpb = 8 // nbits

    def compress(self, u8_tensor: torch.Tensor) -> torch.Tensor:
        """``[..., K]`` uint8 values -> ``[..., K / vpb]`` packed bytes."""
        if u8_tensor.dtype != torch.uint8:
            raise TypeError(f"expected uint8, got {u8_tensor.dtype}")
        if self.nbits == 8:
            return u8_tensor.clone()
        if u8_tensor.shape[-1] % self.vpb:
            raise ValueError(
                f"last dimension ({u8_tensor.shape[-1]}) must be divisible by {self.vpb} "
                f"for {self.nbits}-bit packing"
            )
        mask = (1 << self.nbits) - 1
        lanes = (u8_tensor.to(torch.int32) & mask).unflatten(-1, (-1, self.vpb))
        weights = 1 << (torch.arange(self.vpb, dtype=torch.int32, device=u8_tensor.device) * self.nbits)
        return (lanes * weights).sum(dim=-1).to(torch.uint8)

    def decompress(self, packed: torch.Tensor) -> torch.Tensor:
        """Inverse of :meth:`compress`."""
        if self.nbits == 8:
            return packed.clone()
        shifts = torch.arange(self.vpb, dtype=torch.int32, device=packed.device) * self.nbits
        vals = (packed.to(torch.int32).unsqueeze(-1) >> shifts) & ((1 << self.nbits) - 1)
        return vals.flatten(-2).to(torch.uint8)

    def __repr__(self) -> str:
        return f"BitPacking(nbits={self.nbits})"


BitPacking1 = BitPacking(1)
BitPacking2 = BitPacking(2)
BitPacking4 = BitPacking(4)
BitPacking8 = BitPacking(8)
