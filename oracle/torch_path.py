"""The reference's CPU forward path restated with torch ops (test infrastructure).

Used (a) as the timed CPU baseline next to the GPU numbers and (b) as a
second, independently written check on ``np_oracle.c``.  It follows the
reference's eager path: unpack indices -> gather codebook rows -> cast to the
activation dtype -> ``torch.nn.functional.linear``.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def unpack_bitloop(packed: torch.Tensor, bits: int, n_indices: int) -> torch.Tensor:
    """Per-bit unpack, one pass over the stream per bit.

    Follows neuropress/transforms/vq_packing.py:174-203 (8/4-bit cases) and
    :284-295 (generic loop).  This is what the reference actually runs on CPU.
    """
    if bits == 8:
        return packed.to(torch.int64)[:n_indices]
    if bits == 4:
        p = packed.to(torch.int32)
        return torch.stack([p & 0xF, (p >> 4) & 0xF], dim=1).flatten().to(torch.int64)[:n_indices]
    p = packed.to(torch.int64)
    out = torch.zeros(n_indices, dtype=torch.int64)
    i = torch.arange(n_indices, dtype=torch.int64)
    for b in range(bits):
        pos = i * bits + b
        out |= ((p[pos >> 3] >> (pos & 7)) & 1) << b
    return out


def unpack_fast(packed: torch.Tensor, bits: int, n_indices: int) -> torch.Tensor:
    """Vectorised unpack for the widths the benchmark uses (same result as the bit loop)."""
    if bits == 16:
        return packed[: 2 * n_indices].view(torch.int16).to(torch.int64) & 0xFFFF
    if bits == 12:
        t = packed[: (n_indices * 12 + 7) // 8].to(torch.int64)
        pad = (-t.numel()) % 3
        if pad:
            t = torch.cat([t, t.new_zeros(pad)])
        t = t.view(-1, 3)
        even = t[:, 0] | ((t[:, 1] & 0xF) << 8)
        odd = (t[:, 1] >> 4) | (t[:, 2] << 4)
        return torch.stack([even, odd], dim=1).flatten()[:n_indices]
    return unpack_bitloop(packed, bits, n_indices)


def vq_decode_cpu(packed, centroids, bits, out_features, in_features, dtype, fast_unpack=True) -> torch.Tensor:
    """The decode half of :func:`vq_linear_cpu`: unpack, gather codebook rows, cast."""
    n_vec = out_features * in_features // centroids.shape[1]
    idx = (unpack_fast if fast_unpack else unpack_bitloop)(packed, bits, n_vec)
    return centroids[idx].reshape(out_features, in_features).to(dtype)


def q_decode_cpu(u8_blob, scale, nbits, group_size, dtype, zero_point=None) -> torch.Tensor:
    """The decode half of :func:`q_linear_cpu` (neuropress/nn/np_linear.py:333-353)."""
    vpb = 8 // nbits
    n, kp = u8_blob.shape
    k = kp * vpb
    shifts = torch.arange(vpb, dtype=torch.int32) * nbits
    vals = ((u8_blob.to(torch.int32).unsqueeze(-1) >> shifts) & ((1 << nbits) - 1)).reshape(n, k)
    vals_f = vals.to(torch.float32).reshape(n, k // group_size, group_size)
    sc = scale.to(torch.float32).reshape(n, k // group_size, 1)
    zp = zero_point.to(torch.float32).reshape(n, k // group_size, 1) if zero_point is not None else float(1 << (nbits - 1))
    return ((vals_f - zp) * sc).reshape(n, k).to(dtype)


def vq_linear_cpu(
    x: torch.Tensor,
    packed: torch.Tensor,
    centroids: torch.Tensor,
    bits: int,
    out_features: int,
    in_features: int,
    bias: torch.Tensor | None = None,
    fast_unpack: bool = True,
) -> torch.Tensor:
    """Follows neuropress/nn/np_vq_linear.py:1091-1095 (``_forward_default``)."""
    n_vec = out_features * in_features // centroids.shape[1]
    idx = (unpack_fast if fast_unpack else unpack_bitloop)(packed, bits, n_vec)
    w = centroids[idx].reshape(out_features, in_features)
    return F.linear(x, w.to(x.dtype), bias)


def q_linear_cpu(
    x: torch.Tensor,
    u8_blob: torch.Tensor,
    scale: torch.Tensor,
    nbits: int,
    group_size: int,
    zero_point: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """Follows neuropress/nn/np_linear.py:333-353 (``_q_dequant_linear``)."""
    vpb = 8 // nbits
    n, kp = u8_blob.shape
    k = kp * vpb
    shifts = torch.arange(vpb, dtype=torch.int32) * nbits
    vals = ((u8_blob.to(torch.int32).unsqueeze(-1) >> shifts) & ((1 << nbits) - 1)).reshape(n, k)
    vals_f = vals.to(torch.float32).reshape(n, k // group_size, group_size)
    sc = scale.to(torch.float32).reshape(n, k // group_size, 1)
    zp = (
        zero_point.to(torch.float32).reshape(n, k // group_size, 1)
        if zero_point is not None
        else float(1 << (nbits - 1))
    )
    w = (vals_f - zp) * sc
    return F.linear(x, w.reshape(n, k).to(x.dtype), bias)
