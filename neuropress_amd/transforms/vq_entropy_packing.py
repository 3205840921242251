"""Prefix-coded (entropy-coded) index formats: storage forms of a VQ index stream.

Three self-describing ``uint8`` buffers, wire-compatible with the reference
(neuropress/transforms/vq_packing.py:298-1384).  All assume a
frequency-sorted codebook (index 0 = most used), so small indices get short
codes:

* :class:`TieredIndexPacking` -- one prefix bit per index picks a *hot*
  (``hot_bits``) or a *cold* (``cold_bits``) payload.
* :class:`NTieredIndexPacking` -- 2 to 4 tiers; level ``k`` spends one prefix
  bit on every index not claimed by an earlier tier.
* :class:`ZeroEscapePacking` -- a 2-bit class per index: index 0 (no payload),
  1..16 (4 bits), 17..256 (8 bits), the rest (``cold_bits``).

Every buffer is: little-endian ``uint32`` header, prefix stream(s), then one
fixed-width payload stream per tier in tier order (each a plain
:class:`IndexPacking` stream of tier-local values, LSB first).

On this backend these are *storage* formats.  A layer that arrives in one of
them is expanded once, at construction, into the fixed-width stream every
kernel reads (``NPVQLinear``); nothing decodes prefixes on the hot path.  All
three classes share one engine: classify every position into a tier, then
gather / scatter each tier's payload by the positions of that tier.
"""

from __future__ import annotations

import struct

import torch

from .vq_packing import IndexPacking

# ---------------------------------------------------------------------------
# Shared pieces
# ---------------------------------------------------------------------------


def _header_bytes(words: list[int], device: torch.device) -> torch.Tensor:
    raw = struct.pack(f"<{len(words)}I", *[w & 0xFFFFFFFF for w in words])
    return torch.frombuffer(bytearray(raw), dtype=torch.uint8).to(device)


def _header_words(packed: torch.Tensor, count: int) -> list[int]:
    raw = bytes(packed[: 4 * count].cpu().numpy().tobytes())
    return list(struct.unpack(f"<{count}I", raw))


def _pack_narrow(values: torch.Tensor, width: int) -> torch.Tensor:
    """1- or 2-bit fields, LSB first, ``ceil(n * width / 8)`` bytes."""
    per = 8 // width
    n = values.numel()
    n_bytes = (n * width + 7) // 8
    padded = values.new_zeros(n_bytes * per)
    padded[:n] = values
    shifts = torch.arange(per, dtype=torch.int64, device=values.device) * width
    return (padded.view(n_bytes, per) << shifts).sum(dim=1).to(torch.uint8)


def _unpack_narrow(buf: torch.Tensor, width: int, n: int) -> torch.Tensor:
    per = 8 // width
    shifts = torch.arange(per, dtype=torch.int64, device=buf.device) * width
    fields = (buf.to(torch.int64).unsqueeze(1) >> shifts) & ((1 << width) - 1)
    return fields.flatten()[:n]


def _payload_nbytes(count: int, bits: int) -> int:
    return (count * bits + 7) // 8


def _pack_payload(values: torch.Tensor, bits: int) -> torch.Tensor:
    """Tier-local values as an ``IndexPacking`` stream (a 4-bit stream of odd length gets a zero nibble)."""
    if values.numel() == 0:
        return torch.zeros(0, dtype=torch.uint8, device=values.device)
    if bits == 4 and values.numel() % 2:
        values = torch.cat([values, values.new_zeros(1)])
    return IndexPacking.pack(values, bits)


def _unpack_payload(buf: torch.Tensor, bits: int, count: int) -> torch.Tensor:
    if count == 0:
        return torch.zeros(0, dtype=torch.int64, device=buf.device)
    return IndexPacking.unpack(buf, bits, count)


def _assemble(tier_of: torch.Tensor, payloads: list[tuple[torch.Tensor, int, int, int] | None]) -> torch.Tensor:
    """Indices from per-position tier numbers and per-tier ``(stream, bits, count, base)``.

    Tier ``k``'s ``j``-th payload value belongs to the ``j``-th position whose
    tier is ``k``; ``None`` marks a tier without payload (value = 0).
    """
    out = torch.zeros(tier_of.numel(), dtype=torch.int64, device=tier_of.device)
    for k, entry in enumerate(payloads):
        if entry is None:
            continue
        stream, bits, count, base = entry
        if count == 0:
            continue
        where = (tier_of == k).nonzero(as_tuple=True)[0]
        if where.numel() != count:
            raise ValueError(
                f"prefix stream names {where.numel()} indices of tier {k}, header says {count}."
            )
        out[where] = _unpack_payload(stream, bits, count) + base
    return out


def _row_offsets(tier_of: torch.Tensor, n_tiers: int, n_rows: int, n_groups: int) -> list[torch.Tensor]:
    """Per tier: int32 ``[n_rows + 1]`` cumulative count of that tier's indices before each row."""
    tier_cpu = tier_of.cpu()
    rows = torch.arange(n_rows, dtype=torch.int64).repeat_interleave(n_groups)
    counts = torch.bincount(rows * n_tiers + tier_cpu, minlength=n_rows * n_tiers).view(n_rows, n_tiers)
    out = []
    for k in range(n_tiers):
        off = torch.zeros(n_rows + 1, dtype=torch.int32)
        off[1:] = counts[:, k].cumsum(0).to(torch.int32)
        out.append(off)
    return out


def _check_rows(what: str, n_indices: int, n_rows: int, n_groups: int) -> None:
    if n_indices != n_rows * n_groups:
        raise ValueError(
            f"compute_row_offsets: n_rows*n_groups={n_rows * n_groups} != n_indices={n_indices} in header."
        )


# ---------------------------------------------------------------------------
# Two tiers, one prefix bit
# ---------------------------------------------------------------------------


class TieredIndexPacking:
    """Hot / cold prefix code (reference: neuropress/transforms/vq_packing.py:298-610).

    Buffer: ``n_indices, n_hot, cold_bits, hot_bits`` (4 x uint32), prefix
    stream (bit ``i`` = 1 when index ``i`` is cold), hot stream, cold stream.
    Indices ``< 2**hot_bits`` are hot; both streams hold the index itself.
    A 12-byte header without ``hot_bits`` (older writers) reads as ``hot_bits = 4``.
    """

    DEFAULT_HOT_BITS: int = 4
    HEADER_BYTES: int = 16
    _LEGACY_HEADER_BYTES: int = 12

    @staticmethod
    def hot_threshold(hot_bits: int) -> int:
        return 1 << hot_bits

    @staticmethod
    def pack(indices: torch.Tensor, cold_bits: int, hot_bits: int = 4) -> torch.Tensor:
        if not (IndexPacking._MIN_BITS <= cold_bits <= IndexPacking._MAX_BITS):
            raise ValueError(
                f"cold_bits must be in [{IndexPacking._MIN_BITS}, {IndexPacking._MAX_BITS}], got {cold_bits}."
            )
        if not (4 <= hot_bits <= 16):
            raise ValueError(f"hot_bits must be in [4, 16], got {hot_bits}.")
        flat = indices.flatten().to(torch.int64)
        cold = flat >= TieredIndexPacking.hot_threshold(hot_bits)
        n_hot = int((~cold).sum().item())
        return torch.cat([
            _header_bytes([flat.numel(), n_hot, cold_bits, hot_bits], flat.device),
            _pack_narrow(cold.to(torch.int64), 1),
            _pack_payload(flat[~cold], hot_bits),
            _pack_payload(flat[cold], cold_bits),
        ])  # fmt: skip

    @staticmethod
    def _parse_header(packed: torch.Tensor) -> tuple[int, int, int, int, int]:
        """``(n_indices, n_hot, cold_bits, hot_bits, header_bytes)``."""
        legacy, full = TieredIndexPacking._LEGACY_HEADER_BYTES, TieredIndexPacking.HEADER_BYTES
        if packed.numel() < legacy:
            raise ValueError(
                f"TieredIndexPacking: buffer too short ({packed.numel()} bytes, need at least {legacy})."
            )
        if packed.numel() >= full:
            n, n_hot, cold_bits, hot_bits = _header_words(packed, 4)
            if 4 <= hot_bits <= 16:
                return n, n_hot, cold_bits, hot_bits, full
        n, n_hot, cold_bits = _header_words(packed, 3)
        return n, n_hot, cold_bits, 4, legacy

    @staticmethod
    def _split(packed: torch.Tensor):
        n, n_hot, cold_bits, hot_bits, at = TieredIndexPacking._parse_header(packed)
        prefix = packed[at : at + (n + 7) // 8]
        at += (n + 7) // 8
        hot = packed[at : at + _payload_nbytes(n_hot, hot_bits)]
        at += _payload_nbytes(n_hot, hot_bits)
        cold = packed[at : at + _payload_nbytes(n - n_hot, cold_bits)]
        return n, n_hot, cold_bits, hot_bits, prefix, hot, cold

    @staticmethod
    def split_streams(packed: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, int, int]:
        """``(prefix_stream, hot_stream, cold_stream, cold_bits, hot_bits)``: views of the buffer in
        the order ``kernels.vq_linear_tiered`` takes them (the reference splits the same way at
        module construction, nn/np_vq_linear.py:644-696)."""
        _, _, cold_bits, hot_bits, prefix, hot, cold = TieredIndexPacking._split(packed)
        return prefix, hot, cold, cold_bits, hot_bits

    @staticmethod
    def unpack(packed: torch.Tensor) -> torch.Tensor:
        n, n_hot, cold_bits, hot_bits, prefix, hot, cold = TieredIndexPacking._split(packed)
        tier_of = _unpack_narrow(prefix, 1, n)
        return _assemble(tier_of, [(hot, hot_bits, n_hot, 0), (cold, cold_bits, n - n_hot, 0)])

    @staticmethod
    def compute_row_offsets(packed: torch.Tensor, n_rows: int, n_groups: int) -> tuple[torch.Tensor, torch.Tensor]:
        """``(hot_row_offsets, cold_row_offsets)``: int32 CPU tensors ``[n_rows + 1]``."""
        n, _, _, _, prefix, _, _ = TieredIndexPacking._split(packed)
        _check_rows("TieredIndexPacking", n, n_rows, n_groups)
        hot_off, cold_off = _row_offsets(_unpack_narrow(prefix, 1, n), 2, n_rows, n_groups)
        return hot_off, cold_off

    @staticmethod
    def effective_bits(n_hot: int, n_total: int, cold_bits: int, hot_bits: int = 4) -> float:
        """Average bits per index: ``1 + hot_bits * p_hot + cold_bits * (1 - p_hot)``."""
        if n_total == 0:
            return float(cold_bits)
        p_hot = n_hot / n_total
        return 1.0 + hot_bits * p_hot + cold_bits * (1.0 - p_hot)


# ---------------------------------------------------------------------------
# Two to four tiers, cascaded prefix bits
# ---------------------------------------------------------------------------


class NTieredIndexPacking:
    """Cascaded binary splitting (reference: neuropress/transforms/vq_packing.py:612-1034).

    ``tier_bits = [b0 < b1 < ...]``: tier ``k`` holds indices in
    ``[2**b(k-1), 2**bk)`` (tier 0 from 0) as ``index - 2**b(k-1)`` in ``bk``
    bits; the last tier takes everything from ``2**b(D-2)`` up.  Buffer:
    ``magic, n_indices, D`` then ``(count_k, bits_k)`` per tier (uint32 each),
    prefix streams 0..D-2 (stream ``k`` has one bit per index not claimed by
    tiers ``< k``; 0 = "tier k"), then the D payload streams.
    """

    MAGIC: int = 0x4E565154
    MIN_TIERS: int = 2
    MAX_TIERS: int = 4

    @staticmethod
    def tier_thresholds(tier_bits: list[int]) -> list[int]:
        return [1 << b for b in tier_bits]

    @staticmethod
    def _validate_tier_bits(tier_bits: list[int]) -> None:
        d = len(tier_bits)
        if not (NTieredIndexPacking.MIN_TIERS <= d <= NTieredIndexPacking.MAX_TIERS):
            raise ValueError(
                f"tier_bits length must be in [{NTieredIndexPacking.MIN_TIERS}, "
                f"{NTieredIndexPacking.MAX_TIERS}], got {d}."
            )
        for i, b in enumerate(tier_bits):
            if not (IndexPacking._MIN_BITS <= b <= IndexPacking._MAX_BITS):
                raise ValueError(
                    f"tier_bits[{i}]={b} out of range [{IndexPacking._MIN_BITS}, {IndexPacking._MAX_BITS}]."
                )
        for i in range(1, d):
            if tier_bits[i] <= tier_bits[i - 1]:
                raise ValueError(
                    f"tier_bits must be strictly increasing, got tier_bits[{i - 1}]={tier_bits[i - 1]}, "
                    f"tier_bits[{i}]={tier_bits[i]}."
                )

    @staticmethod
    def _tier_of_values(flat: torch.Tensor, tier_bits: list[int]) -> torch.Tensor:
        bounds = torch.tensor([1 << b for b in tier_bits[:-1]], dtype=torch.int64, device=flat.device)
        return torch.bucketize(flat, bounds, right=True)  # number of thresholds <= value

    @staticmethod
    def pack(indices: torch.Tensor, tier_bits: list[int]) -> torch.Tensor:
        NTieredIndexPacking._validate_tier_bits(tier_bits)
        flat = indices.flatten().to(torch.int64)
        d = len(tier_bits)
        tier_of = NTieredIndexPacking._tier_of_values(flat, tier_bits)
        words = [NTieredIndexPacking.MAGIC, flat.numel(), d]
        prefixes, payloads = [], []
        alive = tier_of  # tiers of the indices still unclaimed, in order
        for k in range(d):
            members = flat[tier_of == k]
            words += [members.numel(), tier_bits[k]]
            payloads.append(_pack_payload(members - (0 if k == 0 else 1 << tier_bits[k - 1]), tier_bits[k]))
            if k < d - 1:
                prefixes.append(_pack_narrow((alive != k).to(torch.int64), 1))
                alive = alive[alive != k]
        return torch.cat([_header_bytes(words, flat.device), *prefixes, *payloads])

    @staticmethod
    def _parse_header(packed: torch.Tensor) -> tuple[int, int, list[int], list[int], int]:
        """``(n_indices, n_tiers, tier_counts, tier_bits, header_bytes)``."""
        if packed.numel() < 12:
            raise ValueError(
                f"NTieredIndexPacking: buffer too short ({packed.numel()} bytes, need at least 12)."
            )
        magic, n, d = _header_words(packed, 3)
        if magic != NTieredIndexPacking.MAGIC:
            raise ValueError(
                f"NTieredIndexPacking: bad magic 0x{magic:08X}, expected 0x{NTieredIndexPacking.MAGIC:08X}."
            )
        size = 12 + 8 * d
        if packed.numel() < size:
            raise ValueError(f"NTieredIndexPacking: buffer too short for {d} tiers ({packed.numel()} < {size}).")
        pairs = _header_words(packed, 3 + 2 * d)[3:]
        return n, d, pairs[0::2], pairs[1::2], size

    @staticmethod
    def split_streams(packed: torch.Tensor) -> tuple[list[torch.Tensor], list[torch.Tensor], list[int]]:
        """``(prefix_streams, tier_streams, tier_bits)``: views of the buffer in the order
        ``kernels.vq_linear_ntier`` takes them."""
        n, d, counts, bits, at = NTieredIndexPacking._parse_header(packed)
        prefixes, alive_n = [], n
        for k in range(d - 1):
            nb = (alive_n + 7) // 8
            prefixes.append(packed[at : at + nb])
            at += nb
            alive_n -= counts[k]
        tiers = []
        for k in range(d):
            nb = _payload_nbytes(counts[k], bits[k])
            tiers.append(packed[at : at + nb])
            at += nb
        return prefixes, tiers, list(bits)

    @staticmethod
    def _tiers_and_payloads(packed: torch.Tensor):
        n, d, counts, bits, at = NTieredIndexPacking._parse_header(packed)
        prefix_streams = []
        alive_n = n
        for k in range(d - 1):
            nb = (alive_n + 7) // 8
            prefix_streams.append((packed[at : at + nb], alive_n))
            at += nb
            alive_n -= counts[k]
        payloads = []
        for k in range(d):
            nb = _payload_nbytes(counts[k], bits[k])
            payloads.append((packed[at : at + nb], bits[k], counts[k], 0 if k == 0 else 1 << bits[k - 1]))
            at += nb
        tier_of = torch.full((n,), d - 1, dtype=torch.int64, device=packed.device)
        alive = torch.arange(n, dtype=torch.int64, device=packed.device)
        for k, (stream, count) in enumerate(prefix_streams):
            rest = _unpack_narrow(stream, 1, count).bool()
            tier_of[alive[~rest]] = k
            alive = alive[rest]
        return n, d, tier_of, payloads

    @staticmethod
    def unpack(packed: torch.Tensor) -> torch.Tensor:
        _, _, tier_of, payloads = NTieredIndexPacking._tiers_and_payloads(packed)
        return _assemble(tier_of, payloads)

    @staticmethod
    def compute_row_offsets(packed: torch.Tensor, n_rows: int, n_groups: int) -> list[torch.Tensor]:
        """One int32 CPU tensor ``[n_rows + 1]`` per tier."""
        n, d, tier_of, _ = NTieredIndexPacking._tiers_and_payloads(packed)
        _check_rows("NTieredIndexPacking", n, n_rows, n_groups)
        return _row_offsets(tier_of, d, n_rows, n_groups)

    @staticmethod
    def effective_bits(tier_counts: list[int], tier_bits: list[int]) -> float:
        """Average bits per index, prefix bits included."""
        total = sum(tier_counts)
        if total == 0:
            return float(tier_bits[-1])
        bits = 0
        alive = total
        for k, (count, width) in enumerate(zip(tier_counts, tier_bits)):
            if k < len(tier_bits) - 1:
                bits += alive  # one prefix bit for every index still unclaimed at level k
                alive -= count
            bits += count * width
        return bits / total

    @staticmethod
    def is_ntier_buffer(packed: torch.Tensor) -> bool:
        return packed.numel() >= 4 and _header_words(packed, 1)[0] == NTieredIndexPacking.MAGIC


# ---------------------------------------------------------------------------
# Four classes, flat 2-bit prefix, no payload for index 0
# ---------------------------------------------------------------------------


class ZeroEscapePacking:
    """Zero-escape code (reference: neuropress/transforms/vq_packing.py:1037-1384).

    Class per index (2 bits): 0 = index 0, 1 = 1..16 (4-bit payload, index - 1),
    2 = 17..256 (8-bit payload, index - 17), 3 = the rest (``cold_bits`` payload,
    index - 257).  Buffer: ``magic, n_indices, cold_bits, n_zero, n_hot, n_warm``
    (6 x uint32), class stream, hot, warm and cold payload streams.
    """

    MAGIC: int = 0x5A455343
    HEADER_BYTES: int = 24
    TIER_0_MAX: int = 1
    TIER_1_MAX: int = 17
    TIER_2_MAX: int = 257
    _BASES = (0, 1, 17, 257)

    @staticmethod
    def pack(indices: torch.Tensor, cold_bits: int) -> torch.Tensor:
        if not (IndexPacking._MIN_BITS <= cold_bits <= IndexPacking._MAX_BITS):
            raise ValueError(
                f"cold_bits must be in [{IndexPacking._MIN_BITS}, {IndexPacking._MAX_BITS}], got {cold_bits}."
            )
        flat = indices.flatten().to(torch.int64)
        bounds = torch.tensor(ZeroEscapePacking._BASES[1:], dtype=torch.int64, device=flat.device)
        cls = torch.bucketize(flat, bounds, right=True)
        members = [flat[cls == k] for k in range(4)]
        return torch.cat([
            _header_bytes([ZeroEscapePacking.MAGIC, flat.numel(), cold_bits, members[0].numel(),
                           members[1].numel(), members[2].numel()], flat.device),
            _pack_narrow(cls, 2),
            _pack_payload(members[1] - 1, 4),
            _pack_payload(members[2] - 17, 8),
            _pack_payload(members[3] - 257, cold_bits),
        ])  # fmt: skip

    @staticmethod
    def _parse_header(packed: torch.Tensor) -> tuple[int, int, int, int, int, int]:
        """``(n_indices, cold_bits, n_zero, n_hot, n_warm, header_bytes)``."""
        size = ZeroEscapePacking.HEADER_BYTES
        if packed.numel() < size:
            raise ValueError(
                f"ZeroEscapePacking: buffer too short ({packed.numel()} bytes, need at least {size})."
            )
        magic, n, cold_bits, n_zero, n_hot, n_warm = _header_words(packed, 6)
        if magic != ZeroEscapePacking.MAGIC:
            raise ValueError(
                f"ZeroEscapePacking: bad magic 0x{magic:08X}, expected 0x{ZeroEscapePacking.MAGIC:08X}."
            )
        return n, cold_bits, n_zero, n_hot, n_warm, size

    @staticmethod
    def split_streams(packed: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, int]:
        """``(class_stream, hot_stream, warm_stream, cold_stream, cold_bits)``: views of the buffer in
        the order ``kernels.vq_linear_zero_escape`` takes them."""
        n, cold_bits, n_zero, n_hot, n_warm, at = ZeroEscapePacking._parse_header(packed)
        out = []
        for nb in ((2 * n + 7) // 8, _payload_nbytes(n_hot, 4), _payload_nbytes(n_warm, 8),
                   _payload_nbytes(n - n_zero - n_hot - n_warm, cold_bits)):
            out.append(packed[at : at + nb])
            at += nb
        return out[0], out[1], out[2], out[3], cold_bits

    @staticmethod
    def _classes_and_payloads(packed: torch.Tensor):
        n, cold_bits, n_zero, n_hot, n_warm, at = ZeroEscapePacking._parse_header(packed)
        n_cold = n - n_zero - n_hot - n_warm
        nb = (2 * n + 7) // 8
        cls = _unpack_narrow(packed[at : at + nb], 2, n)
        at += nb
        payloads: list = [None]
        for count, bits, base in ((n_hot, 4, 1), (n_warm, 8, 17), (n_cold, cold_bits, 257)):
            nb = _payload_nbytes(count, bits)
            payloads.append((packed[at : at + nb], bits, count, base))
            at += nb
        return n, cls, payloads

    @staticmethod
    def unpack(packed: torch.Tensor) -> torch.Tensor:
        _, cls, payloads = ZeroEscapePacking._classes_and_payloads(packed)
        return _assemble(cls, payloads)

    @staticmethod
    def compute_row_offsets(packed: torch.Tensor, n_rows: int, n_groups: int) -> list[torch.Tensor]:
        """Four int32 CPU tensors ``[n_rows + 1]``: zero, hot, warm, cold."""
        n, cls, _ = ZeroEscapePacking._classes_and_payloads(packed)
        _check_rows("ZeroEscapePacking", n, n_rows, n_groups)
        return _row_offsets(cls, 4, n_rows, n_groups)

    @staticmethod
    def effective_bits(n_zero: int, n_hot: int, n_warm: int, n_cold: int, cold_bits: int) -> float:
        """Average bits per index: 2 prefix bits plus 0 / 4 / 8 / ``cold_bits`` of payload."""
        total = n_zero + n_hot + n_warm + n_cold
        if total == 0:
            return float(cold_bits)
        return (2 * total + 4 * n_hot + 8 * n_warm + cold_bits * n_cold) / total

    @staticmethod
    def is_zero_escape_buffer(packed: torch.Tensor) -> bool:
        return packed.numel() >= 4 and _header_words(packed, 1)[0] == ZeroEscapePacking.MAGIC


def decode_to_flat(
    packed: torch.Tensor, *, use_tiered: bool = False, tier_bits: list[int] | None = None, zero_escape: bool = False
) -> torch.Tensor:
    """Indices (int64) of a buffer in the format the three flags name (same precedence as the
    reference: zero-escape, then n-tier, then two-tier; neuropress/transforms/vq.py:220-247)."""
    if zero_escape:
        return ZeroEscapePacking.unpack(packed)
    if tier_bits is not None:
        return NTieredIndexPacking.unpack(packed)
    if use_tiered:
        return TieredIndexPacking.unpack(packed)
    raise ValueError("decode_to_flat: no entropy-coded format named")
