"""Prefix-coded index formats (two-tier, n-tier, zero-escape): host classes vs the C oracle,
hand-assembled buffers, an independent big-integer packer, and the assertions the reference's
own tests make (tests/transforms/test_tiered_packing.py, test_ntier_packing.py,
test_zero_escape_packing.py: round trips, header fields, byte-count formulas, effective bits).

The reference holds no byte-level vectors for these formats; the hand-assembled buffers below are
written out field by field from the format descriptions
(neuropress/transforms/vq_packing.py:298-332, 612-646, 1037-1075)."""

import math
import struct

import numpy as np
import pytest
import torch

from neuropress_amd.transforms.vq_packing import (
    IndexPacking,
    NTieredIndexPacking,
    TieredIndexPacking,
    ZeroEscapePacking,
)
from oracle import oracle


def _bits_le(fields):
    """Independent packer: (value, width) fields concatenated LSB first through one big integer."""
    acc, pos = 0, 0
    for v, w in fields:
        assert 0 <= v < (1 << w)
        acc |= v << pos
        pos += w
    return acc.to_bytes((pos + 7) // 8, "little")


def _zipf(n, nc, seed):
    g = torch.Generator().manual_seed(seed)
    p = 1.0 / torch.arange(1, nc + 1, dtype=torch.float64) ** 1.1
    return torch.multinomial(p / p.sum(), n, replacement=True, generator=g)


def _t(b: bytes) -> torch.Tensor:
    return torch.frombuffer(bytearray(b), dtype=torch.uint8)


# ----------------------------------------------------------------- hand-assembled buffers ---


def test_tiered_hand_assembled_buffer():
    idx = [3, 200, 15, 16, 0, 77, 9]  # hot (< 16): 3, 15, 0, 9; cold: 200, 16, 77
    want = (struct.pack("<4I", 7, 4, 8, 4)
            + _bits_le([(0, 1), (1, 1), (0, 1), (1, 1), (0, 1), (1, 1), (0, 1)])
            + _bits_le([(3, 4), (15, 4), (0, 4), (9, 4)])
            + _bits_le([(200, 8), (16, 8), (77, 8)]))
    got = TieredIndexPacking.pack(torch.tensor(idx), cold_bits=8)
    assert bytes(got.numpy().tobytes()) == want
    assert TieredIndexPacking.unpack(_t(want)).tolist() == idx
    assert oracle.entropy_unpack("tiered", np.frombuffer(want, np.uint8)).tolist() == idx


def test_tiered_legacy_header_reads_as_four_hot_bits():
    idx = [1, 40, 2]
    legacy = (struct.pack("<3I", 3, 2, 8) + _bits_le([(0, 1), (1, 1), (0, 1)])
              + _bits_le([(1, 4), (2, 4)]) + _bits_le([(40, 8)]))
    assert TieredIndexPacking._parse_header(_t(legacy)) == (3, 2, 8, 4, 12)
    assert TieredIndexPacking.unpack(_t(legacy)).tolist() == idx
    assert oracle.entropy_unpack("tiered", np.frombuffer(legacy, np.uint8)).tolist() == idx


def test_ntier_hand_assembled_buffer():
    tier_bits = [4, 8, 12]  # tier 0: [0, 16); tier 1: [16, 256) stored - 16; tier 2: >= 256 stored - 256
    idx = [5, 300, 16, 255, 0, 4095, 17]
    tiers = [0, 2, 1, 1, 0, 2, 1]
    level0 = [(int(t != 0), 1) for t in tiers]
    level1 = [(int(t != 1), 1) for t in tiers if t != 0]
    want = (struct.pack("<3I", 0x4E565154, 7, 3) + struct.pack("<6I", 2, 4, 3, 8, 2, 12)
            + _bits_le(level0) + _bits_le(level1)
            + _bits_le([(5, 4), (0, 4)])
            + _bits_le([(0, 8), (239, 8), (1, 8)])
            + _bits_le([(44, 12), (3839, 12)]))
    got = NTieredIndexPacking.pack(torch.tensor(idx), tier_bits)
    assert bytes(got.numpy().tobytes()) == want
    assert NTieredIndexPacking.unpack(_t(want)).tolist() == idx
    assert oracle.entropy_unpack("ntier", np.frombuffer(want, np.uint8)).tolist() == idx
    assert NTieredIndexPacking.is_ntier_buffer(got) and not ZeroEscapePacking.is_zero_escape_buffer(got)


def test_zero_escape_hand_assembled_buffer():
    idx = [0, 1, 16, 17, 256, 257, 0, 1000, 5]
    cls = [0, 1, 1, 2, 2, 3, 0, 3, 1]
    want = (struct.pack("<6I", 0x5A455343, 9, 10, 2, 3, 2)
            + _bits_le([(c, 2) for c in cls])
            + _bits_le([(0, 4), (15, 4), (4, 4)])      # 1, 16, 5 stored minus 1 (odd count: zero nibble pads the byte)
            + _bits_le([(0, 8), (239, 8)])             # 17, 256 stored minus 17
            + _bits_le([(0, 10), (743, 10)]))          # 257, 1000 stored minus 257
    got = ZeroEscapePacking.pack(torch.tensor(idx), cold_bits=10)
    assert bytes(got.numpy().tobytes()) == want
    assert ZeroEscapePacking.unpack(_t(want)).tolist() == idx
    assert oracle.entropy_unpack("zero_escape", np.frombuffer(want, np.uint8)).tolist() == idx
    assert ZeroEscapePacking.is_zero_escape_buffer(got) and not NTieredIndexPacking.is_ntier_buffer(got)


# ------------------------------------------------------------------------- round trips ---


@pytest.mark.parametrize("cold_bits,hot_bits", [(4, 4), (8, 4), (12, 4), (16, 8), (17, 8), (20, 16)])
@pytest.mark.parametrize("n", [0, 1, 2, 7, 33, 1000])
def test_tiered_round_trip_matches_oracle(cold_bits, hot_bits, n):
    idx = _zipf(n, 1 << cold_bits, 100 + n) if n else torch.zeros(0, dtype=torch.int64)
    buf = TieredIndexPacking.pack(idx, cold_bits, hot_bits)
    assert buf.dtype == torch.uint8
    assert torch.equal(TieredIndexPacking.unpack(buf), idx)
    assert np.array_equal(oracle.entropy_unpack("tiered", buf.numpy()), idx.numpy())
    n_hot = int((idx < (1 << hot_bits)).sum())
    # byte count = header + prefix + hot + cold (reference: tests/transforms/test_tiered_packing.py:278-296)
    assert buf.numel() == 16 + (n + 7) // 8 + math.ceil(n_hot * hot_bits / 8) + math.ceil((n - n_hot) * cold_bits / 8)
    assert struct.unpack("<4I", bytes(buf[:16].numpy().tobytes())) == (n, n_hot, cold_bits, hot_bits)


@pytest.mark.parametrize("tier_bits", [[4, 8], [4, 12], [4, 8, 12], [4, 8, 12, 17], [5, 9, 16], [8, 20]])
@pytest.mark.parametrize("n", [0, 1, 5, 64, 777])
def test_ntier_round_trip_matches_oracle(tier_bits, n):
    idx = _zipf(n, 1 << tier_bits[-1], 200 + n) if n else torch.zeros(0, dtype=torch.int64)
    buf = NTieredIndexPacking.pack(idx, tier_bits)
    assert torch.equal(NTieredIndexPacking.unpack(buf), idx)
    assert np.array_equal(oracle.entropy_unpack("ntier", buf.numpy()), idx.numpy())
    n_, d, counts, bits, hdr = NTieredIndexPacking._parse_header(buf)
    assert (n_, d, bits, hdr) == (n, len(tier_bits), tier_bits, 12 + 8 * len(tier_bits)) and sum(counts) == n
    alive, size = n, hdr
    for k in range(d - 1):
        size += (alive + 7) // 8
        alive -= counts[k]
    size += sum(math.ceil(c * b / 8) for c, b in zip(counts, bits))
    assert buf.numel() == size


@pytest.mark.parametrize("cold_bits", [9, 12, 16, 17, 20])
@pytest.mark.parametrize("n", [0, 1, 3, 100, 1001])
def test_zero_escape_round_trip_matches_oracle(cold_bits, n):
    nc = min((1 << cold_bits) + 257, 1 << 20)
    idx = _zipf(n, nc, 300 + n) if n else torch.zeros(0, dtype=torch.int64)
    buf = ZeroEscapePacking.pack(idx, cold_bits)
    assert torch.equal(ZeroEscapePacking.unpack(buf), idx)
    assert np.array_equal(oracle.entropy_unpack("zero_escape", buf.numpy()), idx.numpy())
    n_, cb, n_zero, n_hot, n_warm, hdr = ZeroEscapePacking._parse_header(buf)
    assert (n_, cb, hdr) == (n, cold_bits, 24)
    assert n_zero == int((idx == 0).sum()) and n_hot == int(((idx >= 1) & (idx <= 16)).sum())
    assert n_warm == int(((idx >= 17) & (idx <= 256)).sum())
    n_cold = n - n_zero - n_hot - n_warm
    assert buf.numel() == 24 + (2 * n + 7) // 8 + math.ceil(n_hot / 2) + n_warm + math.ceil(n_cold * cold_bits / 8)


def test_extreme_populations_round_trip():
    for idx in (torch.zeros(50, dtype=torch.int64), torch.full((51,), 15), torch.full((49,), 65535),
                torch.arange(4096), torch.tensor([0, 65535] * 9)):
        assert torch.equal(TieredIndexPacking.unpack(TieredIndexPacking.pack(idx, 16)), idx)
        assert torch.equal(NTieredIndexPacking.unpack(NTieredIndexPacking.pack(idx, [4, 8, 16])), idx)
        assert torch.equal(ZeroEscapePacking.unpack(ZeroEscapePacking.pack(idx, 16)), idx)


# ---------------------------------------------------------------- errors, offsets, bits ---


def test_argument_errors_match_the_reference_messages():
    idx = torch.arange(8)
    with pytest.raises(ValueError, match=r"cold_bits must be in \[4, 20\], got 3"):
        TieredIndexPacking.pack(idx, 3)
    with pytest.raises(ValueError, match=r"hot_bits must be in \[4, 16\], got 2"):
        TieredIndexPacking.pack(idx, 8, hot_bits=2)
    with pytest.raises(ValueError, match="buffer too short"):
        TieredIndexPacking.unpack(torch.zeros(5, dtype=torch.uint8))
    with pytest.raises(ValueError, match="tier_bits length must be in"):
        NTieredIndexPacking.pack(idx, [4])
    with pytest.raises(ValueError, match="strictly increasing"):
        NTieredIndexPacking.pack(idx, [8, 8])
    with pytest.raises(ValueError, match="out of range"):
        NTieredIndexPacking.pack(idx, [2, 8])
    with pytest.raises(ValueError, match="bad magic"):
        NTieredIndexPacking.unpack(torch.zeros(40, dtype=torch.uint8))
    with pytest.raises(ValueError, match="bad magic"):
        ZeroEscapePacking.unpack(torch.zeros(40, dtype=torch.uint8))
    with pytest.raises(ValueError, match=r"cold_bits must be in"):
        ZeroEscapePacking.pack(idx, 21)


def test_row_offsets_are_cumulative_tier_counts_per_row():
    n_rows, n_groups = 6, 10
    idx = _zipf(n_rows * n_groups, 4096, 7)
    rows = idx.view(n_rows, n_groups)

    def cum(mask):
        return [0] + mask.sum(1).cumsum(0).tolist()

    hot, cold = TieredIndexPacking.compute_row_offsets(TieredIndexPacking.pack(idx, 12), n_rows, n_groups)
    assert hot.dtype == torch.int32 and hot.tolist() == cum(rows < 16) and cold.tolist() == cum(rows >= 16)
    offs = NTieredIndexPacking.compute_row_offsets(NTieredIndexPacking.pack(idx, [4, 8, 12]), n_rows, n_groups)
    assert [o.tolist() for o in offs] == [cum(rows < 16), cum((rows >= 16) & (rows < 256)), cum(rows >= 256)]
    offs = ZeroEscapePacking.compute_row_offsets(ZeroEscapePacking.pack(idx, 12), n_rows, n_groups)
    assert [o.tolist() for o in offs] == [cum(rows == 0), cum((rows >= 1) & (rows <= 16)),
                                          cum((rows >= 17) & (rows <= 256)), cum(rows >= 257)]
    with pytest.raises(ValueError, match="n_rows\\*n_groups"):
        TieredIndexPacking.compute_row_offsets(TieredIndexPacking.pack(idx, 12), n_rows, n_groups + 1)


def test_effective_bits_values():
    # the reference's own expectations (tests/transforms/test_tiered_packing.py:115-131)
    assert abs(TieredIndexPacking.effective_bits(100, 100, 8) - 5.0) < 1e-9
    assert abs(TieredIndexPacking.effective_bits(0, 100, 8) - 9.0) < 1e-9
    assert abs(TieredIndexPacking.effective_bits(50, 100, 8) - 7.0) < 1e-9
    assert TieredIndexPacking.effective_bits(0, 0, 8) == 8.0
    # n-tier: prefix bits = 1 per index at level 0 + 1 per index left at level 1
    assert abs(NTieredIndexPacking.effective_bits([50, 30, 20], [4, 8, 12]) - (1 + 0.5 + 2.0 + 2.4 + 2.4)) < 1e-9
    assert abs(ZeroEscapePacking.effective_bits(10, 20, 30, 40, 16) - (2 + (80 + 240 + 640) / 100)) < 1e-9
    # measured size agrees with the formula
    idx = _zipf(20000, 65536, 5)
    buf = NTieredIndexPacking.pack(idx, [4, 8, 16])
    _, _, counts, bits, hdr = NTieredIndexPacking._parse_header(buf)
    assert abs((buf.numel() - hdr) * 8 / idx.numel() - NTieredIndexPacking.effective_bits(counts, bits)) < 0.01
    assert buf.numel() < IndexPacking.pack(idx, 16).numel()  # the skewed stream is shorter than fixed width
