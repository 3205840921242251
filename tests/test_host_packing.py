"""IndexPacking / BitPacking host code: mirrors the reference's packing tests
(tests/transforms/test_vq_packing.py, test_vq_packing_extended.py) and checks the
window-based implementation against the big-integer golden streams."""

import math
from pathlib import Path

import numpy as np
import pytest
import torch

from neuropress_amd.nn.np_linear import _pack_u8, _unpack_u8
from neuropress_amd.t2n.packing import BitPacking, BitPacking4
from neuropress_amd.transforms.vq_packing import IndexPacking

G = np.load(Path(__file__).parent / "golden" / "vectors.npz")


@pytest.mark.parametrize("bits", range(4, 21))
def test_matches_bigint_stream(bits):
    idx = torch.from_numpy(G[f"stream_b{bits}/idx"])
    packed = torch.from_numpy(G[f"stream_b{bits}/packed"].copy())
    assert torch.equal(IndexPacking.pack(idx, bits), packed)
    assert torch.equal(IndexPacking.unpack(packed, bits, idx.numel()), idx)


@pytest.mark.parametrize("bits", range(4, 17))
def test_pack_unpack_roundtrip(bits):
    torch.manual_seed(bits)
    idx = torch.randint(0, 1 << bits, (128,), dtype=torch.int64)
    packed = IndexPacking.pack(idx, bits)
    assert packed.dtype == torch.uint8 and packed.numel() == math.ceil(128 * bits / 8)
    out = IndexPacking.unpack(packed, bits, 128)
    assert out.dtype == torch.int64 and torch.equal(out, idx)


@pytest.mark.parametrize("bits", [5, 6, 7, 9, 10, 12, 14])
def test_odd_counts(bits):
    for n in [1, 3, 7, 13, 33, 99]:
        idx = torch.randint(0, 1 << bits, (n,), dtype=torch.int64)
        assert torch.equal(IndexPacking.unpack(IndexPacking.pack(idx, bits), bits, n), idx)


def test_4bit_lsb_first_and_odd_count():
    assert IndexPacking.pack(torch.tensor([3, 11]), 4)[0].item() == 3 | (11 << 4)
    with pytest.raises(ValueError, match="even"):
        IndexPacking.pack(torch.tensor([0, 1, 2]), 4)


def test_invalid_bits():
    with pytest.raises(ValueError, match="bits"):
        IndexPacking.pack(torch.tensor([0]), 2)
    with pytest.raises(ValueError, match="bits"):
        IndexPacking.unpack(torch.zeros(4, dtype=torch.uint8), 21, 1)


def test_bits_for():
    assert [IndexPacking.bits_for(n) for n in (2, 16, 17, 256, 257, 4096, 4097, 65536)] == [4, 4, 5, 8, 9, 12, 13, 16]
    for bad in (0, 1, (1 << 20) + 1):
        with pytest.raises(ValueError):
            IndexPacking.bits_for(bad)


@pytest.mark.parametrize("nbits", [1, 2, 4, 8])
def test_bitpacking_roundtrip_and_layout(nbits):
    vals = torch.randint(0, 1 << nbits, (5, 64), dtype=torch.int64).to(torch.uint8)
    bp = BitPacking(nbits)
    packed = bp.compress(vals)
    assert packed.shape == (5, 64 * nbits // 8)
    assert torch.equal(bp.decompress(packed), vals)
    assert torch.equal(_unpack_u8(_pack_u8(vals, nbits), nbits), vals)


def test_bitpacking4_low_nibble_first():
    # neuropress/t2n/packing.py:10-14: packed = (x[2i] & 0xF) | (x[2i+1] << 4)
    assert BitPacking4.compress(torch.tensor([[3, 11]], dtype=torch.uint8)).item() == 0xB3
    with pytest.raises(ValueError):
        BitPacking4.compress(torch.zeros(1, 3, dtype=torch.uint8))
    for name in ("q4_sym", "q4_asym"):
        assert torch.equal(BitPacking4.compress(torch.from_numpy(G[f"{name}/codes"])), torch.from_numpy(G[f"{name}/blob"]))
