"""Property tests (hypothesis) of the index wire format and the slice-list builder: three
independent implementations -- Python big integers, the host packing code, the C oracle --
must agree on arbitrary inputs, and the slice-list blob must always decode to its input."""

import ctypes

import numpy as np
import torch
from hypothesis import given, settings
from hypothesis import strategies as st

from neuropress_amd import _lib
from neuropress_amd.transforms.vq_packing import IndexPacking
from tests import cases


def _bigint_pack(idx: list[int], bits: int) -> bytes:
    acc = 0
    for i, v in enumerate(idx):
        acc |= v << (i * bits)
    return acc.to_bytes((len(idx) * bits + 7) // 8, "little")


@st.composite
def _index_lists(draw):
    bits = draw(st.integers(4, 20))
    n = draw(st.integers(1, 70))
    if bits == 4 and n % 2:
        n += 1  # the 4-bit packer wants whole bytes, as the reference's does
    idx = draw(st.lists(st.integers(0, (1 << bits) - 1), min_size=n, max_size=n))
    return bits, idx


@settings(max_examples=150, deadline=None)
@given(_index_lists())
def test_three_packers_agree(oracle_lib, case):
    bits, idx = case
    want = np.frombuffer(_bigint_pack(idx, bits), dtype=np.uint8)
    t = torch.tensor(idx, dtype=torch.int64)
    host = IndexPacking.pack(t, bits).numpy()
    assert np.array_equal(host, want)
    assert np.array_equal(oracle_lib.pack_indices(np.asarray(idx, dtype=np.int64), bits), want)
    assert torch.equal(IndexPacking.unpack(torch.from_numpy(want.copy()), bits, len(idx)), t)
    assert np.array_equal(oracle_lib.unpack_indices(want, bits, len(idx)), np.asarray(idx, dtype=np.int64))


@settings(max_examples=40, deadline=None)
@given(
    n=st.integers(1, 150),
    groups=st.integers(1, 40),
    nc=st.integers(2, 30000),
    target=st.sampled_from([1, 8, 256]),
    seed=st.integers(0, 2**31 - 1),
    skew=st.booleans(),
)
def test_slice_lists_always_decode_to_their_input(n, groups, nc, target, seed, skew):
    bits = IndexPacking.bits_for(nc)
    g = cases.gen(seed)
    count = n * groups
    if bits == 4 and count % 2:
        return
    idx = torch.randint(0, nc, (count,), generator=g)
    if skew:  # most indices in the first few codebook rows
        idx = torch.where(torch.rand(count, generator=g) < 0.8, idx % min(nc, 7), idx)
    packed = IndexPacking.pack(idx, bits)
    size = ctypes.c_int64(0)
    args = (packed.data_ptr(), packed.numel(), bits, n, groups * 8, 8, nc, target)
    _lib.call("npamd_vq_sliced_build", *args, None, 0, ctypes.byref(size))
    blob = torch.zeros(size.value, dtype=torch.uint8)
    _lib.call("npamd_vq_sliced_build", *args, blob.data_ptr(), blob.numel(), ctypes.byref(size))
    _lib.call("npamd_vq_sliced_check", blob.data_ptr(), blob.numel())
    dec, info = cases.decode_sliced_blob(blob.numpy())
    assert np.array_equal(dec, idx.reshape(n, groups).numpy())
    assert (info["hits"] == 1).all() and (info["writes"] == 1).all()


@st.composite
def _skewed_indices(draw):
    """Index lists the prefix codes are meant for: mostly small values, a few anywhere in range."""
    top_bits = draw(st.integers(9, 20))
    n = draw(st.integers(0, 90))
    small = st.integers(0, 300)
    anywhere = st.integers(0, (1 << top_bits) - 1)
    return top_bits, draw(st.lists(st.one_of(small, small, anywhere), min_size=n, max_size=n))


@settings(max_examples=120, deadline=None)
@given(_skewed_indices(), st.sampled_from([4, 6, 8]), st.integers(0, 2))
def test_prefix_coded_formats_round_trip_and_agree_with_the_oracle(oracle_lib, case, hot_bits, extra_tiers):
    """pack -> unpack is the identity for all three prefix-coded formats, on the host classes and
    through the oracle's sequential decoders, and the per-row tier counts add up."""
    from neuropress_amd.transforms.vq_packing import NTieredIndexPacking, TieredIndexPacking, ZeroEscapePacking
    from oracle import oracle as orc

    top_bits, idx = case
    t = torch.tensor(idx, dtype=torch.int64)
    tier_bits = sorted({hot_bits, *[hot_bits + 3 * (i + 1) for i in range(extra_tiers)], top_bits})
    if len(tier_bits) < 2:
        tier_bits = [4, top_bits]
    for kind, buf, unpack in (
        ("tiered", TieredIndexPacking.pack(t, top_bits, hot_bits), TieredIndexPacking.unpack),
        ("ntier", NTieredIndexPacking.pack(t, tier_bits), NTieredIndexPacking.unpack),
        ("zero_escape", ZeroEscapePacking.pack(t, top_bits), ZeroEscapePacking.unpack),
    ):
        assert unpack(buf).tolist() == idx, kind
        assert orc.entropy_unpack(kind, buf.numpy()).tolist() == idx, kind
    if idx:
        offs = NTieredIndexPacking.compute_row_offsets(NTieredIndexPacking.pack(t, tier_bits), 1, len(idx))
        assert sum(int(o[1]) for o in offs) == len(idx)
