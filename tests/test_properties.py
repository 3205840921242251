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
