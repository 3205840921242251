"""Slice-list form of the VQ indices: host builder, checker and layout (no GPU needed).

The builder is pinned by an independent numpy reader of the layout
(``cases.decode_sliced_blob``): the blob must decode back to exactly the index
matrix it was built from, with every (row, group) filed once and every
(partial vector, row) cell written once.
"""

import ctypes

import numpy as np
import pytest
import torch

from neuropress_amd import _lib
from neuropress_amd.transforms.vq_packing import IndexPacking
from tests import cases


def _build(packed: torch.Tensor, bits, n, k, nc, target=256, vl=8):
    size = ctypes.c_int64(0)
    args = (packed.data_ptr(), packed.numel(), bits, n, k, vl, nc, target)
    _lib.call("npamd_vq_sliced_build", *args, None, 0, ctypes.byref(size))
    blob = torch.zeros(size.value, dtype=torch.uint8)
    _lib.call("npamd_vq_sliced_build", *args, blob.data_ptr(), blob.numel(), ctypes.byref(size))
    assert size.value == blob.numel()
    return blob


def _layer(seed, n, k, nc, bits=None, zipf=False):
    g = cases.gen(seed)
    bits = bits or IndexPacking.bits_for(nc)
    count = n * (k // 8)
    idx = cases.zipf_indices(g, nc, count) if zipf else torch.randint(0, nc, (count,), generator=g)
    return idx.reshape(n, k // 8), IndexPacking.pack(idx, bits), bits


@pytest.mark.parametrize(
    "n,k,nc,bits,zipf",
    [
        (72, 96, 300, None, False),  # one slice, one workgroup row block
        (130, 8, 9000, None, False),  # two slices, a single group
        (1000, 64, 20000, None, False),  # last slice shorter than 4096 rows
        (1100, 256, 65536, 16, False),  # more rows than one workgroup holds
        (517, 1024, 65536, 16, True),  # Zipf: slice 0 takes most entries
        (300, 128, 4096, 12, False),  # 12-bit stream
        (64, 64, 1 << 20, 20, False),  # 20-bit indices, 256 slices
        (6, 8, 3, 4, False),
    ],
)
def test_build_round_trip(n, k, nc, bits, zipf):
    idx, packed, bits = _layer(n + k, n, k, nc, bits, zipf)
    blob = _build(packed, bits, n, k, nc)
    _lib.call("npamd_vq_sliced_check", blob.data_ptr(), blob.numel())
    dec, info = cases.decode_sliced_blob(blob.numpy())
    h = info["header"]
    assert (h["n"], h["k"], h["vl"], h["nc"]) == (n, k, 8, nc)
    assert h["n_slices"] == -(-nc // 4096) and h["slice_rows"] == 4096
    assert h["n_entries"] == n * (k // 8) and h["total_bytes"] == blob.numel()
    assert np.array_equal(dec, idx.numpy())
    assert (info["hits"] == 1).all() and (info["writes"] == 1).all()
    assert h["groups_max"] <= 512  # the kernel's LDS map: 8 KiB of activations per token, a slice, a zero row


def test_build_fills_the_requested_workgroups():
    """A config-3-like layer (scaled down) gets about one workgroup per compute unit
    and little padding."""
    n, k, nc = 7168, 2048, 65536
    idx, packed, bits = _layer(1, n, k, nc, 16)
    blob = _build(packed, bits, n, k, nc, target=256)
    h = cases.decode_sliced_blob(blob.numpy())[1]["header"]
    assert 200 <= h["n_workgroups"] <= 256
    slots = h["n_quads"] * 256
    assert slots < 1.4 * h["n_entries"]  # tasks of ~16 entries; strip w padded to the layer's longest strip w, in whole quads


def test_out_of_range_indices_are_clamped_like_the_kernels():
    n, k, nc = 16, 64, 1000  # 10-bit stream can hold up to 1023
    idx = torch.randint(0, 1024, (n * (k // 8),), generator=cases.gen(5))
    packed = IndexPacking.pack(idx, 10)
    blob = _build(packed, 10, n, k, nc)
    dec, _ = cases.decode_sliced_blob(blob.numpy())
    assert np.array_equal(dec, idx.clamp(max=nc - 1).reshape(n, k // 8).numpy())


def test_build_errors():
    idx, packed, bits = _layer(2, 32, 64, 500)
    size = ctypes.c_int64(0)

    def build(**kw):
        a = dict(packed=packed.data_ptr(), nbytes=packed.numel(), bits=bits, n=32, k=64, vl=8, nc=500,
                 target=0, blob=None, cap=0)  # fmt: skip
        a.update(kw)
        _lib.call("npamd_vq_sliced_build", a["packed"], a["nbytes"], a["bits"], a["n"], a["k"], a["vl"],
                  a["nc"], a["target"], a["blob"], a["cap"], ctypes.byref(size))  # fmt: skip

    with pytest.raises(RuntimeError, match="VL = 8"):
        build(vl=4)
    with pytest.raises(RuntimeError, match="packed buffer too short"):
        build(nbytes=packed.numel() - 1)
    with pytest.raises(RuntimeError, match=r"bits must be in \[4, 20\]"):
        build(bits=3)
    with pytest.raises(RuntimeError, match="not divisible"):
        build(k=60)
    build()
    small = torch.zeros(size.value - 1, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="needed"):
        build(blob=small.data_ptr(), cap=small.numel())


def test_check_rejects_damaged_blobs():
    n, k, nc = 200, 128, 20000
    idx, packed, bits = _layer(3, n, k, nc)
    blob = _build(packed, bits, n, k, nc)
    h = cases.decode_sliced_blob(blob.numpy())[1]["header"]

    def check(b):
        _lib.call("npamd_vq_sliced_check", b.data_ptr(), b.numel())

    check(blob)
    with pytest.raises(RuntimeError, match="too short"):
        check(blob[:64].clone())
    with pytest.raises(RuntimeError, match="header says"):
        check(blob[:-256].clone())
    bad = blob.clone()
    bad[0] = 0
    with pytest.raises(RuntimeError, match="magic"):
        check(bad)
    # An entry pointing past the end of the last (short) slice, a duplicated entry
    # and a row outside the layer must all be caught.
    quads = h["off_entries"]
    bad = blob.clone()
    bad[quads : quads + 2] = torch.tensor([0xFF, 0xFF], dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="entry field out of range"):
        check(bad)
    bad = blob.clone()  # entry 1 of lane 0 := entry 0 (row field, then group field)
    bad[quads + 2 : quads + 4] = bad[quads : quads + 2]
    bad[quads + 9] = bad[quads + 8]
    with pytest.raises(RuntimeError, match="filed twice|not filed"):
        check(bad)
    bad = blob.clone()
    row0 = h["off_rowmap"]
    bad[row0 : row0 + 4] = torch.tensor([0x00, 0x00, 0x00, 0x7F], dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="row outside the workgroup.s row block"):
        check(bad)


def test_workspace_bytes_and_header_struct():
    n, k, nc = 64, 64, 20000
    idx, packed, bits = _layer(4, n, k, nc)
    blob = _build(packed, bits, n, k, nc)
    h = cases.decode_sliced_blob(blob.numpy())[1]["header"]
    hdr = ctypes.create_string_buffer(blob[:128].numpy().tobytes(), 128)
    lib = _lib.load()
    assert h["n_partials"] < 256  # fused finish: a 64-bit word and a float per (token, row)
    assert lib.npamd_vq_sliced_workspace_bytes(ctypes.addressof(hdr), 1) == n * 12
    assert lib.npamd_vq_sliced_workspace_bytes(ctypes.addressof(hdr), 3) == 3 * n * 12
    assert lib.npamd_vq_sliced_workspace_bytes(None, 1) == 0


def test_gemv_sliced_validates_before_touching_the_gpu():
    n, k, nc = 64, 64, 20000
    idx, packed, bits = _layer(6, n, k, nc)
    blob = _build(packed, bits, n, k, nc)
    hdr = ctypes.create_string_buffer(blob[:128].numpy().tobytes(), 128)
    hp = ctypes.addressof(hdr)

    def call(**kw):
        a = dict(x=16, ldx=k, perm=None, hdr=hp, blob=16, cb=16, cbdt=_lib.F16, bias=None, y=16, ldy=n, m=1,
                 act=_lib.F16, ws=16, wsb=1 << 30, st=None)  # fmt: skip
        a.update(kw)
        _lib.call("npamd_vq_gemv_sliced", a["x"], a["ldx"], a["perm"], a["hdr"], a["blob"], a["cb"], a["cbdt"], a["bias"],
                  a["y"], a["ldy"], a["m"], a["act"], a["ws"], a["wsb"], a["st"])  # fmt: skip

    with pytest.raises(RuntimeError, match="header is null"):
        call(hdr=None)
    with pytest.raises(RuntimeError, match="activation dtype"):
        call(cbdt=_lib.F16, act=_lib.BF16)
    with pytest.raises(RuntimeError, match="f16 or bf16"):
        call(act=_lib.F32, cbdt=_lib.F32)
    with pytest.raises(RuntimeError, match="exceeds the fused limit"):
        call(m=33)
    with pytest.raises(RuntimeError, match="row stride"):
        call(ldx=k - 8)
    with pytest.raises(RuntimeError, match="null pointer"):
        call(x=None)
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        call(x=8)
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        call(perm=4)
    with pytest.raises(RuntimeError, match="workspace of"):
        call(wsb=16)
    bad = ctypes.create_string_buffer(b"\0" * 128, 128)
    with pytest.raises(RuntimeError, match="not a slice-list header"):
        call(hdr=ctypes.addressof(bad))
    call(m=0)  # nothing to do: returns before any launch
