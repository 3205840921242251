"""Seeded synthetic layers shared by the tests (same generators as bench.py)."""

from __future__ import annotations

import numpy as np
import torch

from neuropress_amd.transforms.vq_packing import IndexPacking


def gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def vq_layer(seed, n, k, nc, vl=8, bits=None, act=torch.float16, m=1, bias=False, std=0.02):
    g = gen(seed)
    bits = bits or IndexPacking.bits_for(nc)
    cb = (torch.randn(nc, vl, generator=g) * std).to(torch.float16)
    idx = torch.randint(0, nc, (n * (k // vl),), generator=g)
    packed = IndexPacking.pack(idx, bits)
    x = torch.randn(m, k, generator=g).to(act)
    b = torch.randn(n, generator=g).to(act) if bias else None
    return dict(cb=cb, idx=idx, packed=packed, bits=bits, x=x, bias=b, n=n, k=k, vl=vl, nc=nc)


def zipf_indices(g, nc, count, s=1.1):
    p = 1.0 / torch.arange(1, nc + 1, dtype=torch.float64) ** s
    return torch.multinomial(p / p.sum(), count, replacement=True, generator=g)


def rvq_layer(seed, n, k, nc_main=65536, nc_res=256, vl=8, act=torch.float16, m=1, zipf=True):
    g = gen(seed)
    cbm = (torch.randn(nc_main, vl, generator=g) * 0.02).to(torch.float16)
    cbr = (torch.randn(nc_res, vl, generator=g) * 0.02).to(torch.float16)
    cnt = n * (k // vl)
    im = zipf_indices(g, nc_main, cnt) if zipf else torch.randint(0, nc_main, (cnt,), generator=g)
    ir = zipf_indices(g, nc_res, cnt) if zipf else torch.randint(0, nc_res, (cnt,), generator=g)
    bm, br = IndexPacking.bits_for(nc_main), IndexPacking.bits_for(nc_res)
    scale = (torch.rand(n, generator=g) + 0.5).to(torch.float16)
    wbias = (torch.randn(n, generator=g) * 0.01).to(torch.float16)
    x = torch.randn(m, k, generator=g).to(act)
    return dict(cbm=cbm, cbr=cbr, im=im, ir=ir, pm=IndexPacking.pack(im, bm), pr=IndexPacking.pack(ir, br),
                bm=bm, br=br, scale=scale, wbias=wbias, x=x, n=n, k=k, vl=vl)


def q4_layer(seed, n, k, nbits=4, gs=32, act=torch.float16, m=1, asym=False, bias=False):
    from neuropress_amd.t2n.packing import BitPacking

    g = gen(seed)
    codes = torch.randint(0, 1 << nbits, (n, k), generator=g, dtype=torch.int64).to(torch.uint8)
    blob = BitPacking(nbits).compress(codes)
    scale = (torch.rand(n * (k // gs), generator=g) * 0.019 + 0.001).to(torch.float16)
    zp = (torch.rand(n * (k // gs), generator=g) * ((1 << nbits) - 1)).to(torch.float16) if asym else None
    x = torch.randn(m, k, generator=g).to(act)
    b = torch.randn(n, generator=g).to(act) if bias else None
    return dict(codes=codes, blob=blob, scale=scale, zp=zp, x=x, bias=b, n=n, k=k, nbits=nbits, gs=gs)


def within_tol(y: np.ndarray, ref: np.ndarray, atol=1e-2, rtol=1e-2):
    """The output bar of the path: |y - ref| <= 1e-2 + 1e-2 * |ref| against an
    f32-or-better accumulated reference.  Returns (ok, max_abs, max_rel_excess)."""
    err = np.abs(y.astype(np.float64) - ref)
    bound = atol + rtol * np.abs(ref)
    return bool((err <= bound).all()), float(err.max(initial=0.0)), float((err / bound).max(initial=0.0))


def decode_sliced_blob(blob: np.ndarray) -> tuple[np.ndarray, dict]:
    """Read a slice-list blob back into the ``[N, K/8]`` index matrix it was built from.

    An independent reader of the layout: header (with the 16 strip lengths every
    workgroup shares), 32-byte workgroup records, per-lane row map, and per
    workgroup, wave, quad and lane a 12-byte record of four uint16 fields (13-bit
    codebook row, top bit = bit 8 of the group) followed by the four groups' low bytes.  ``hits`` counts how often each (row, group)
    pair was filed and ``writes`` how often each (partial, row) cell is written;
    both must be 1 everywhere.
    """
    import struct

    names = ("magic", "version", "n", "k", "vl", "nc", "slice_rows", "n_slices", "n_workgroups",
             "n_partials", "groups_max", "flags", "n_quads", "n_entries", "off_workgroups",
             "off_rowmap", "off_entries", "total_bytes")  # fmt: skip
    h = dict(zip(names, struct.unpack("<2I9iI6q", blob[:96].tobytes())))
    wave_quads = struct.unpack("<16H", blob[96:128].tobytes())
    h["wave_quads"] = wave_quads
    assert h["magic"] == 0x4C53504E and h["version"] == 3 and h["vl"] == 8
    n, groups, n_wg = h["n"], h["k"] // 8, h["n_workgroups"]
    wg_quads = max(sum(wave_quads), 1)
    assert h["n_quads"] == n_wg * wg_quads
    wgs = np.frombuffer(blob, dtype="<u4", count=n_wg * 8, offset=h["off_workgroups"]).reshape(n_wg, 8).astype(np.int64)
    rowmap = np.frombuffer(blob, dtype="<u4", count=n_wg * 1024, offset=h["off_rowmap"]).reshape(n_wg, 16, 64).astype(np.int64)
    quads = np.frombuffer(blob, dtype=np.uint8, count=h["n_quads"] * 768, offset=h["off_entries"]).reshape(n_wg, wg_quads, 64, 12)
    idx = np.full((n, groups), -1, dtype=np.int64)
    hits = np.zeros((n, groups), dtype=np.int32)
    writes = np.zeros((h["n_partials"], n), dtype=np.int32)
    for w in range(n_wg):
        sl, partial, g_begin, g_count, row_begin, row_count = wgs[w, :6]
        assert row_count <= 1024 and row_begin + row_count <= n
        if h["flags"] & 1:  # workgroup w works on slice w % n_slices
            assert sl == w % h["n_slices"]
        quad_begin = 0
        for s in range(16):
            nq = wave_quads[s]
            rows = rowmap[w, s]
            has_row = rows != 0xFFFFFFFF
            assert ((rows[has_row] >= row_begin) & (rows[has_row] < row_begin + row_count)).all()
            np.add.at(writes, (np.full(int(has_row.sum()), partial), rows[has_row]), 1)
            if nq == 0:
                continue
            q = quads[w, quad_begin : quad_begin + nq].astype(np.int64)  # [nq, lane, 12]
            quad_begin += nq
            field = (q[..., 0:8:2] | (q[..., 1:8:2] << 8)).transpose(1, 0, 2).reshape(64, nq * 4)  # [lane, step]
            local = field & 0x1FFF  # bits 0-12: the row; bit 15: bit 8 of the group
            g_local = q[..., 8:12].transpose(1, 0, 2).reshape(64, nq * 4) | ((field >> 15) << 8)
            live = local != 4096  # 4096 = the zero row padding entries select
            assert (g_local < g_count).all() and (local[live] < h["slice_rows"]).all()
            assert not live[~has_row].any(), "live entry in a lane without a row"
            rr = np.broadcast_to(rows[:, None], local.shape)[live]
            gg = (g_begin + g_local)[live]
            idx[rr, gg] = (sl * h["slice_rows"] + local)[live]
            np.add.at(hits, (rr, gg), 1)
    return idx, {"header": h, "hits": hits, "writes": writes}
