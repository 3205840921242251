"""Parity of the prefix-coded decode GEMVs (two-tier, n-tier, zero-escape streams read as stored)
against the CPU oracle, through the C ABI.

The coded buffer of a layer is made by the host packers (themselves pinned against the oracle's
decoders and hand-assembled buffers in tests/test_host_entropy_packing.py), split into its
streams, and handed to the wrappers with the packers' per-row offsets.  Bar: outputs within
1e-2 abs + 1e-2 rel of the oracle's double-accumulated contraction of the oracle-decoded weight;
with one-hot activations the decoded weight itself must come back bit for bit.
"""

import numpy as np
import pytest
import torch

from neuropress_amd.transforms.vq_packing import (
    IndexPacking,
    NTieredIndexPacking,
    TieredIndexPacking,
    ZeroEscapePacking,
)
from oracle import oracle as orc
from tests import cases

pytestmark = pytest.mark.gpu


def _layer(seed, n, k, nc, vl, act, m, zipf=True):
    g = cases.gen(seed)
    cb = (torch.randn(nc, vl, generator=g) * 0.05).to(torch.float16)
    cnt = n * (k // vl)
    idx = cases.zipf_indices(g, nc, cnt) if zipf else torch.randint(0, nc, (cnt,), generator=g)
    x = torch.randn(m, k, generator=g).to(act)
    bias = torch.randn(n, generator=g).to(act)
    return dict(cb=cb, idx=idx, x=x, bias=bias, n=n, k=k, vl=vl, nc=nc)


def _ref(oracle_lib, L, act):
    code = orc.torch_dtype_code(act)
    bits = IndexPacking.bits_for(L["nc"])
    w = oracle_lib.vq_decode(IndexPacking.pack(L["idx"], bits).numpy(), bits, orc.to_bits(L["cb"]), L["n"], L["k"], code)
    return oracle_lib.linear_f64(orc.to_bits(L["x"]), code, w, code, orc.to_bits(L["bias"]), code)


def _check(y, ref):
    ok, max_abs, excess = cases.within_tol(y.float().cpu().numpy(), ref)
    assert ok, f"max abs err {max_abs:.3e}, {excess:.2f}x the 1e-2 bound"


def _call(kind, gpu, L, x, bias):
    """Pack L's indices in format `kind`, split, upload and run the matching wrapper."""
    from neuropress_amd import kernels

    n, g = L["n"], L["k"] // L["vl"]
    cold_bits = IndexPacking.bits_for(L["nc"])
    dev = lambda t: t.contiguous().to(gpu)
    cb = dev(L["cb"])
    if kind.startswith("tiered"):
        hot_bits = int(kind[6:] or 4)
        buf = TieredIndexPacking.pack(L["idx"], cold_bits, hot_bits)
        prefix, hot, cold, cbits, hbits = TieredIndexPacking.split_streams(buf)
        hot_off, cold_off = TieredIndexPacking.compute_row_offsets(buf, n, g)
        assert (cbits, hbits) == (cold_bits, hot_bits)
        return kernels.vq_linear_tiered(x, dev(prefix), dev(hot), dev(cold), dev(hot_off), dev(cold_off), cb,
                                        cbits, hbits, L["vl"], bias)
    if kind.startswith("ntier"):
        tier_bits = {"ntier2": [4, cold_bits], "ntier3": [4, 8, cold_bits], "ntier4": [4, 6, 8, cold_bits]}[kind]
        buf = NTieredIndexPacking.pack(L["idx"], tier_bits)
        prefixes, tiers, bits = NTieredIndexPacking.split_streams(buf)
        offs = NTieredIndexPacking.compute_row_offsets(buf, n, g)
        assert bits == tier_bits
        return kernels.vq_linear_ntier(x, [dev(p) for p in prefixes], [dev(t) for t in tiers], [dev(o) for o in offs],
                                       cb, bits, L["vl"], bias)
    buf = ZeroEscapePacking.pack(L["idx"], cold_bits)
    cls, hot, warm, cold, cbits = ZeroEscapePacking.split_streams(buf)
    offs = ZeroEscapePacking.compute_row_offsets(buf, n, g)
    return kernels.vq_linear_zero_escape(x, dev(cls), dev(hot), dev(warm), dev(cold), *[dev(o) for o in offs], cb,
                                         cbits, L["vl"], bias)


KINDS = ["tiered", "tiered8", "ntier2", "ntier3", "ntier4", "zesc"]


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("m", [1, 3, 11])
def test_coded_gemv_matches_oracle(gpu, oracle_lib, act, kind, m):
    """Zipf(1.1) indices over 4096 rows (most indices in the hot classes); 37 rows of 70 groups:
    rows end inside a 64-index segment and inside a byte of every stream."""
    L = _layer(11 + m, 37, 560, 4096, 8, act, m)
    y = _call(kind, gpu, L, L["x"].to(gpu), L["bias"].to(gpu))
    assert y.shape == (m, 37) and y.dtype == act
    _check(y, _ref(oracle_lib, L, act))


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("nc,vl,zipf", [(65536, 8, True), (65536, 8, False), (300, 4, True), (4096, 6, False)])
def test_coded_gemv_reads_the_weight_back_exactly(gpu, kind, nc, vl, zipf):
    """One-hot activations: y[m, n] = W[n, k_m] exactly, so every index must have been found in
    its stream.  Uniform indices put almost everything in the cold class, Zipf in the hot ones;
    vector lengths 4 and 6 take the element loop."""
    n, groups = 70, 67
    k = groups * vl
    L = _layer(5 + nc + vl, n, k, nc, vl, torch.float16, 1, zipf=zipf)
    w = L["cb"][L["idx"]].reshape(n, k)
    eye = torch.eye(k, dtype=torch.float16)
    for k0 in (0, k - 16):
        y = _call(kind, gpu, L, eye[k0:k0 + 16].to(gpu), None)
        assert torch.equal(y.cpu(), w[:, k0:k0 + 16].t())


def test_coded_gemv_full_size_row(gpu, oracle_lib):
    """A 4096-wide reduction (eight segments per row) on 512 rows, 65536-row codebook."""
    L = _layer(77, 512, 4096, 65536, 8, torch.bfloat16, 2)
    ref = _ref(oracle_lib, L, torch.bfloat16)
    for kind in ("tiered8", "ntier3", "zesc"):
        _check(_call(kind, gpu, L, L["x"].to(gpu), L["bias"].to(gpu)), ref)


def test_coded_gemv_argument_errors(gpu):
    from neuropress_amd import kernels

    L = _layer(3, 8, 64, 256, 8, torch.float16, 1)
    buf = TieredIndexPacking.pack(L["idx"], 8, 4)
    prefix, hot, cold, cbits, hbits = TieredIndexPacking.split_streams(buf)
    hot_off, cold_off = TieredIndexPacking.compute_row_offsets(buf, 8, 8)
    d = lambda t: t.contiguous().to(gpu)
    args = [d(prefix), d(hot), d(cold), d(hot_off), d(cold_off), d(L["cb"]), cbits, hbits, 8]
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        kernels.vq_linear_tiered(L["x"].float().to(gpu), *args)
    with pytest.raises(RuntimeError, match="exceeds the fused limit"):
        kernels.vq_linear_tiered(torch.zeros(33, 64, dtype=torch.float16, device=gpu), *args)
    bad = list(args)
    bad[3] = d(hot_off)[:-1]
    with pytest.raises(RuntimeError, match="N \\+ 1 entries"):
        kernels.vq_linear_tiered(L["x"].to(gpu), *bad)
    bad = list(args)
    bad[3] = d(hot_off).long()
    with pytest.raises(RuntimeError, match="int32"):
        kernels.vq_linear_tiered(L["x"].to(gpu), *bad)
