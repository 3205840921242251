"""The 128-column tile-decode GEMM (csrc/gemm_tile2.hip) through the C ABI, against the oracle.

The library takes this kernel by itself only for large layers with codebooks LDS does not hold; the
tests force it (NPAMD_TILE_WIDE=2) on small ragged shapes the oracle finishes in milliseconds, and
compare with the oracle's decode + double-accumulated product, with the one-pass decode through
one-hot activations (bit for bit), and with itself from run to run.
"""

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests import cases

pytestmark = pytest.mark.gpu


@pytest.fixture
def tile_wide(monkeypatch):
    """force(mode, splits): NPAMD_TILE_WIDE / NPAMD_TILE_SPLITS for one test (the library reads its
    tuning variables once, so they are re-read on the way in and out)."""
    from neuropress_amd import _lib

    def force(mode: int, splits: int = 0):
        monkeypatch.setenv("NPAMD_TILE_WIDE", str(mode))
        monkeypatch.setenv("NPAMD_TILE_SPLITS", str(splits))
        _lib.load().npamd_diag_reload_tuning()

    yield force
    monkeypatch.delenv("NPAMD_TILE_WIDE", raising=False)
    monkeypatch.delenv("NPAMD_TILE_SPLITS", raising=False)
    _lib.load().npamd_diag_reload_tuning()


def _ref(oracle_lib, L, act):
    code = orc.torch_dtype_code(act)
    w = oracle_lib.vq_decode(L["packed"].numpy(), L["bits"], orc.to_bits(L["cb"]), L["n"], L["k"], code)
    bias = None if L["bias"] is None else orc.to_bits(L["bias"])
    return oracle_lib.linear_f64(orc.to_bits(L["x"]), code, w, code, bias, code)


def _check(y, ref):
    ok, max_abs, excess = cases.within_tol(y.float().cpu().numpy(), ref)
    assert ok, f"max abs err {max_abs:.3e}, {excess:.2f}x the 1e-2 bound"


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 17, 96, 130, 257, 300, 384, 400])
@pytest.mark.parametrize(
    "n,k,splits",
    [(300, 448, 1), (300, 448, 2), (130, 1024, 2), (264, 1088, 3), (1004, 512, 0), (300, 192, 1), (300, 256, 1), (300, 128, 1)],
)
def test_wide_tile_gemm_against_the_oracle(gpu, oracle_lib, tile_wide, act, m, n, k, splits):
    """Ragged N (two to eight 128-column blocks, N % 8 != 0 once: element stores), K of 3 to 17 steps (odd and
    even counts per part: the loop ends in two steps of its own behind pairs; two steps are fewer than the
    kernel takes, so the 64-column kernel answers), every row tile count (one to three per wave, two row
    blocks at 400 tokens), K whole, in two halves that meet in the kernel, and in three parts that meet in
    the reduction kernel."""
    from neuropress_amd import kernels

    tile_wide(2, splits)
    L = cases.vq_layer(700 + m + n, n, k, 65536, bits=16, act=act, m=m, bias=True, std=0.05)
    cb = L["cb"].to(act).to(gpu)  # the kernel takes the codebook in the activation dtype
    y = kernels.vq_gemm_tile(L["x"].to(gpu), L["packed"].to(gpu), cb, 16, n, L["bias"].to(gpu))
    _check(y, _ref(oracle_lib, L, act))
    y2 = kernels.vq_gemm_tile(L["x"].to(gpu), L["packed"].to(gpu), cb, 16, n, L["bias"].to(gpu))
    assert torch.equal(y, y2), "the result depends on which half of K finished first"


@pytest.mark.parametrize("m", [17, 200, 384])
def test_wide_tile_gemm_takes_activations_with_a_row_stride(gpu, tile_wide, m):
    """x as a view of a wider buffer (row stride 2 K + 8 elements, rows 16-byte aligned): the x tile's transfers
    take the stride from the call; the result equals the one on a contiguous copy bit for bit."""
    from neuropress_amd import kernels

    n, k = 300, 448
    tile_wide(2, 2)
    L = cases.vq_layer(650 + m, n, k, 65536, bits=16, act=torch.bfloat16, m=m, bias=True, std=0.05)
    pk, cb, bias = L["packed"].to(gpu), L["cb"].bfloat16().to(gpu), L["bias"].to(gpu)
    wide = torch.full((m, 2 * k + 8), float("nan"), dtype=torch.bfloat16, device=gpu)
    wide[:, :k] = L["x"].to(gpu)
    view = wide[:, :k]
    assert view.stride(0) == 2 * k + 8 and not view.is_contiguous()
    assert torch.equal(kernels.vq_gemm_tile(view, pk, cb, 16, n, bias), kernels.vq_gemm_tile(view.contiguous(), pk, cb, 16, n, bias))


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("splits", [1, 2, 4])
def test_wide_tile_gemm_decodes_bit_exactly(gpu, tile_wide, act, splits):
    """One-hot activations: y[m, n] is the single product 1 * W[n, k_m], so the kernel must return the
    one-pass decode (itself bit-exact against the oracle) exactly, whichever way K is split."""
    from neuropress_amd import kernels

    n, k = 200, 1024
    L = cases.vq_layer(77, n, k, 65536, bits=16, act=act, m=1, std=0.05)
    pk, cb = L["packed"].to(gpu), L["cb"].to(gpu)
    wt = kernels.vq_dequant(pk, cb, 16, n, k, act).t().contiguous()
    tile_wide(2, splits)
    eye = torch.eye(k, dtype=act, device=gpu)
    cba = cb.to(act)
    assert torch.equal(kernels.vq_gemm_tile(eye, pk, cba, 16, n, None), wt), "1024 tokens"
    assert torch.equal(kernels.vq_gemm_tile(eye[100:330], pk, cba, 16, n, None), wt[100:330]), "230 tokens"
    assert torch.equal(kernels.vq_gemm_tile(eye[5:26], pk, cba, 16, n, None), wt[5:26]), "21 tokens"


def test_wide_and_narrow_tile_gemm_agree_on_a_large_layer(gpu, tile_wide):
    """A layer of the size the library takes the 128-column kernel for by itself (2^25 weights), K in two
    halves: against the 64-column kernel and the dense product of the decoded weight."""
    from neuropress_amd import _lib, kernels

    n, k, m = 8192, 4096, 384
    g = cases.gen(5)
    cb = (torch.randn(65536, 8, generator=g) * 0.02).to(torch.float16)
    pk = torch.randint(0, 65536, (n * k // 8,), generator=g, dtype=torch.int32).to(torch.int16).view(torch.uint8).to(gpu)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(gpu)
    cba = cb.to(torch.bfloat16).to(gpu)
    assert _lib.load().npamd_gemm_tile_workspace_bytes(m, n, k) > 0
    tile_wide(1)
    y_auto = kernels.vq_gemm_tile(x, pk, cba, 16, n, None)
    tile_wide(0)
    y_narrow = kernels.vq_gemm_tile(x, pk, cba, 16, n, None)
    ref = x.float() @ kernels.vq_dequant(pk, cb.to(gpu), 16, n, k, torch.bfloat16).float().t()
    for y in (y_auto, y_narrow):
        err = (y.float() - ref).abs()
        assert bool((err <= 1e-2 + 1e-2 * ref.abs()).all()), float(err.max())
    # same products, f32 sums in a different order: they differ by output roundings at most
    assert float((y_auto.float() - y_narrow.float()).abs().max()) <= 2.0 ** -6


def _q_ref(oracle_lib, L, act):
    code = orc.torch_dtype_code(act)
    zp = None if L["zp"] is None else orc.to_bits(L["zp"])
    w = oracle_lib.q_decode(L["blob"].numpy(), orc.to_bits(L["scale"]), zp, L["nbits"], L["gs"], code)
    bias = None if L["bias"] is None else orc.to_bits(L["bias"])
    return oracle_lib.linear_f64(orc.to_bits(L["x"]), code, w, code, bias, code)


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("nbits,asym,gs", [(4, False, 32), (4, True, 32), (4, False, 128), (8, False, 32), (8, True, 64)])
@pytest.mark.parametrize("m", [1, 17, 130, 257, 384, 400, 520])
@pytest.mark.parametrize("n,k,splits", [(300, 512, 1), (300, 512, 2), (264, 1024, 3), (300, 448, 1), (300, 448, 2), (300, 192, 1)])
def test_wide_tile_gemm_group_affine_against_the_oracle(gpu, oracle_lib, tile_wide, act, nbits, asym, gs, m, n, k, splits):
    """int4 / int8 codes through the 128-column kernel (packed bytes staged in LDS, decoded between the MFMAs):
    symmetric and with zero points, group sizes of 32 to 128, one to three row tiles per wave and the 256-row
    blocks taken past 384 tokens, K whole, in two halves and in three parts, odd and even step counts."""
    from neuropress_amd import kernels

    if k % gs:
        pytest.skip("K is not a multiple of the group size")

    tile_wide(2, splits)
    Q = cases.q4_layer(800 + m + nbits, n, k, nbits=nbits, gs=gs, act=act, m=m, asym=asym, bias=True)
    zp = None if Q["zp"] is None else Q["zp"].to(gpu)
    args = (Q["x"].to(gpu), Q["blob"].to(gpu), Q["scale"].to(gpu), nbits, gs, zp, Q["bias"].to(gpu))
    y = kernels.q_gemm_tile(*args)
    _check(y, _q_ref(oracle_lib, Q, act))
    assert torch.equal(y, kernels.q_gemm_tile(*args)), "the result depends on which half of K finished first"


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("nbits,asym,gs", [(4, False, 32), (4, True, 128), (8, False, 32), (8, True, 32)])
def test_wide_tile_gemm_group_affine_decodes_bit_exactly(gpu, tile_wide, act, nbits, asym, gs):
    """One-hot activations through the 128-column kernel return the one-pass decode exactly."""
    from neuropress_amd import kernels

    n, k = 200, 1024
    Q = cases.q4_layer(63, n, k, nbits=nbits, gs=gs, act=act, m=1, asym=asym)
    blob, sc = Q["blob"].to(gpu), Q["scale"].to(gpu)
    zp = None if Q["zp"] is None else Q["zp"].to(gpu)
    wt = kernels.q_dequant(blob, sc, nbits, gs, zp, act).t().contiguous()
    eye = torch.eye(k, dtype=act, device=gpu)
    for splits in (1, 2, 4):
        tile_wide(2, splits)
        assert torch.equal(kernels.q_gemm_tile(eye, blob, sc, nbits, gs, zp), wt), f"1024 tokens, {splits} splits"
        assert torch.equal(kernels.q_gemm_tile(eye[100:330], blob, sc, nbits, gs, zp), wt[100:330]), f"230 tokens, {splits} splits"


@pytest.mark.parametrize("m", [130, 384])
def test_wide_tile_gemm_meets_through_a_workspace_nobody_cleared(gpu, tile_wide, m):
    """The two K halves of a tile meet through a word of the workspace that holds the call's own
    random number; the workspace comes from torch's allocator as it is.  Whatever the memory held
    before -- all ones, the words a previous call left -- the result is the same, and a graph that
    replays one call (number included) gives it on every replay."""
    from neuropress_amd import _lib, kernels

    n, k = 520, 1024
    tile_wide(2, 2)
    L = cases.vq_layer(900 + m, n, k, 65536, bits=16, act=torch.bfloat16, m=m, bias=True, std=0.05)
    x, pk, cb, bias = L["x"].to(gpu), L["packed"].to(gpu), L["cb"].bfloat16().to(gpu), L["bias"].to(gpu)
    tile_wide(2, 1)
    whole = kernels.vq_gemm_tile(x, pk, cb, 16, n, bias)  # K in one piece: no workspace
    tile_wide(2, 2)
    need = _lib.load().npamd_gemm_tile_workspace_bytes(m, n, k)
    assert need > 0
    expect = kernels.vq_gemm_tile(x, pk, cb, 16, n, bias)
    assert float((expect.float() - whole.float()).abs().max()) <= 2.0 ** -6  # f32 sums in another order
    for fill in (0xFF, 0x00, 0x5A):
        junk = torch.full((need + (1 << 20),), fill, dtype=torch.uint8, device=gpu)
        del junk  # back to the allocator: the next call's workspace is carved out of it
        for _ in range(3):  # the second and third call find the words the one before left
            assert torch.equal(kernels.vq_gemm_tile(x, pk, cb, 16, n, bias), expect)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            y = kernels.vq_gemm_tile(x, pk, cb, 16, n, bias)
    for _ in range(4):
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, expect)
        assert torch.equal(kernels.vq_gemm_tile(x, pk, cb, 16, n, bias), expect)  # eager work between the replays
