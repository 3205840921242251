"""Parity of the HIP kernels against the CPU oracle, through the C ABI (ctypes wrappers).

Bars: decoded weights bit-exact; layer outputs within 1e-2 abs + 1e-2 rel of
the oracle's double-accumulated contraction of the oracle-decoded weight.
"""

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests import cases

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float16, torch.float32]


def _bits_equal(t: torch.Tensor, ref: np.ndarray):
    got = orc.to_bits(t)
    assert got.dtype == ref.dtype and got.shape == ref.shape
    assert np.array_equal(got, ref), f"{(got != ref).sum()} of {ref.size} elements differ"


# ------------------------------------------------------------------ decode ---


@pytest.mark.parametrize("vl", [4, 8, 6])
@pytest.mark.parametrize("bits", [4, 8, 10, 12, 14, 16])
@pytest.mark.parametrize("dtype", DTYPES)
def test_vq_dequant_bit_exact(gpu, oracle_lib, bits, dtype, vl):
    # Odd N so the last index ends mid-byte (the reference's own case:
    # tests/nn/test_np_vq_linear.py:546-562 of the reference).
    from neuropress_amd import kernels

    n, k = 37, 16 * vl
    nc = min(1 << bits, 4096)
    L = cases.vq_layer(100 + bits, n, k, nc, vl=vl, bits=bits, std=1.0)
    ref = oracle_lib.vq_decode(L["packed"].numpy(), bits, orc.to_bits(L["cb"]), n, k, orc.torch_dtype_code(dtype))
    out = kernels.vq_dequant(L["packed"].to(gpu), L["cb"].to(gpu), bits, n, k, dtype)
    assert out.dtype == dtype and out.shape == (n, k)
    _bits_equal(out, ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", [8, 11, 16])
def test_vq_dequant_vl4_odd_vector_count(gpu, oracle_lib, dtype, bits):
    """Vector length 4 decodes two vectors per thread; 37 rows of 3 vectors leave a single one at
    the end."""
    from neuropress_amd import kernels

    n, k = 37, 12
    L = cases.vq_layer(170 + bits, n, k, min(1 << bits, 2048), vl=4, bits=bits, std=1.0)
    ref = oracle_lib.vq_decode(L["packed"].numpy(), bits, orc.to_bits(L["cb"]), n, k, orc.torch_dtype_code(dtype))
    _bits_equal(kernels.vq_dequant(L["packed"].to(gpu), L["cb"].to(gpu), bits, n, k, dtype), ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nc,bits,vl", [(4096, 12, 8), (3000, 12, 8), (4096, 16, 8), (1025, 11, 8),
                                        (4096, 12, 4), (8192, 13, 4), (3001, 16, 4)])
def test_vq_dequant_lds_codebook_bit_exact(gpu, oracle_lib, dtype, nc, bits, vl):
    """Layers of at least 2^20 vectors with a table of 16 to 64 KiB decode from an LDS copy of it
    (512 blocks, each a contiguous run of vectors), for vector length 8 and 4 (an odd row count
    with VL = 4 ends in half a 16-byte unit).  2050 rows of 4096 columns: the last block's run
    is ragged.  Checked bit for bit against the oracle."""
    from neuropress_amd import kernels

    n, k = 2050, 4096
    L = cases.vq_layer(300 + nc + bits, n, k, nc, vl=vl, bits=bits, std=1.0)
    ref = oracle_lib.vq_decode(L["packed"].numpy(), bits, orc.to_bits(L["cb"]), n, k, orc.torch_dtype_code(dtype))
    out = kernels.vq_dequant(L["packed"].to(gpu), L["cb"].to(gpu), bits, n, k, dtype)
    _bits_equal(out, ref)


def test_vq_dequant_special_values(gpu, oracle_lib):
    """Codebook holding inf, subnormals, the largest finite half and signed zeros."""
    from neuropress_amd import kernels

    bits_pat = np.array([0x0000, 0x8000, 0x7C00, 0xFC00, 0x0001, 0x8001, 0x03FF, 0x7BFF,
                         0x3555, 0xB555, 0x0400, 0x3C01, 0x3BFF, 0x1234, 0xABCD, 0x4321], dtype=np.uint16)
    cb = orc.from_bits(bits_pat.reshape(2, 8), torch.float16)
    idx = torch.tensor([0, 1, 1, 0, 1, 0])
    from neuropress_amd.transforms.vq_packing import IndexPacking

    packed = IndexPacking.pack(idx, 4)
    for dtype in DTYPES:
        ref = oracle_lib.vq_decode(packed.numpy(), 4, bits_pat.reshape(2, 8), 2, 24, orc.torch_dtype_code(dtype))
        out = kernels.vq_dequant(packed.to(gpu), cb.to(gpu), 4, 2, 24, dtype)
        _bits_equal(out, ref)


@pytest.mark.parametrize("bits", [4, 5, 7, 9, 12, 13, 16])
def test_widen_indices(gpu, bits):
    from neuropress_amd import kernels
    from neuropress_amd.transforms.vq_packing import IndexPacking

    idx = torch.randint(0, 1 << bits, (1001 if bits != 4 else 1002,), generator=cases.gen(bits))
    packed = IndexPacking.pack(idx, bits).to(gpu)
    got = kernels.unpack_indices(packed, idx.numel(), bits).cpu()
    assert torch.equal(got, idx)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("with_affine", [True, False])
def test_rvq_dequant_bit_exact(gpu, oracle_lib, dtype, with_affine):
    from neuropress_amd import kernels

    L = cases.rvq_layer(7, 24, 128, nc_main=4096, nc_res=256)
    sc = L["scale"] if with_affine else None
    wb = L["wbias"] if with_affine else None
    ref = oracle_lib.rvq_decode(
        L["pm"].numpy(), L["bm"], L["pr"].numpy(), L["br"], orc.to_bits(L["cbm"]), orc.to_bits(L["cbr"]),
        None if sc is None else orc.to_bits(sc), None if wb is None else orc.to_bits(wb),
        24, 128, orc.torch_dtype_code(dtype))
    out = kernels.rvq_dequant(
        L["pm"].to(gpu), L["bm"], L["pr"].to(gpu), L["br"], L["cbm"].to(gpu), L["cbr"].to(gpu),
        None if sc is None else sc.to(gpu), None if wb is None else wb.to(gpu), 24, 128, dtype)
    _bits_equal(out, ref)


@pytest.mark.parametrize("nbits,gs", [(4, 32), (4, 128), (8, 32), (2, 16), (1, 8), (4, 24)])
@pytest.mark.parametrize("asym", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_q_dequant_bit_exact(gpu, oracle_lib, nbits, gs, asym, dtype):
    from neuropress_amd import kernels

    n, k = 19, gs * 8
    L = cases.q4_layer(50 + nbits, n, k, nbits=nbits, gs=gs, asym=asym)
    ref = oracle_lib.q_decode(L["blob"].numpy(), orc.to_bits(L["scale"]),
                              None if L["zp"] is None else orc.to_bits(L["zp"]), nbits, gs,
                              orc.torch_dtype_code(dtype))
    out = kernels.q_dequant(L["blob"].to(gpu), L["scale"].to(gpu), nbits, gs,
                            None if L["zp"] is None else L["zp"].to(gpu), dtype)
    _bits_equal(out, ref)


# ---------------------------------------------------------------- contraction ---


def _vq_ref(oracle_lib, L, act):
    code = orc.torch_dtype_code(act)
    w = oracle_lib.vq_decode(L["packed"].numpy(), L["bits"], orc.to_bits(L["cb"]), L["n"], L["k"], code)
    bias = None if L["bias"] is None else orc.to_bits(L["bias"])
    return oracle_lib.linear_f64(orc.to_bits(L["x"]), code, w, code, bias, code)


def _check(y: torch.Tensor, ref: np.ndarray):
    ok, max_abs, excess = cases.within_tol(y.float().cpu().numpy(), ref)
    assert ok, f"max abs err {max_abs:.3e}, {excess:.2f}x the 1e-2 bound"


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits,nc", [(4, 16), (8, 256), (12, 4096), (16, 65536)])
@pytest.mark.parametrize("m", [1, 2, 5, 16, 17, 32])
@pytest.mark.parametrize("vl", [8, 4])
def test_vq_gemv_fast_path(gpu, oracle_lib, act, bits, nc, m, vl):
    from neuropress_amd import kernels

    # N not a multiple of 16, K = 5 chunks of 64 (not a multiple of the 256-k step).
    # Vector length 4 (the reference's default, np_vq_linear.py:109): two codebook rows per operand.
    L = cases.vq_layer(200 + bits + m, 100, 320, nc, vl=vl, bits=bits, act=act, m=m, bias=True, std=0.05)
    y = kernels.vq_linear(L["x"].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), bits, vl,
                          L["bias"].to(gpu), out_features=100)
    assert y.shape == (m, 100) and y.dtype == act
    _check(y, _vq_ref(oracle_lib, L, act))


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits,nc", [(4, 16), (8, 256), (12, 4096), (16, 65536)])
@pytest.mark.parametrize("m", [1, 2, 5, 16])
@pytest.mark.parametrize("vl", [8, 4])
def test_vq_gemv_column_perm(gpu, oracle_lib, act, bits, nc, m, vl):
    """npamd_vq_gemv_perm == the plain GEMV fed with x[:, column_perm] (reference:
    np_vq_linear.py:1027-1028), checked against the oracle on the permuted activations.  x has a
    row stride larger than K, so a kernel that ignored the permutation or the stride would fail."""
    from neuropress_amd import kernels

    n, k = 100, 320
    L = cases.vq_layer(700 + bits + m, n, k, nc, vl=vl, bits=bits, act=act, m=m, bias=True, std=0.05)
    perm = torch.randperm(k, generator=cases.gen(9 + m))
    xw = torch.zeros(m, k + 64, dtype=act)
    xw[:, :k] = L["x"]
    x_gpu = xw.to(gpu)[:, :k]  # stride k + 64
    assert kernels.vq_linear_perm_supported(m, n, k, nc, vl, bits)
    y = kernels.vq_linear(x_gpu, L["packed"].to(gpu), L["cb"].to(gpu), bits, vl, L["bias"].to(gpu),
                          out_features=n, column_perm=perm.to(torch.int32).to(gpu))
    assert y.shape == (m, n) and y.dtype == act
    _check(y, _vq_ref(oracle_lib, dict(L, x=L["x"][:, perm].contiguous()), act))
    # bit-identical to the unpermuted kernel on pre-gathered activations
    y2 = kernels.vq_linear(L["x"][:, perm].contiguous().to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), bits, vl,
                           L["bias"].to(gpu), out_features=n)
    assert torch.equal(y, y2)


def test_vq_gemv_column_perm_limits(gpu):
    """Shapes the permuted GEMV does not take are refused with a message, not computed wrongly."""
    from neuropress_amd import kernels

    L = cases.vq_layer(41, 64, 4096, 256, bits=8, act=torch.float16, m=9)  # 9 * 4096 > 16384 elements
    perm = torch.randperm(4096, generator=cases.gen(1)).to(torch.int32).to(gpu)
    assert not kernels.vq_linear_perm_supported(9, 64, 4096, 256, 8, 8)
    # 28672 rows are more blocks than compute units: the permuted kernel must leave room for two per CU.
    assert kernels.vq_linear_perm_supported(1, 28672, 4096, 4096, 8, 16)      # 74 KiB of LDS
    assert not kernels.vq_linear_perm_supported(2, 28672, 4096, 4096, 8, 16)  # 98 KiB
    # 14336 rows are fewer blocks (of four row tiles) than compute units: one per CU either way.
    assert kernels.vq_linear_perm_supported(2, 14336, 4096, 4096, 8, 16)
    with pytest.raises(RuntimeError, match="column_perm needs"):
        kernels.vq_linear(L["x"].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), 8, 8, None, 64, column_perm=perm)
    with pytest.raises(RuntimeError, match="int32"):
        kernels.vq_linear(L["x"][:4].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), 8, 8, None, 64,
                          column_perm=perm.long())
    y = kernels.vq_linear(L["x"][:4].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), 8, 8, None, 64, column_perm=perm)
    w = L["cb"][L["idx"]].reshape(64, 4096).float()
    ref = L["x"][:4][:, perm.cpu().long()].float() @ w.T
    assert (y.float().cpu() - ref).abs().max().item() < 1e-2


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
def test_vq_gemv_precast_codebook(gpu, oracle_lib, act):
    from neuropress_amd import kernels

    L = cases.vq_layer(31, 64, 512, 4096, act=act, m=2, std=0.05)
    y = kernels.vq_linear(L["x"].to(gpu), L["packed"].to(gpu), L["cb"].to(act).to(gpu), 12, 8, None, 64)
    _check(y, _vq_ref(oracle_lib, L, act))


@pytest.mark.parametrize("vl,bits,nc,k", [(4, 10, 1024, 96), (8, 14, 16384, 72), (8, 16, 65536, 200), (2, 4, 16, 64)])
@pytest.mark.parametrize("m", [1, 3])
def test_vq_gemv_generic_path(gpu, oracle_lib, vl, bits, nc, k, m):
    from neuropress_amd import kernels

    L = cases.vq_layer(300 + bits, 37, k, nc, vl=vl, bits=bits, act=torch.float16, m=m, bias=True, std=0.05)
    y = kernels.vq_linear(L["x"].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), bits, vl, L["bias"].to(gpu), 37)
    _check(y, _vq_ref(oracle_lib, L, torch.float16))


@pytest.mark.parametrize("bits", [4, 8, 10, 12, 14, 16])
@pytest.mark.parametrize("m", [1, 17, 130])
def test_vq_gemm_tile_reference_shapes(gpu, oracle_lib, bits, m):
    """The reference's Triton test shapes (tests/nn/test_vq_triton.py:11-29): N=72, K=96, VL=4, bf16."""
    from neuropress_amd import kernels

    nc = min(1 << bits, 4096)
    L = cases.vq_layer(400 + bits, 72, 96, nc, vl=4, bits=bits, act=torch.bfloat16, m=m, bias=True, std=1.0)
    y = kernels.vq_gemm_tile(L["x"].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), bits, 72, L["bias"].to(gpu))
    ref = _vq_ref(oracle_lib, L, torch.bfloat16)
    # K=96 with unit-variance weights: the reference's own tolerance for this case.
    assert np.allclose(y.float().cpu().numpy(), ref, rtol=2e-2, atol=5e-2)


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bits,nc", [(8, 256), (12, 4096), (16, 65536)])
@pytest.mark.parametrize("m", [1, 17, 96, 130, 300])
@pytest.mark.parametrize("vl", [8, 4])
def test_vq_gemm_tile_fast_path(gpu, oracle_lib, act, bits, nc, m, vl):
    from neuropress_amd import kernels

    # N = 300 spans two 256-column blocks with a ragged tail; K = 448 = 3.5 macro-steps.
    L = cases.vq_layer(500 + bits + m, 300, 448, nc, vl=vl, bits=bits, act=act, m=m, bias=True, std=0.05)
    y = kernels.vq_gemm_tile(L["x"].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), bits, 300, L["bias"].to(gpu))
    _check(y, _vq_ref(oracle_lib, L, act))


@pytest.mark.parametrize("k", [64, 128, 192])
@pytest.mark.parametrize("m", [1, 130, 300])
def test_tile_gemm_short_reductions(gpu, oracle_lib, k, m):
    """One to three 64-k steps: fewer steps than x tiles in flight (two or three) and than the
    producers' pipeline is deep, so every prefetch past the end re-reads the last step."""
    from neuropress_amd import kernels

    for nc, bits in ((256, 8), (65536, 16)):
        L = cases.vq_layer(640 + k + m, 150, k, nc, bits=bits, act=torch.bfloat16, m=m, bias=True, std=0.05)
        y = kernels.vq_gemm_tile(L["x"].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), bits, 150, L["bias"].to(gpu))
        _check(y, _vq_ref(oracle_lib, L, torch.bfloat16))
    for nbits in (4, 8):
        Q = cases.q4_layer(650 + k + m, 150, k, nbits=nbits, gs=32, act=torch.float16, m=m, bias=True)
        y = kernels.q_gemm_tile(Q["x"].to(gpu), Q["blob"].to(gpu), Q["scale"].to(gpu), nbits, 32, None, Q["bias"].to(gpu))
        _check(y, _q_ref(oracle_lib, Q, torch.float16))


def _rvq_ref(oracle_lib, L, act):
    code = orc.torch_dtype_code(act)
    w = oracle_lib.rvq_decode(L["pm"].numpy(), L["bm"], L["pr"].numpy(), L["br"], orc.to_bits(L["cbm"]),
                              orc.to_bits(L["cbr"]), orc.to_bits(L["scale"]), orc.to_bits(L["wbias"]),
                              L["n"], L["k"], code)
    return oracle_lib.linear_f64(orc.to_bits(L["x"]), code, w, code)


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,tile", [(1, False), (4, False), (25, False), (4, True), (150, True)])
def test_rvq_linear(gpu, oracle_lib, act, m, tile):
    from neuropress_amd import kernels

    L = cases.rvq_layer(9, 80, 256, act=act, m=m)
    y = kernels.rvq_linear(L["x"].to(gpu), L["pm"].to(gpu), L["bm"], L["pr"].to(gpu), L["br"], L["cbm"].to(gpu),
                           L["cbr"].to(gpu), L["scale"].to(gpu), L["wbias"].to(gpu), 80, None, tile=tile)
    _check(y, _rvq_ref(oracle_lib, L, act))


@pytest.mark.parametrize("nc_main,nc_res", [(65536, 200), (65536, 40000), (4096, 256), (256, 130)])
@pytest.mark.parametrize("m", [1, 20])
def test_rvq_gemv_residual_table_sizes(gpu, oracle_lib, nc_main, nc_res, m):
    """The fused GEMV keeps a small residual codebook in LDS (a table that is not a power of two
    long included) and looks a large one up in memory; both against the oracle."""
    from neuropress_amd import kernels

    L = cases.rvq_layer(400 + nc_res, 96, 512, nc_main=nc_main, nc_res=nc_res, act=torch.float16, m=m)
    y = kernels.rvq_linear(L["x"].to(gpu), L["pm"].to(gpu), L["bm"], L["pr"].to(gpu), L["br"], L["cbm"].to(gpu),
                           L["cbr"].to(gpu), L["scale"].to(gpu), L["wbias"].to(gpu), 96, None, tile=False)
    _check(y, _rvq_ref(oracle_lib, L, torch.float16))


def _q_ref(oracle_lib, L, act):
    code = orc.torch_dtype_code(act)
    w = oracle_lib.q_decode(L["blob"].numpy(), orc.to_bits(L["scale"]),
                            None if L["zp"] is None else orc.to_bits(L["zp"]), L["nbits"], L["gs"], code)
    bias = None if L["bias"] is None else orc.to_bits(L["bias"])
    return oracle_lib.linear_f64(orc.to_bits(L["x"]), code, w, code, bias, code)


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,k", [(301, 384), (64, 4096), (37, 14336), (5, 2048 + 128), (4200, 256), (8300, 256)])
@pytest.mark.parametrize("gs", [32, 128])
@pytest.mark.parametrize("m", [1, 2])
@pytest.mark.parametrize("asym", [False, True])
def test_q4_rowwise_gemv(gpu, oracle_lib, act, n, k, gs, m, asym):
    """One fp16 token takes the row-wise kernel (nibbles read as base + q, group offsets folded
    out), two tokens and bf16 the MFMA GEMV.  Row counts that are not a multiple of the rows per wave
    (8300 rows: two per wave), K of one partial pass, of several passes (14336: eight waves per
    block) and of a partial last pass."""
    from neuropress_amd import kernels

    L = cases.q4_layer(700 + n + m, n, k, gs=gs, act=act, m=m, bias=True, asym=asym)
    zp = None if L["zp"] is None else L["zp"].to(gpu)
    y = kernels.q_linear(L["x"].to(gpu), L["blob"].to(gpu), L["scale"].to(gpu), 4, gs, zp, L["bias"].to(gpu))
    assert y.shape == (m, n) and y.dtype == act
    _check(y, _q_ref(oracle_lib, L, act))


@pytest.mark.parametrize("n,k", [(301, 384), (64, 4096), (37, 14336), (5, 2048 + 128), (4200, 256), (13000, 128),
                                 (20000, 64)])
@pytest.mark.parametrize("gs", [32, 64])
@pytest.mark.parametrize("asym", [False, True])
def test_q4_stream_gemv(gpu, oracle_lib, monkeypatch, n, k, gs, asym):
    """The resident-grid int4 GEMV (one fp16 token; taken by itself only for layers with many
    rows, forced here with NPAMD_Q4_STREAM=2): K of one partial pass, of one and of several whole
    passes and of a partial last pass; rows fewer than the row lanes of a block; one, two, an even
    and an odd number of iterations; rows that do not fill the last iteration."""
    from neuropress_amd import _lib, kernels

    if k % gs:
        pytest.skip("K not a multiple of the group size")
    L = cases.q4_layer(800 + n, n, k, gs=gs, act=torch.float16, m=1, bias=True, asym=asym)
    zp = None if L["zp"] is None else L["zp"].to(gpu)
    monkeypatch.setenv("NPAMD_Q4_STREAM", "2")
    _lib.load().npamd_diag_reload_tuning()  # the library reads its tuning variables once
    try:
        y = kernels.q_linear(L["x"].to(gpu), L["blob"].to(gpu), L["scale"].to(gpu), 4, gs, zp, L["bias"].to(gpu))
        torch.cuda.synchronize()
    finally:
        monkeypatch.delenv("NPAMD_Q4_STREAM")
        _lib.load().npamd_diag_reload_tuning()
    assert y.shape == (1, n) and y.dtype == torch.float16
    _check(y, _q_ref(oracle_lib, L, torch.float16))
    y_rowwise = kernels.q_linear(L["x"].to(gpu), L["blob"].to(gpu), L["scale"].to(gpu), 4, gs, zp, L["bias"].to(gpu))
    assert (y.float() - y_rowwise.float()).abs().max().item() <= 2e-3 * max(1.0, y.float().abs().max().item())


@pytest.mark.parametrize("n,k", [(16384, 4096), (8192, 8192)])
def test_q4_one_token_at_the_size_where_the_launcher_changes_kernel(gpu, oracle_lib, n, k):
    """64 Mi weights: the smallest layers the launcher gives to the resident-grid kernel with
    no variable set; one fp16 token against the oracle."""
    from neuropress_amd import kernels

    L = cases.q4_layer(77, n, k, gs=32, act=torch.float16, m=1, bias=True)
    y = kernels.q_linear(L["x"].to(gpu), L["blob"].to(gpu), L["scale"].to(gpu), 4, 32, None, L["bias"].to(gpu))
    _check(y, _q_ref(oracle_lib, L, torch.float16))


@pytest.mark.parametrize("asym", [False, True])
def test_q4_rowwise_gemv_large_activations(gpu, asym):
    """Activations of a few hundred: the folded-out offset (72 * sum x) is then far larger than
    the result.  Checked against the contraction with the unrounded weight (q - zp) * s in
    float64 (what the reference's fused kernel computes, kernels/q4_linear.cu:113-122): the
    only error left must be the fp16 rounding of the output."""
    from neuropress_amd import kernels

    L = cases.q4_layer(731, 96, 4096, gs=32, act=torch.float16, m=1, asym=asym)
    x = (L["x"].float() * 300).to(torch.float16)
    zp = L["zp"].double().reshape(96, 128).repeat_interleave(32, dim=1) if asym else 8
    q = torch.stack([L["blob"] & 0xF, L["blob"] >> 4], dim=-1).reshape(96, 4096).double() - zp
    w = q * L["scale"].double().reshape(96, 128).repeat_interleave(32, dim=1)
    ref = x.double() @ w.T
    y = kernels.q_linear(x.to(gpu), L["blob"].to(gpu), L["scale"].to(gpu), 4, 32,
                         L["zp"].to(gpu) if asym else None).cpu().double()
    assert ((y - ref).abs() <= 2.0 ** -10 * ref.abs() + 1e-2).all()


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("m", [1, 16, 17, 200])
@pytest.mark.parametrize("nbits,asym", [(4, False), (4, True), (8, False), (8, True)])
def test_q4_linear_fast_path(gpu, oracle_lib, act, gs, m, nbits, asym):
    """4 and 8 bits, with and without zero points, on the MFMA GEMV (<= 16 tokens) and tile GEMM."""
    from neuropress_amd import kernels

    L = cases.q4_layer(600 + gs + m, 300, 384, nbits=nbits, gs=gs, act=act, m=m, bias=True, asym=asym)
    zp = None if L["zp"] is None else L["zp"].to(gpu)
    y = kernels.q_linear(L["x"].to(gpu), L["blob"].to(gpu), L["scale"].to(gpu), nbits, gs, zp, L["bias"].to(gpu))
    assert y.shape == (m, 300)
    _check(y, _q_ref(oracle_lib, L, act))


@pytest.mark.parametrize("rows", [1, 2, 4])
@pytest.mark.parametrize("m", [1, 5, 16, 29])
def test_gemv_row_tiles_per_block(gpu, oracle_lib, monkeypatch, rows, m):
    """The fused GEMV shares x between 1, 2 or 4 row tiles of a block; which one a layer gets
    depends on its row count and the device's size, so every variant is forced here (tuning
    override NPAMD_GEMV_R) on ragged shapes: codebook in LDS, codebook gathered from memory,
    fused column permutation, int4, residual VQ."""
    from neuropress_amd import _lib, kernels

    monkeypatch.setenv("NPAMD_GEMV_R", str(rows))
    _lib.load().npamd_diag_reload_tuning()  # the library reads its tuning variables once
    n, k = 200, 576  # 12.5 row tiles, 9 chunks of 64
    for bits, nc in ((8, 256), (16, 65536)):
        L = cases.vq_layer(900 + bits + m, n, k, nc, bits=bits, act=torch.bfloat16, m=m, bias=True, std=0.05)
        dev = {key: L[key].to(gpu) for key in ("x", "packed", "cb", "bias")}
        y = kernels.vq_linear(dev["x"], dev["packed"], dev["cb"], bits, 8, dev["bias"], out_features=n)
        _check(y, _vq_ref(oracle_lib, L, torch.bfloat16))
        if nc == 256 and m <= 16:  # the permuted GEMV takes up to 16 tokens
            perm = torch.randperm(k, generator=cases.gen(3 + m))
            yp = kernels.vq_linear(dev["x"], dev["packed"], dev["cb"], bits, 8, dev["bias"], out_features=n,
                                   column_perm=perm.to(torch.int32).to(gpu))
            _check(yp, _vq_ref(oracle_lib, dict(L, x=L["x"][:, perm].contiguous()), torch.bfloat16))
    Q = cases.q4_layer(950 + m, n, k, gs=32, act=torch.bfloat16, m=m, bias=True)
    y = kernels.q_linear(Q["x"].to(gpu), Q["blob"].to(gpu), Q["scale"].to(gpu), 4, 32, None, Q["bias"].to(gpu))
    _check(y, _q_ref(oracle_lib, Q, torch.bfloat16))
    R = cases.rvq_layer(11 + m, 80, 256, act=torch.float16, m=m)
    y = kernels.rvq_linear(R["x"].to(gpu), R["pm"].to(gpu), R["bm"], R["pr"].to(gpu), R["br"], R["cbm"].to(gpu),
                           R["cbr"].to(gpu), R["scale"].to(gpu), R["wbias"].to(gpu), 80, None, tile=False)
    _check(y, _rvq_ref(oracle_lib, R, torch.float16))
    monkeypatch.delenv("NPAMD_GEMV_R")
    _lib.load().npamd_diag_reload_tuning()


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kind", ["vq12", "vq16", "vq12_vl4", "vq16_vl4", "vq10_vl4", "rvq", "q4", "q4_asym", "q4_asym_gs128", "q8", "q8_asym", "q8_gs128", "q2_asym"])
def test_fused_kernels_decode_bit_exactly(gpu, act, kind):
    """One-hot activations read the decoded weight back through the contraction kernels: with
    x = rows of the identity, y[m, n] is the single product 1 * W[n, k_m], which f32 accumulation
    and the final rounding leave untouched.  So the MFMA GEMV (16 rows at a time) and the tile
    GEMM (all K rows at once; on this shape it splits the reduction in two) must reproduce the one-pass
    decode, itself checked bit for bit against the oracle, exactly."""
    from neuropress_amd import _lib, kernels

    n, k = 200, 1024
    assert _lib.load().npamd_gemm_tile_workspace_bytes(230, n, k) > 0  # this shape splits the reduction
    if kind.startswith("vq"):
        bits = int(kind[2:4])
        vl = 4 if kind.endswith("vl4") else 8  # 10-bit stream: the element-wise kernels
        L = cases.vq_layer(61 + bits, n, k, 1 << bits, vl=vl, bits=bits, act=act, m=1, std=0.05)
        pk, cb = L["packed"].to(gpu), L["cb"].to(gpu)
        w = kernels.vq_dequant(pk, cb, bits, n, k, act)
        gemv = lambda x: kernels.vq_linear(x, pk, cb, bits, vl, None, n)
        tile = lambda x: kernels.vq_gemm_tile(x, pk, cb, bits, n, None)
    elif kind == "rvq":
        L = cases.rvq_layer(62, n, k, act=act, m=1)
        d = {key: (v.to(gpu) if torch.is_tensor(v) else v) for key, v in L.items()}
        args = (d["pm"], L["bm"], d["pr"], L["br"], d["cbm"], d["cbr"], d["scale"], d["wbias"], n)
        w = kernels.rvq_dequant(*args, k, act)
        gemv = lambda x: kernels.rvq_linear(x, *args, None, tile=False)
        tile = lambda x: kernels.rvq_linear(x, *args, None, tile=True)
    else:
        nbits = int(kind[1])  # 2 bits: the element-wise kernels
        gs = 128 if kind.endswith("gs128") else 32
        L = cases.q4_layer(63, n, k, nbits=nbits, gs=gs, act=act, m=1, asym="asym" in kind)
        blob, sc = L["blob"].to(gpu), L["scale"].to(gpu)
        zp = None if L["zp"] is None else L["zp"].to(gpu)
        w = kernels.q_dequant(blob, sc, nbits, gs, zp, act)
        gemv = lambda x: kernels.q_linear(x, blob, sc, nbits, gs, zp)
        tile = lambda x: kernels.q_gemm_tile(x, blob, sc, nbits, gs, zp)
    eye = torch.eye(k, dtype=act, device=gpu)
    wt = w.t().contiguous()  # [K, N]: row k is what token "one-hot k" must produce
    for k0 in (0, 48, k - 16):
        assert torch.equal(gemv(eye[k0:k0 + 16]), wt[k0:k0 + 16]), f"GEMV, rows {k0}.."
    assert torch.equal(gemv(eye[40:72]), wt[40:72]), "GEMV, 32 tokens (two token tiles)"
    assert torch.equal(gemv(eye[5:26]), wt[5:26]), "GEMV, 21 tokens"
    assert torch.equal(gemv(eye[7:9]), wt[7:9])   # two tokens (int4: still the MFMA kernel)
    assert torch.equal(tile(eye), wt), "tile GEMM, 1024 tokens"
    assert torch.equal(tile(eye[100:330]), wt[100:330]), "tile GEMM, 230 tokens"


@pytest.fixture
def gemv_parts(monkeypatch):
    """Sets NPAMD_GEMV_PARTS (rows of an MFMA tile traded for parts of k) for one test; the
    library reads its tuning variables once, so they are re-read on the way in and out."""
    from neuropress_amd import _lib

    def force(parts: int):
        monkeypatch.setenv("NPAMD_GEMV_PARTS", str(parts))
        _lib.load().npamd_diag_reload_tuning()

    yield force
    monkeypatch.delenv("NPAMD_GEMV_PARTS", raising=False)
    _lib.load().npamd_diag_reload_tuning()


@pytest.mark.parametrize("parts,m", [(2, 1), (2, 5), (2, 8), (4, 1), (4, 3), (4, 4), (4, 7), (2, 12)])
@pytest.mark.parametrize("n,k", [(37, 192), (100, 1088), (8, 64), (260, 4160)])
@pytest.mark.parametrize("kind", ["vq8", "vq12", "vq16_bf16", "vq12_vl4", "rvq", "q4", "q4_asym", "q8"])
def test_gemv_rows_traded_for_k_parts(gpu, oracle_lib, gemv_parts, kind, n, k, parts, m):
    """The fused GEMV with 8 or 4 rows x 2 or 4 parts of k per MFMA tile (taken by itself for
    layers of few rows; forced here): row counts that do not fill a tile, K of one chunk, K whose
    chunks do not fill the last step, every token count a tile holds — and one above
    (7 tokens at four parts, 12 at two), which must fall back to whole tiles.  Table in LDS
    (256 and 4096 rows, the residual's 256) and in memory (65536 rows)."""
    from neuropress_amd import kernels

    gemv_parts(parts)
    if kind.startswith("vq"):
        bits = int(kind[2:].split("_")[0])
        act = torch.bfloat16 if kind.endswith("bf16") else torch.float16
        vl = 4 if kind.endswith("vl4") else 8
        L = cases.vq_layer(300 + bits + m, n, k, 1 << bits, vl=vl, bits=bits, act=act, m=m, bias=True)
        y = kernels.vq_linear(L["x"].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), bits, vl, L["bias"].to(gpu), n)
        ref = _vq_ref(oracle_lib, L, act)
    elif kind == "rvq":
        L = cases.rvq_layer(310 + m, n, k, act=torch.float16, m=m)
        y = kernels.rvq_linear(L["x"].to(gpu), L["pm"].to(gpu), L["bm"], L["pr"].to(gpu), L["br"], L["cbm"].to(gpu),
                               L["cbr"].to(gpu), L["scale"].to(gpu), L["wbias"].to(gpu), n, None, tile=False)
        ref = _rvq_ref(oracle_lib, L, torch.float16)
    else:
        nbits = int(kind[1])
        L = cases.q4_layer(320 + m, n, k, nbits=nbits, gs=32, act=torch.float16, m=m, asym="asym" in kind, bias=True)
        zp = None if L["zp"] is None else L["zp"].to(gpu)
        y = kernels.q_linear(L["x"].to(gpu), L["blob"].to(gpu), L["scale"].to(gpu), nbits, 32, zp, L["bias"].to(gpu))
        ref = _q_ref(oracle_lib, L, torch.float16)
    assert y.shape == (m, n)
    _check(y, ref)


@pytest.fixture
def gemv_tuning(monkeypatch):
    """Sets NPAMD_* tuning variables for one test (the library reads them once: they are re-read on
    the way in and out)."""
    from neuropress_amd import _lib

    names = []

    def force(**variables):
        for name, value in variables.items():
            monkeypatch.setenv(name, str(value))
            names.append(name)
        _lib.load().npamd_diag_reload_tuning()

    yield force
    for name in names:
        monkeypatch.delenv(name, raising=False)
    _lib.load().npamd_diag_reload_tuning()


@pytest.mark.parametrize("m", [1, 9, 16, 17, 25, 32])
@pytest.mark.parametrize("n,k", [(37, 192), (100, 1088), (260, 4160)])
@pytest.mark.parametrize("kind", ["vq16", "vq16_bf16", "vq12_mem", "vq12_vl4_mem", "rvq", "q4", "q4_asym", "q8"])
def test_gemv_staged_activations(gpu, oracle_lib, gemv_tuning, kind, n, k, m):
    """The fused GEMV with a step's activations staged through a per-wave LDS area (taken by itself
    from three tokens on layers of one row tile per block; forced here at every token count, whole
    tiles): token counts on both sides of a token tile, rows past M, K whose chunks do not fill
    the last step, lookups from memory and (residual VQ) with a table in LDS next to the staging
    areas."""
    from neuropress_amd import kernels

    tuning = {"NPAMD_GEMV_XSTAGE": 2, "NPAMD_GEMV_PARTS": 1}
    if kind.endswith("_mem"):
        tuning["NPAMD_GEMV_LDS_CB"] = 0
    gemv_tuning(**tuning)
    if kind.startswith("vq"):
        bits = int(kind[2:4])
        act = torch.bfloat16 if "bf16" in kind else torch.float16
        vl = 4 if "vl4" in kind else 8
        L = cases.vq_layer(500 + bits + m, n, k, 1 << bits, vl=vl, bits=bits, act=act, m=m, bias=True)
        y = kernels.vq_linear(L["x"].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), bits, vl, L["bias"].to(gpu), n)
        ref = _vq_ref(oracle_lib, L, act)
    elif kind == "rvq":
        L = cases.rvq_layer(510 + m, n, k, act=torch.float16, m=m)
        y = kernels.rvq_linear(L["x"].to(gpu), L["pm"].to(gpu), L["bm"], L["pr"].to(gpu), L["br"], L["cbm"].to(gpu),
                               L["cbr"].to(gpu), L["scale"].to(gpu), L["wbias"].to(gpu), n, None, tile=False)
        ref = _rvq_ref(oracle_lib, L, torch.float16)
    else:
        nbits = int(kind[1])
        L = cases.q4_layer(520 + m, n, k, nbits=nbits, gs=32, act=torch.float16, m=m, asym="asym" in kind, bias=True)
        zp = None if L["zp"] is None else L["zp"].to(gpu)
        y = kernels.q_linear(L["x"].to(gpu), L["blob"].to(gpu), L["scale"].to(gpu), nbits, 32, zp, L["bias"].to(gpu))
        ref = _q_ref(oracle_lib, L, torch.float16)
    assert y.shape == (m, n)
    _check(y, ref)


@pytest.mark.parametrize("kind", ["vq16", "rvq", "q4"])
def test_gemv_staged_activations_decode_bit_exactly(gpu, gemv_tuning, kind):
    """One-hot activations through the staged GEMV: every (token, k) must come back out of the
    staging area where the MFMA operand layout expects it."""
    from neuropress_amd import kernels

    n, k, act = 45, 1088, torch.float16
    if kind == "vq16":
        L = cases.vq_layer(541, n, k, 65536, bits=16, act=act, m=1, std=0.05)
        pk, cb = L["packed"].to(gpu), L["cb"].to(gpu)
        w = kernels.vq_dequant(pk, cb, 16, n, k, act)
        gemv = lambda x: kernels.vq_linear(x, pk, cb, 16, 8, None, n)
    elif kind == "rvq":
        L = cases.rvq_layer(542, n, k, act=act, m=1)
        d = {key: (v.to(gpu) if torch.is_tensor(v) else v) for key, v in L.items()}
        args = (d["pm"], L["bm"], d["pr"], L["br"], d["cbm"], d["cbr"], d["scale"], d["wbias"], n)
        w = kernels.rvq_dequant(*args, k, act)
        gemv = lambda x: kernels.rvq_linear(x, *args, None, tile=False)
    else:
        L = cases.q4_layer(543, n, k, act=act, m=1)
        blob, sc = L["blob"].to(gpu), L["scale"].to(gpu)
        w = kernels.q_dequant(blob, sc, 4, 32, None, act)
        gemv = lambda x: kernels.q_linear(x, blob, sc, 4, 32, None)
    gemv_tuning(NPAMD_GEMV_XSTAGE=2, NPAMD_GEMV_PARTS=1)
    eye = torch.eye(k, dtype=act, device=gpu)
    wt = w.t().contiguous()
    for k0, count in ((0, 16), (250, 16), (k - 32, 32), (500, 21), (1020, 9)):
        assert torch.equal(gemv(eye[k0:k0 + count]), wt[k0:k0 + count]), f"{count} tokens one-hot at {k0}"


@pytest.mark.parametrize("parts", [2, 4])
@pytest.mark.parametrize("kind", ["vq12", "vq16", "rvq", "q4"])
def test_gemv_k_parts_decode_bit_exactly(gpu, gemv_parts, kind, parts):
    """One-hot activations through the k-parts GEMV: y[m, n] is the single product 1 * W[n, k_m],
    so every (row, part, k slot) of the tile layout must land where the one-pass decode has it."""
    from neuropress_amd import kernels

    n, k, act = 45, 1024, torch.float16
    if kind.startswith("vq"):
        bits = int(kind[2:])
        L = cases.vq_layer(340 + bits, n, k, 1 << bits, bits=bits, act=act, m=1, std=0.05)
        pk, cb = L["packed"].to(gpu), L["cb"].to(gpu)
        w = kernels.vq_dequant(pk, cb, bits, n, k, act)
        gemv = lambda x: kernels.vq_linear(x, pk, cb, bits, 8, None, n)
    elif kind == "rvq":
        L = cases.rvq_layer(341, n, k, act=act, m=1)
        d = {key: (v.to(gpu) if torch.is_tensor(v) else v) for key, v in L.items()}
        args = (d["pm"], L["bm"], d["pr"], L["br"], d["cbm"], d["cbr"], d["scale"], d["wbias"], n)
        w = kernels.rvq_dequant(*args, k, act)
        gemv = lambda x: kernels.rvq_linear(x, *args, None, tile=False)
    else:
        L = cases.q4_layer(342, n, k, act=act, m=1)
        blob, sc = L["blob"].to(gpu), L["scale"].to(gpu)
        w = kernels.q_dequant(blob, sc, 4, 32, None, act)
        gemv = lambda x: kernels.q_linear(x, blob, sc, 4, 32, None)
    gemv_parts(parts)
    eye = torch.eye(k, dtype=act, device=gpu)
    wt = w.t().contiguous()
    tokens = 16 // parts
    for k0 in range(0, k, 8 * tokens // 2 + 24):  # windows that straddle chunks and steps
        k1 = min(k0 + tokens, k)
        if kind == "q4" and k1 - k0 < 2:
            continue  # one token of int4 takes the row-wise kernel
        assert torch.equal(gemv(eye[k0:k1]), wt[k0:k1]), f"tokens one-hot at {k0}..{k1}"


@pytest.mark.parametrize("nbits,gs,asym", [(4, 32, True), (8, 32, False), (2, 16, True), (1, 8, False), (4, 24, False)])
@pytest.mark.parametrize("m", [2, 20])
def test_q_linear_generic_path(gpu, oracle_lib, nbits, gs, asym, m):
    from neuropress_amd import kernels

    L = cases.q4_layer(700 + nbits, 21, gs * 4, nbits=nbits, gs=gs, act=torch.float16, m=m, asym=asym, bias=True)
    y = kernels.q_linear(L["x"].to(gpu), L["blob"].to(gpu), L["scale"].to(gpu), nbits, gs,
                         None if L["zp"] is None else L["zp"].to(gpu), L["bias"].to(gpu))
    _check(y, _q_ref(oracle_lib, L, torch.float16))


def test_q_known_answers(gpu):
    """Reference KATs (tests/test_quantized_weight_regressions.py:848-859 of the reference):
    code 15, zero point 2, scale 1 -> 13; an underflowed scale decodes the block to 0."""
    from neuropress_amd import kernels

    codes = torch.full((2, 32), 15, dtype=torch.uint8)
    from neuropress_amd.t2n.packing import BitPacking4

    blob = BitPacking4.compress(codes).to(gpu)
    scale = torch.tensor([1e-12, 1.0]).to(torch.float16).to(gpu)
    zp = torch.full((2,), 2.0, dtype=torch.float16, device=gpu)
    w = kernels.q_dequant(blob, scale, 4, 32, zp, torch.float32).cpu()
    assert torch.all(w[0] == 0) and torch.all(w[1] == 13)


# ------------------------------------------------------------------ edges ---


def test_empty_and_error_paths(gpu):
    from neuropress_amd import kernels

    L = cases.vq_layer(1, 16, 64, 256)
    cb, packed = L["cb"].to(gpu), L["packed"].to(gpu)
    y = kernels.vq_linear(torch.empty(0, 64, device=gpu, dtype=torch.float16), packed, cb, 8, 8, None, 16)
    assert y.shape == (0, 16)
    with pytest.raises(RuntimeError, match="too short"):
        kernels.vq_dequant(packed[:10], cb, 8, 16, 64, torch.float16)
    with pytest.raises(RuntimeError, match="bits"):
        kernels.vq_dequant(packed, cb, 3, 16, 64, torch.float16)
    with pytest.raises(RuntimeError, match="exceeds the fused limit"):
        kernels.vq_linear(torch.zeros(33, 64, device=gpu, dtype=torch.float16), packed, cb, 8, 8, None, 16)
    with pytest.raises(RuntimeError, match="GPU"):
        kernels.vq_dequant(L["packed"], L["cb"], 8, 16, 64, torch.float16)
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        kernels.vq_linear(torch.zeros(1, 64, device=gpu), packed, cb, 8, 8, None, 16)


def test_out_of_range_index_is_clamped(gpu):
    """A 16-bit stream pointing past a small codebook must not read outside it."""
    from neuropress_amd import kernels
    from neuropress_amd.transforms.vq_packing import IndexPacking

    cb = torch.arange(4 * 8, dtype=torch.float16).reshape(4, 8).to(gpu)
    packed = IndexPacking.pack(torch.tensor([0, 3, 60000, 65535] * 2), 16).to(gpu)
    w = kernels.vq_dequant(packed, cb, 16, 1, 64, torch.float16)
    assert torch.equal(w.reshape(8, 8)[2], cb[3]) and torch.equal(w.reshape(8, 8)[3], cb[3])


def test_strided_x_and_stream(gpu, oracle_lib):
    """Row-strided activations and a non-default stream."""
    from neuropress_amd import kernels

    L = cases.vq_layer(77, 48, 256, 256, m=3)
    xbig = torch.zeros(3, 512, dtype=torch.float16, device=gpu)
    xbig[:, :256] = L["x"].to(gpu)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        y = kernels.vq_linear(xbig[:, :256], L["packed"].to(gpu), L["cb"].to(gpu), 8, 8, None, 48)
    s.synchronize()
    _check(y, _vq_ref(oracle_lib, L, torch.float16))


# ------------------------------------------------------------------ split-K ---


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [17, 130, 400])
@pytest.mark.parametrize("k", [1024, 2048 + 64])
def test_vq_gemm_tile_split_k(gpu, oracle_lib, act, m, k):
    """Few output columns and a long K: the tile GEMM splits K over blockIdx.z and adds the
    f32 partial tiles in a second kernel (K not a multiple of the split length included)."""
    from neuropress_amd import _lib, kernels

    n = 200
    assert _lib.load().npamd_gemm_tile_workspace_bytes(m, n, k) >= 2 * m * n * 4
    L = cases.vq_layer(800 + m + k, n, k, 65536, bits=16, act=act, m=m, bias=True, std=0.05)
    y = kernels.vq_gemm_tile(L["x"].to(gpu), L["packed"].to(gpu), L["cb"].to(gpu), 16, n, L["bias"].to(gpu))
    assert y.shape == (m, n) and y.dtype == act
    _check(y, _vq_ref(oracle_lib, L, act))


@pytest.mark.parametrize("m", [40, 300])
def test_q4_and_rvq_gemm_tile_split_k(gpu, oracle_lib, m):
    from neuropress_amd import kernels

    Q = cases.q4_layer(820 + m, 136, 2048, gs=32, act=torch.float16, m=m, bias=True)
    y = kernels.q_gemm_tile(Q["x"].to(gpu), Q["blob"].to(gpu), Q["scale"].to(gpu), 4, 32, None, Q["bias"].to(gpu))
    _check(y, _q_ref(oracle_lib, Q, torch.float16))
    R = cases.rvq_layer(830 + m, 80, 1024, act=torch.float16, m=m)
    y = kernels.rvq_linear(R["x"].to(gpu), R["pm"].to(gpu), R["bm"], R["pr"].to(gpu), R["br"], R["cbm"].to(gpu),
                           R["cbr"].to(gpu), R["scale"].to(gpu), R["wbias"].to(gpu), 80, None, tile=True)
    _check(y, _rvq_ref(oracle_lib, R, torch.float16))


@pytest.mark.parametrize("bits,nc", [(8, 256), (12, 4096), (10, 600), (16, 65536)])
@pytest.mark.parametrize("m", [1, 3])
def test_vq_lut_gather_matches_a_float64_gather(gpu, oracle_lib, bits, nc, m):
    """y[m, j] = sum_g lut[m, g, idx[j, g]] (reference: kernels/vq_linear_lut.cu:121-142), against the
    same sum taken in float64 over oracle-unpacked indices; and, with the table the reference's
    caller builds from x and the codebook, against the layer's output."""
    from neuropress_amd import kernels

    n, k, vl = 70, 8 * 37, 8
    groups = k // vl
    L = cases.vq_layer(300 + bits + m, n, k, nc, bits=bits, act=torch.float16, m=m, std=0.05)
    idx = oracle_lib.unpack_indices(L["packed"].numpy(), bits, n * groups).reshape(n, groups)
    assert np.array_equal(idx, L["idx"].reshape(n, groups).numpy())
    lut = (L["x"].float().reshape(m * groups, vl) @ L["cb"].float().T).reshape(m, groups, nc)
    y = kernels.vq_lut_gather(lut.to(gpu), L["packed"].to(gpu), bits, n)
    assert y.shape == (m, n) and y.dtype == torch.float32
    want = np.take_along_axis(lut.double().numpy()[:, None, :, :], idx[None, :, :, None], axis=3)[..., 0].sum(-1)
    assert np.abs(y.cpu().numpy() - want).max() <= 1e-4
    code = orc.DT_F16
    w = oracle_lib.vq_decode(L["packed"].numpy(), bits, orc.to_bits(L["cb"]), n, k, code)
    ref = oracle_lib.linear_f64(orc.to_bits(L["x"]), code, w, code)
    ok, max_abs, _ = cases.within_tol(y.cpu().numpy(), ref)
    assert ok, max_abs
