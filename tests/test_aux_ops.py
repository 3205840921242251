"""RMSNorm and the embedding lookups of quantized tables.

CPU: the oracle's restatements against the torch op sequences the reference's modules run
(neuropress/nn/np_rms_norm.py:48-50, np_vq_embedding.py:120-142, np_embedding.py:120-183, 455-473),
written here with plain torch ops on small inputs.  GPU: the HIP kernels against the oracle -
bit-exact for the two lookups (index arithmetic plus IEEE roundings), within one unit in the last
place of a 16-bit output dtype for RMSNorm (its float summation order is the kernel's own)."""

import numpy as np
import pytest
import torch

from neuropress_amd.t2n.packing import BitPacking
from oracle import oracle as orc

DTYPES = [torch.float16, torch.bfloat16, torch.float32]


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _vq_table(seed, vocab, groups, nc, vl=8):
    g = _gen(seed)
    cb = (torch.randn(nc, vl, generator=g) * 0.05).half()
    idx = torch.randint(0, nc, (vocab, groups), generator=g)
    return cb, idx


def _torch_vq_embedding(ids, idx, cb, scale, inv_perm, out_dtype):
    out = cb[idx[ids.flatten()]].reshape(ids.numel(), -1)
    if inv_perm is not None:
        out = out[:, inv_perm]
    if scale != 1.0:
        out = out * scale
    if out_dtype is not None:
        out = out.to(out_dtype)
    return out


def _q_table(seed, vocab, dim, nbits, group_size, asym):
    g = _gen(seed)
    codes = torch.randint(0, 1 << nbits, (vocab, dim), generator=g, dtype=torch.uint8)
    scale = (torch.rand(vocab * dim // group_size, generator=g) * 0.02 + 0.001).half()
    zp = torch.randint(0, 1 << nbits, (vocab * dim // group_size,), generator=g).half() if asym else None
    return codes, BitPacking(nbits).compress(codes), scale, zp


def _torch_q_embedding(ids, codes, scale, zp, nbits, group_size, padding_idx, embed_scale, out_dtype):
    vocab, dim = codes.shape
    flat = ids.flatten()
    vals = codes[flat].float().reshape(flat.numel(), dim // group_size, group_size)
    sc = scale.reshape(vocab, -1)[flat].float().unsqueeze(-1)
    z = zp.reshape(vocab, -1)[flat].float().unsqueeze(-1) if zp is not None else float(1 << (nbits - 1))
    out = ((vals - z) * sc).reshape(flat.numel(), dim).to(scale.dtype)
    if padding_idx is not None:
        out[flat == padding_idx] = 0.0
    if out_dtype is not None:
        out = out.to(out_dtype)
    if embed_scale != 1.0:
        out = out * embed_scale
    return out


# ------------------------------------------------------------------------------ oracle, CPU ---


@pytest.mark.parametrize("dtype", DTYPES)
def test_oracle_rms_norm_matches_the_reference_expression(oracle_lib, dtype):
    g = _gen(1)
    x = (torch.randn(5, 96, generator=g) * 3).to(dtype)
    w = (torch.rand(96, generator=g) + 0.5).to(dtype)
    got = orc.rms_norm_f64(orc.to_bits(x), orc.to_bits(w), orc.torch_dtype_code(dtype), 1e-6)
    xd, wd = x.double(), w.double()
    want = xd * torch.rsqrt(xd.pow(2).mean(-1, keepdim=True) + 1e-6) * wd
    assert np.allclose(got, want.numpy(), rtol=1e-12, atol=0)
    # a unit-RMS row with unit weight is returned unchanged; scaling x leaves the result (almost) unchanged
    ones = torch.ones(1, 16, dtype=dtype)
    assert np.allclose(orc.rms_norm_f64(orc.to_bits(ones), orc.to_bits(ones[0]), orc.torch_dtype_code(dtype), 0.0), 1.0)


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("scale", [1.0, 45.25483399593904])
@pytest.mark.parametrize("perm", [False, True])
def test_oracle_vq_embedding_matches_torch_ops(oracle_lib, out_dtype, scale, perm):
    cb, idx = _vq_table(2, 50, 6, 300)
    ids = torch.tensor([[0, 49, 7], [7, 3, 21]])
    inv_perm = torch.argsort(torch.randperm(48, generator=_gen(3))) if perm else None
    want = _torch_vq_embedding(ids, idx, cb, scale, inv_perm, out_dtype)
    got = orc.vq_embedding(ids.numpy(), idx.numpy().astype(np.uint16), orc.to_bits(cb), scale,
                           None if inv_perm is None else inv_perm.numpy(), orc.torch_dtype_code(out_dtype))
    assert np.array_equal(got, orc.to_bits(want))


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("nbits,group_size,asym", [(4, 32, False), (4, 16, True), (8, 32, False), (2, 8, True), (1, 8, False)])
@pytest.mark.parametrize("embed_scale,padding_idx", [(1.0, None), (22.627416997969522, 5)])
def test_oracle_q_embedding_matches_torch_ops(oracle_lib, out_dtype, nbits, group_size, asym, embed_scale, padding_idx):
    codes, blob, scale, zp = _q_table(4, 20, 64, nbits, group_size, asym)
    ids = torch.tensor([5, 0, 19, 5, 11])
    want = _torch_q_embedding(ids, codes, scale, zp, nbits, group_size, padding_idx, embed_scale, out_dtype)
    got = orc.q_embedding(ids.numpy(), blob.numpy(), orc.to_bits(scale), None if zp is None else orc.to_bits(zp),
                          nbits, group_size, padding_idx, embed_scale, orc.torch_dtype_code(out_dtype))
    assert np.array_equal(got, orc.to_bits(want))


# ----------------------------------------------------------------------------------- GPU ---


def _ulp(ref: np.ndarray, dtype) -> np.ndarray:
    mant = {torch.float16: 10, torch.bfloat16: 7, torch.float32: 23}[dtype]
    tiny = {torch.float16: 2.0 ** -24, torch.bfloat16: 2.0 ** -133, torch.float32: 2.0 ** -149}[dtype]
    return np.maximum(2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref), 1e-300))) - mant), tiny)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,h", [(1, 640), (7, 4096), (130, 2048), (3, 8192), (5, 100), (2, 16384), (4, 8)])
def test_rms_norm_kernel(gpu, oracle_lib, dtype, m, h):
    from neuropress_amd import kernels

    g = _gen(m * 31 + h)
    x = (torch.randn(m, h, generator=g) * 2.5).to(dtype)
    w = (torch.randn(h, generator=g) * 0.3 + 1.0).to(dtype)
    y = kernels.rms_norm(x.to(gpu), w.to(gpu), 1e-6)
    assert y.shape == (m, h) and y.dtype == dtype
    ref = orc.rms_norm_f64(orc.to_bits(x), orc.to_bits(w), orc.torch_dtype_code(dtype), 1e-6)
    err = np.abs(y.double().cpu().numpy() - ref)
    # f32 arithmetic, one rounding at the store: within one unit in the last place of a 16-bit output;
    # an f32 output sees the arithmetic's own few units (sum of squares, division, square root, two products)
    tol = 8.0 if dtype == torch.float32 else 1.001
    assert (err <= tol * _ulp(ref, dtype)).all(), f"max error {np.max(err / _ulp(ref, dtype)):.2f} ulp"
    assert (err <= 1e-2 + 1e-2 * np.abs(ref)).all()


@pytest.mark.gpu
def test_rms_norm_kernel_strided_rows_and_checks(gpu, oracle_lib):
    from neuropress_amd import kernels

    x = torch.randn(6, 512, generator=_gen(9)).half()
    w = torch.ones(256).half()
    view = x.to(gpu)[:, :256]  # row stride 512
    ref = orc.rms_norm_f64(orc.to_bits(x[:, :256].contiguous()), orc.to_bits(w), 0, 1e-5)
    got = kernels.rms_norm(view, w.to(gpu), 1e-5).double().cpu().numpy()
    assert (np.abs(got - ref) <= 1.001 * _ulp(ref, torch.float16)).all()
    with pytest.raises(RuntimeError, match="share dtype"):
        kernels.rms_norm(view, w.float().to(gpu), 1e-5)
    with pytest.raises(RuntimeError, match="2-D"):
        kernels.rms_norm(view[0], w.to(gpu), 1e-5)
    with pytest.raises(RuntimeError, match="matching"):
        kernels.rms_norm(view, w[:100].to(gpu), 1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("vl,nc", [(8, 65536), (8, 300), (4, 1024)])
@pytest.mark.parametrize("scale,perm", [(1.0, False), (45.25483399593904, False), (1.0, True), (33.941125496954285, True)])
def test_vq_embedding_kernel_is_bit_exact(gpu, oracle_lib, out_dtype, vl, nc, scale, perm):
    from neuropress_amd import kernels

    vocab, groups = 1000, 80
    cb, idx = _vq_table(20 + vl, vocab, groups, nc, vl)
    ids = torch.randint(0, vocab, (3, 17), generator=_gen(5))
    ids[0, 0], ids[0, 1] = 0, vocab - 1
    inv_perm = torch.argsort(torch.randperm(groups * vl, generator=_gen(6))) if perm else None
    out = kernels.vq_embedding(ids.to(gpu), idx.to(torch.int16).to(gpu), cb.to(gpu), scale,
                               None if inv_perm is None else inv_perm.to(torch.int32).to(gpu), out_dtype)
    assert out.shape == (3, 17, groups * vl) and out.dtype == out_dtype
    want = orc.vq_embedding(ids.numpy(), idx.numpy().astype(np.uint16), orc.to_bits(cb), scale,
                            None if inv_perm is None else inv_perm.numpy(), orc.torch_dtype_code(out_dtype))
    assert np.array_equal(orc.to_bits(out.reshape(-1, groups * vl)), want)


@pytest.mark.gpu
@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("nbits,group_size,asym", [(4, 32, False), (4, 32, True), (4, 8, True), (4, 20, False),
                                                   (8, 32, True), (2, 16, False), (1, 8, True)])
@pytest.mark.parametrize("embed_scale,padding_idx", [(1.0, None), (22.627416997969522, 3)])
def test_q_embedding_kernel_is_bit_exact(gpu, oracle_lib, out_dtype, nbits, group_size, asym, embed_scale, padding_idx):
    from neuropress_amd import kernels

    vocab, dim = 500, 640 if group_size != 20 else 160
    codes, blob, scale, zp = _q_table(40 + nbits, vocab, dim, nbits, group_size, asym)
    ids = torch.randint(0, vocab, (2, 33), generator=_gen(7))
    ids[0, :3] = torch.tensor([3, 0, vocab - 1])
    out = kernels.q_embedding(ids.to(gpu), blob.to(gpu), scale.to(gpu), nbits, group_size,
                              None if zp is None else zp.to(gpu), padding_idx, embed_scale, out_dtype)
    assert out.shape == (2, 33, dim) and out.dtype == out_dtype
    want = orc.q_embedding(ids.numpy(), blob.numpy(), orc.to_bits(scale), None if zp is None else orc.to_bits(zp),
                           nbits, group_size, padding_idx, embed_scale, orc.torch_dtype_code(out_dtype))
    assert np.array_equal(orc.to_bits(out.reshape(-1, dim)), want)


@pytest.mark.gpu
def test_embedding_wrappers_reject_bad_input(gpu):
    from neuropress_amd import kernels

    cb, idx = _vq_table(1, 10, 4, 16)
    ids = torch.tensor([1, 2]).to(gpu)
    with pytest.raises(RuntimeError, match="int16"):
        kernels.vq_embedding(ids, idx.to(gpu), cb.to(gpu))
    with pytest.raises(RuntimeError, match="inv_perm must be int32"):
        kernels.vq_embedding(ids, idx.to(torch.int16).to(gpu), cb.to(gpu), inv_perm=torch.arange(32).to(gpu))
    with pytest.raises(RuntimeError, match="nbits must be"):
        kernels.q_embedding(ids, torch.zeros(10, 8, dtype=torch.uint8).to(gpu), torch.ones(10).half().to(gpu), 3, 8)
    with pytest.raises(RuntimeError, match="scale has"):
        kernels.q_embedding(ids, torch.zeros(10, 8, dtype=torch.uint8).to(gpu), torch.ones(7).half().to(gpu), 4, 16)
    empty = kernels.vq_embedding(torch.zeros(0, dtype=torch.int64).to(gpu), idx.to(torch.int16).to(gpu), cb.to(gpu))
    assert empty.shape == (0, 32)
