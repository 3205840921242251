"""NPRMSNorm, NPVQEmbedding, NPEmbedding and their lowering passes on the CPU (torch-op paths and
host logic); the GPU kernels behind them are tested in tests/test_aux_ops.py and tests/test_gpu_aux_modules.py."""

import pytest
import torch
import torch.nn as nn

import neuropress_amd.nn.np_rms_norm as rms_mod
from neuropress_amd import AutoKernelLowering, is_lowered, unlower_model
from neuropress_amd.nn import NPEmbedding, NPRMSNorm, NPVQEmbedding, linearize_qtensor_embeddings, linearize_vq_embeddings
from neuropress_amd.nn.np_embedding import _emb_dequant, _resolve_backend_emb
from neuropress_amd.qweights import ScalarQWeight, VQWeight, attach_quantized_weight


class LlamaRMSNorm(nn.Module):
    def __init__(self, h, eps=1e-5):
        super().__init__()
        self.weight = nn.Parameter(torch.rand(h) + 0.5)
        self.eps = eps

    def forward(self, x):
        xf = x.float()
        return (self.weight.float() * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps))).to(x.dtype)


class GemmaRMSNorm(LlamaRMSNorm):
    def __init__(self, h, eps=1e-6):
        super().__init__(h, eps)
        self.weight = nn.Parameter(torch.randn(h) * 0.1)

    def forward(self, x):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps) * (1.0 + self.weight.float())).to(x.dtype)


class ScaledEmbedding(nn.Embedding):
    def __init__(self, n, d, padding_idx=None, embed_scale=1.0):
        super().__init__(n, d, padding_idx=padding_idx)
        self.embed_scale = embed_scale


def _q_embedding(vocab=40, dim=64, asym=False, padding_idx=None, embed_scale=1.0, seed=0, dtype=torch.float16):
    g = torch.Generator().manual_seed(seed)
    codes = torch.randint(0, 16, (vocab, dim), generator=g, dtype=torch.uint8)
    scale = (torch.rand(vocab * dim // 32, generator=g) * 0.02 + 0.001).half()
    zp = torch.randint(0, 16, (vocab * dim // 32,), generator=g).half() if asym else None
    emb = ScaledEmbedding(vocab, dim, padding_idx=padding_idx, embed_scale=embed_scale)
    attach_quantized_weight(emb, ScalarQWeight.from_codes(codes, scale, 4, 32, zero_point=zp, dequant_to_dtype=dtype))
    return emb, codes, scale, zp


def _vq_embedding(vocab=30, dim=48, nc=600, perm=False, embed_scale=1.0, seed=0, **coded):
    g = torch.Generator().manual_seed(seed)
    cb = (torch.randn(nc, 8, generator=g) * 0.05).half()
    idx = torch.randint(0, nc, (vocab * dim // 8,), generator=g)
    p = torch.randperm(dim, generator=g) if perm else None
    emb = ScaledEmbedding(vocab, dim, embed_scale=embed_scale)
    attach_quantized_weight(emb, VQWeight.from_indices(idx, cb, vocab, dim, column_permutation=p, **coded))
    table = cb[idx].reshape(vocab, dim)
    if p is not None:
        table = table[:, torch.argsort(p)]
    return emb, table


def test_rms_norm_module_matches_both_conventions_on_cpu():
    x = torch.randn(3, 5, 32)
    for src in (LlamaRMSNorm(32), GemmaRMSNorm(32)):
        plus_one = rms_mod._uses_plus_one_convention(src, src.weight.data)
        assert plus_one == isinstance(src, GemmaRMSNorm)
        saved = src.weight.detach().clone()
        fused = NPRMSNorm(1.0 + src.weight.data if plus_one else src.weight.data, eps=src.eps, source=src)
        assert torch.equal(src.weight, saved)  # the probe restores the weight
        assert torch.allclose(fused(x), src(x), atol=1e-6)
        assert fused.to_source_module() is src and set(fused.state_dict()) == {"weight"}
    assert rms_mod._is_unfused_rms_norm(LlamaRMSNorm(8)) and not rms_mod._is_unfused_rms_norm(nn.LayerNorm(8))
    assert not rms_mod._is_unfused_rms_norm(NPRMSNorm(torch.ones(8)))
    assert rms_mod.linearize_rms_norms(nn.Sequential(LlamaRMSNorm(8))) == 0  # nothing on a GPU here


@pytest.mark.parametrize("asym", [False, True])
@pytest.mark.parametrize("backend", ["default", "compile", "auto"])
def test_npembedding_backends_match_the_specification(asym, backend):
    emb, codes, scale, zp = _q_embedding(asym=asym, padding_idx=3, embed_scale=8.0, dtype=torch.bfloat16)
    layer = NPEmbedding.from_embedding(emb, backend)
    assert layer.backend.value == ("compile" if backend == "auto" else backend) and layer.qtype == ("asym" if asym else "sym")
    ids = torch.tensor([[3, 0, 39], [7, 3, 21]])
    z = zp.reshape(40, 2)[ids.flatten()].float().unsqueeze(-1) if asym else 8.0
    want = ((codes[ids.flatten()].float().reshape(6, 2, 32) - z) * scale.reshape(40, 2)[ids.flatten()].float().unsqueeze(-1))
    want = want.reshape(6, 64).half()
    if backend != "default":  # F.embedding does not zero the padding row in forward (nor does the reference's default path)
        want[ids.flatten() == 3] = 0
    want = (want.to(torch.bfloat16) * 8.0).reshape(2, 3, 64)
    got = layer(ids)
    assert got.dtype == torch.bfloat16 and torch.equal(got, want)
    assert _emb_dequant(ids, layer.u8_blob, layer.scale, 4, 32, layer.zero_point).shape == want.shape
    back = layer.to_qtensor()
    assert torch.equal(back.u8_blob, emb.weight.u8_blob) and torch.equal(back.qscheme.scale.flatten(), scale)
    assert "padding_idx=3" in layer.extra_repr()


def test_npembedding_errors_and_backend_switch():
    emb, *_ = _q_embedding()
    layer = NPEmbedding.from_embedding(emb, "compile")
    with pytest.raises(RuntimeError, match="original QTensor was not retained"):
        layer.set_backend("default")
    assert layer.set_backend("cuda").backend.value == "cuda"
    with pytest.raises(ValueError):
        _resolve_backend_emb("gemlite")
    with pytest.raises(TypeError, match="Unsupported weight type"):
        NPEmbedding.from_embedding(nn.Embedding(4, 8))
    with pytest.raises(ValueError, match="weight_q is required"):
        NPEmbedding(layer.u8_blob, layer.scale, 40, 64, 32, 4, "sym", "default")


@pytest.mark.parametrize("perm", [False, True])
@pytest.mark.parametrize("coded", [{}, {"use_tiered": True}, {"tier_bits": [4, 8, 10]}, {"zero_escape": True}])
def test_vq_embedding_lowering_on_cpu(perm, coded):
    emb, table = _vq_embedding(perm=perm, embed_scale=6.5, **coded)
    model = nn.Sequential(emb, nn.Linear(48, 4).half())
    assert linearize_vq_embeddings(model) == 1
    layer = model[0]
    assert isinstance(layer, NPVQEmbedding) and layer.out_dtype == torch.float16 and layer.scale == 6.5
    assert [n for n, _ in model.named_children() if n.startswith("_vq_emb_proxy_")] == ["_vq_emb_proxy_0"]
    ids = torch.tensor([[0, 29], [5, 5]])
    want = (table[ids.flatten()] * 6.5).reshape(2, 2, 48)
    assert torch.equal(layer(ids), want)
    assert layer.weight.shape == (30, 48) and torch.equal(layer.weight[5], want[1, 0])
    assert layer.to_qtensor() is emb.weight
    assert is_lowered(model)
    unlower_model(model)
    assert isinstance(model[0], nn.Embedding) and model[0].weight is emb.weight and model[0].embed_scale == 6.5
    assert not [n for n, _ in model.named_children() if n.startswith("_vq_emb_proxy_")]


def test_indices_above_32767_are_read_as_unsigned():
    emb, table = _vq_embedding(vocab=8, dim=16, nc=50000, seed=4)
    emb.weight.qscheme  # 50000-row codebook: about a third of the indices do not fit a signed int16
    model = nn.Sequential(emb)
    linearize_vq_embeddings(model)
    assert (model[0].all_indices < 0).any()
    ids = torch.arange(8)
    assert torch.equal(model[0](ids), table)


def test_auto_lowering_covers_embeddings_and_unlower_restores_them():
    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.tok, *_ = _q_embedding(padding_idx=0, embed_scale=4.0)
            self.vq_tok, _ = _vq_embedding(dim=64)
            self.norm = LlamaRMSNorm(64)

        def forward(self, ids):
            return self.norm(self.tok(ids) + self.vq_tok(ids))

    m = M()
    q_weight, vq_weight = m.tok.weight, m.vq_tok.weight
    AutoKernelLowering().apply(m)
    assert isinstance(m.tok, NPEmbedding) and isinstance(m.vq_tok, NPVQEmbedding)
    assert isinstance(m.norm, LlamaRMSNorm)  # norms are fused only on a GPU
    ids = torch.tensor([[0, 5, 29]])
    y = m(ids)
    unlower_model(m)
    assert isinstance(m.tok, nn.Embedding) and m.tok.padding_idx == 0 and m.tok.embed_scale == 4.0
    assert torch.equal(m.tok.weight.u8_blob, q_weight.u8_blob) and m.vq_tok.weight is vq_weight
    AutoKernelLowering().apply(m)
    assert torch.equal(m(ids), y)


def test_checkpoint_round_trip_with_quantized_embeddings(tmp_path):
    from neuropress_amd.t2n.model_io import load_quantized_model, save_quantized_model

    class M(nn.Module):
        def __init__(self, quantized):
            super().__init__()
            if quantized:
                self.tok, *_ = _q_embedding(asym=True)
                self.vq_tok, _ = _vq_embedding(dim=64, perm=True)
            else:
                self.tok, self.vq_tok = ScaledEmbedding(40, 64), ScaledEmbedding(30, 64)

    src = M(True)
    path = tmp_path / "emb.safetensors"
    save_quantized_model(src, path)
    dst = M(False)
    manifest = load_quantized_model(dst, path)
    assert manifest.qtensor_params == {"tok.weight": "QTensorScaleZp", "vq_tok.weight": "QTensorTractVQ"}
    assert isinstance(dst.tok, NPEmbedding) and isinstance(dst.vq_tok, NPVQEmbedding)
    ids = torch.tensor([1, 7, 29])
    AutoKernelLowering().apply(src)
    assert torch.equal(dst.tok(ids), src.tok(ids)) and torch.equal(dst.vq_tok(ids), src.vq_tok(ids))
