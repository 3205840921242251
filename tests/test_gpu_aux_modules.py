"""NPRMSNorm, NPVQEmbedding and NPEmbedding on the GPU: the modules' HIP paths against their
torch-op specifications run on the CPU, and the lowering pass over a small decoder-shaped model."""

import pytest
import torch
import torch.nn as nn

from neuropress_amd import AutoKernelLowering, is_lowered, unlower_model
from neuropress_amd.nn import NPEmbedding, NPRMSNorm, NPVQEmbedding, NPVQLinear
from neuropress_amd.qweights import VQWeight, attach_quantized_weight
from tests.test_host_aux_modules import GemmaRMSNorm, LlamaRMSNorm, _q_embedding, _vq_embedding

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("cls", [LlamaRMSNorm, GemmaRMSNorm])
def test_rms_norms_are_fused_on_the_gpu_with_the_right_convention(gpu, dtype, cls):
    from neuropress_amd.nn import linearize_rms_norms

    torch.manual_seed(5)
    model = nn.Sequential(cls(256), nn.Identity(), cls(256)).to(gpu).to(dtype)
    x = torch.randn(4, 7, 256, device=gpu).to(dtype)
    want = model(x)
    sources = [model[0], model[2]]
    assert linearize_rms_norms(model) == 2
    assert isinstance(model[0], NPRMSNorm) and model[0].weight.dtype == dtype
    got = model(x)
    # two normalisations in a row, each within one rounding of the unfused f32 computation
    assert torch.allclose(got.float(), want.float(), rtol=2 ** -6 if dtype == torch.bfloat16 else 2 ** -9, atol=1e-3)
    if cls is GemmaRMSNorm:
        assert torch.allclose(model[0].weight.float(), 1.0 + sources[0].weight.float(), atol=1e-2)
    unlower_model(model)
    assert model[0] is sources[0] and model[2] is sources[1]


@pytest.mark.parametrize("asym", [False, True])
@pytest.mark.parametrize("out_dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_npembedding_cuda_backend_equals_the_compile_backend(gpu, asym, out_dtype):
    emb, *_ = _q_embedding(vocab=300, dim=256, asym=asym, padding_idx=2, embed_scale=16.0, dtype=out_dtype)
    spec = NPEmbedding.from_embedding(emb, "compile")
    layer = NPEmbedding.from_embedding(emb, "auto").to(gpu)
    assert layer.backend.value == "cuda"
    ids = torch.randint(0, 300, (3, 11), generator=torch.Generator().manual_seed(1))
    ids[0, 0] = 2
    got = layer(ids.to(gpu))
    assert got.dtype == out_dtype and torch.equal(got.cpu(), spec(ids))


@pytest.mark.parametrize("perm,scale", [(False, 1.0), (True, 1.0), (True, 16.0)])
def test_npvqembedding_gpu_equals_the_torch_path(gpu, perm, scale):
    from neuropress_amd.nn import linearize_vq_embeddings

    emb, table = _vq_embedding(vocab=200, dim=256, nc=40000, perm=perm, embed_scale=scale, seed=3)
    model = nn.Sequential(emb, nn.Linear(256, 8).to(torch.bfloat16))
    linearize_vq_embeddings(model)
    ids = torch.randint(0, 200, (2, 9), generator=torch.Generator().manual_seed(2))
    want = model[0](ids)  # torch ops on the CPU
    model.to(gpu)
    got = model[0](ids.to(gpu))
    assert got.dtype == torch.bfloat16 and torch.equal(got.cpu(), want)
    assert torch.equal(model[0].weight[7].cpu(), model[0](torch.tensor([7]).to(gpu))[0].cpu())


def test_lowering_a_decoder_shaped_model(gpu):
    """Embedding -> norm -> VQ linear -> norm -> VQ linear: the lowered model on the GPU against the
    same modules' torch-op paths on the CPU."""

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            g = torch.Generator().manual_seed(8)
            self.tok, _ = _vq_embedding(vocab=120, dim=128, nc=512, embed_scale=11.3137, seed=8)
            self.norm1, self.norm2 = GemmaRMSNorm(128), LlamaRMSNorm(256)
            cb = (torch.randn(512, 8, generator=g) * 0.05).half()
            self.up = attach_quantized_weight(nn.Linear(128, 256, bias=False), VQWeight.from_indices(
                torch.randint(0, 512, (256 * 16,), generator=g), cb, 256, 128))
            self.down = attach_quantized_weight(nn.Linear(256, 128, bias=False), VQWeight.from_indices(
                torch.randint(0, 512, (128 * 32,), generator=g), cb, 128, 256))
            self.register_parameter("anchor", nn.Parameter(torch.zeros(1, dtype=torch.float16)))  # model dtype marker

        def forward(self, ids):
            h = self.norm1(self.tok(ids))
            return self.down(self.norm2(torch.nn.functional.silu(self.up(h))))

    torch.manual_seed(0)
    ref = Block()
    ref.norm1.half(), ref.norm2.half()
    AutoKernelLowering(vq_backend="default").apply(ref)  # CPU: torch-op paths, norms stay unfused
    ids = torch.tensor([[0, 3, 119, 57, 3]])
    want = ref(ids).float()

    torch.manual_seed(0)
    model = Block()
    model.norm1.half(), model.norm2.half()
    model.to(gpu)
    AutoKernelLowering().apply(model)
    model.to(gpu)
    assert isinstance(model.tok, NPVQEmbedding) and isinstance(model.norm1, NPRMSNorm) and isinstance(model.up, NPVQLinear)
    assert is_lowered(model)
    got = model(ids.to(gpu)).float().cpu()
    assert torch.allclose(got, want, rtol=1e-2, atol=1e-2), (got - want).abs().max()
