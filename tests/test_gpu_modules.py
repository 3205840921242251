"""GPU tests of the drop-in modules and of the full benchmark sizes (Llama-3-8B layers).

Module tests: every band of NPVQLinear / NPLinear on the GPU against the
torch-op specification of the same layer on the CPU.  Full-size tests use
size-independent properties: decode equals torch's own gather on the device
(a library routine), codebook-permutation invariance (bit-exact), a zero
codebook yields exactly the bias, M-split invariance, linearity.
"""

import numpy as np
import pytest
import torch
import torch.nn as nn

import neuropress_amd.nn.np_vq_linear as vqmod
from neuropress_amd import AutoKernelLowering
from neuropress_amd.nn import NPLinear, NPVQLinear, VQProxy
from neuropress_amd.qweights import ScalarQWeight, VQWeight, attach_quantized_weight
from tests import cases

pytestmark = pytest.mark.gpu


def _close(y_gpu, y_ref):
    ok, max_abs, excess = cases.within_tol(y_gpu.float().cpu().numpy(), y_ref.double().cpu().numpy())
    assert ok, f"max abs err {max_abs:.3e} = {excess:.2f}x the 1e-2 bound"


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("bits,nc", [(8, 256), (10, 1024), (12, 4096), (16, 65536)])
@pytest.mark.parametrize("vl", [8, 4])
def test_npvqlinear_all_bands_match_default(gpu, act, bits, nc, vl, monkeypatch):
    """Vector length 8 (the benchmark configurations) and 4 (the reference's default)."""
    monkeypatch.setattr(vqmod, "_FUSED_MAX_TOKENS", 16)
    monkeypatch.setattr(vqmod, "_TILE_MAX_TOKENS", 64)
    monkeypatch.setattr(vqmod, "_TILE_MIN_GRID_FRACTION", 0.0)  # small layers: force the tile band
    L = cases.vq_layer(40 + bits, 96, 256, nc, vl=vl, bits=bits, bias=True, std=0.05)
    ref_layer = NPVQLinear(VQProxy(L["cb"]), L["packed"], bits, 96, 256, vl, "default", bias=L["bias"].float())
    proxy = VQProxy(L["cb"]).to(gpu)
    layer = NPVQLinear(proxy, L["packed"], bits, 96, 256, vl, "cuda_wmma", bias=L["bias"].float()).to(gpu)
    assert layer._mfma_layer()
    for shape in [(1, 256), (2, 8, 256), (40, 256), (3, 50, 256)]:  # fused, fused(16), tile, dense
        x = torch.randn(*shape, generator=cases.gen(1)).to(act)
        y = layer(x.to(gpu))
        assert y.shape == (*shape[:-1], 96) and y.dtype == act
        # specification: gather + F.linear in f32 with the weight rounded to the activation dtype
        w = L["cb"][L["idx"]].reshape(96, 256).to(act).float()
        _close(y, torch.nn.functional.linear(x.float(), w, L["bias"].float()))
        if act == torch.float32:
            assert torch.allclose(y.cpu(), ref_layer(x), atol=1e-4)


def test_lowering_auto_runs_hip_backends_on_gpu(gpu):
    class M(nn.Module):
        def __init__(self):
            super().__init__()
            L = cases.vq_layer(5, 64, 128, 4096, bias=False)
            self.fc = attach_quantized_weight(nn.Linear(128, 64, bias=True),
                                              VQWeight.from_indices(L["idx"], L["cb"], 64, 128))
            Q = cases.q4_layer(6, 64, 128)
            self.q = attach_quantized_weight(nn.Linear(128, 64, bias=False),
                                             ScalarQWeight.from_codes(Q["codes"], Q["scale"], 4, 32))

        def forward(self, x):
            return self.fc(x) + self.q(x)

    torch.manual_seed(0)
    m = M()
    x = torch.randn(5, 128).half()
    AutoKernelLowering(vq_backend="default", linear_backend="compile").apply(m)
    ref = m(x.float())
    from neuropress_amd import unlower_model

    unlower_model(m)
    m = m.to(gpu)
    AutoKernelLowering().apply(m)
    m = m.to(gpu)
    assert m.fc.backend.value == "cuda_wmma" and m.q.backend.value == "cuda"
    _close(m(x.to(gpu)), ref)
    _close(m(torch.cat([x] * 8).to(gpu))[:5], ref)  # 40 tokens: past the fused band


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
def test_nplinear_bands(gpu, act, monkeypatch):
    import neuropress_amd.nn.np_linear as qmod

    monkeypatch.setattr(qmod, "_Q_TILE_MAX_TOKENS", 64)
    monkeypatch.setattr(qmod, "_Q_TILE_MIN_GRID_FRACTION", 0.0)  # small layer: force the fused GEMM band
    Q = cases.q4_layer(8, 80, 256, bias=True)
    layer = NPLinear(Q["blob"], Q["scale"], 80, 256, 32, 4, "sym", "cuda", bias=Q["bias"].float()).to(gpu)
    w = ((Q["codes"].float() - 8).reshape(80, 8, 32) * Q["scale"].float().reshape(80, 8, 1)).reshape(80, 256)
    for m in (1, 16, 40, 100):
        x = torch.randn(m, 256, generator=cases.gen(m)).to(act)
        _close(layer(x.to(gpu)), torch.nn.functional.linear(x.float(), w.to(act).float(), Q["bias"].float()))


def test_residual_module_bands(gpu, monkeypatch):
    monkeypatch.setattr(vqmod, "_TILE_MAX_TOKENS", 64)
    monkeypatch.setattr(vqmod, "_TILE_MIN_GRID_FRACTION", 0.0)  # small layers: force the tile band
    L = cases.rvq_layer(12, 48, 256, nc_main=65536, nc_res=256)
    mk = lambda backend: NPVQLinear(VQProxy(L["cbm"]), L["pm"], L["bm"], 48, 256, 8, backend,
                                    residual_proxy=VQProxy(L["cbr"]), packed_residual=L["pr"],
                                    residual_bits=L["br"], row_scale=L["scale"], row_bias=L["wbias"])
    ref_layer = mk("default")
    layer = mk("cuda_wmma").to(gpu)
    layer.proxy.to(gpu), layer.residual_proxy.to(gpu)
    w = ref_layer._dense_weight_torch(torch.float16).float()
    for m in (1, 30, 100):
        x = torch.randn(m, 256, generator=cases.gen(m)).half()
        _close(layer(x.to(gpu)), x.float() @ w.T)


def test_long_k_layers_of_one_row_tile_keep_the_gemv_to_32_tokens(gpu, monkeypatch):
    """tokens x K above 2^18 normally ends the GEMV band at 16 tokens; a layer of one row tile per
    workgroup whose lookups go to memory runs the GEMV that stages its activations and keeps it
    to 32 tokens (65536-row codebook, int4), one with a 4096-row table (looked up in LDS) does
    not.  Outputs against the dense product of the decoded weight."""
    import neuropress_amd.nn.np_linear as qmod
    from neuropress_amd import kernels

    calls = []
    for name in ("vq_linear", "vq_gemm_tile", "q_linear", "q_gemm_tile"):
        real = getattr(kernels, name)
        monkeypatch.setattr(kernels, name, lambda *a, _real=real, _name=name, **kw: (calls.append(_name), _real(*a, **kw))[1])
    monkeypatch.setattr(vqmod, "_TILE_MIN_GRID_FRACTION", 0.0)
    monkeypatch.setattr(qmod, "_Q_TILE_MIN_GRID_FRACTION", 0.0)
    n, k, m = 48, 16384, 24
    x = torch.randn(m, k, generator=cases.gen(3)).half()
    for nc, expect in ((65536, "vq_linear"), (4096, "vq_gemm_tile")):
        L = cases.vq_layer(70 + nc, n, k, nc, bias=False, std=0.05)
        layer = NPVQLinear(VQProxy(L["cb"]).to(gpu), L["packed"], L["bits"], n, k, 8, "cuda_wmma").to(gpu)
        assert kernels.gemv_stages_activations(m, n, k, nc) == (nc == 65536)
        calls.clear()
        y = layer(x.to(gpu))
        assert calls == [expect], calls
        _close(y, x.float() @ L["cb"][L["idx"]].reshape(n, k).float().T)
    Q = cases.q4_layer(71, n, k)
    qlayer = NPLinear(Q["blob"], Q["scale"], n, k, 32, 4, "sym", "cuda").to(gpu)
    calls.clear()
    y = qlayer(x.to(gpu))
    assert calls == ["q_linear"], calls
    w = ((Q["codes"].float() - 8).reshape(n, k // 32, 32) * Q["scale"].float().reshape(n, k // 32, 1)).reshape(n, k)
    _close(y, x.float() @ w.half().float().T)


def test_residual_layers_take_the_gemv_to_32_tokens_and_then_the_tile_band(gpu, monkeypatch):
    """A residual layer keeps the fused GEMV up to 32 tokens at any reduction length and takes the
    tile GEMM above, like a plain layer."""
    from neuropress_amd import kernels

    calls = []
    real = kernels.rvq_linear
    monkeypatch.setattr(kernels, "rvq_linear",
                        lambda *a, _real=real, **kw: (calls.append((a[0].shape[0], kw.get("tile"))), _real(*a, **kw))[1])
    monkeypatch.setattr(vqmod, "_TILE_MIN_GRID_FRACTION", 0.0)
    for k, expect in ((256, [(4, False), (32, False), (40, True)]), (16384, [(4, False), (32, False), (40, True)])):
        L = cases.rvq_layer(21, 32, k, nc_main=4096, nc_res=16)
        layer = NPVQLinear(VQProxy(L["cbm"]), L["pm"], L["bm"], 32, k, 8, "cuda_wmma",
                           residual_proxy=VQProxy(L["cbr"]), packed_residual=L["pr"], residual_bits=L["br"],
                           row_scale=L["scale"], row_bias=L["wbias"]).to(gpu)
        layer.proxy.to(gpu), layer.residual_proxy.to(gpu)
        w = layer._dense_weight_torch(torch.float16).float().cpu()
        calls.clear()
        for m in (4, 32, 40):
            x = (torch.randn(m, k, generator=cases.gen(m)) * 0.3).half()
            _close(layer(x.to(gpu)), x.float() @ w.T)
        assert calls == expect


def test_skewed_layers_time_the_sliced_gemv_against_the_fused_one(gpu):
    """Full-size layers are timed when their slice lists are built and take the slice-list GEMV only
    for the token counts where it won.  Evenly spread indices: it wins at least at one token.
    Zipf(1.1) indices put nine tenths of them in one codebook slice, where the fused GEMV's lookups
    hit in L1: the limit can only be lower.  Results are right on either path."""
    n, k, nc = 4096, 4096, 65536
    g = cases.gen(91)
    cb = (torch.randn(nc, 8, generator=g) * 0.02).half()
    x = (torch.randn(4, k, generator=g) * 0.5).half()
    limits = {}
    for name, idx in (("uniform", torch.randint(0, nc, (n * k // 8,), generator=g)),
                      ("zipf", cases.zipf_indices(g, nc, n * k // 8))):
        packed = idx.to(torch.int32).to(torch.int16).view(torch.uint8)
        layer = NPVQLinear(VQProxy(cb).to(gpu), packed, 16, n, k, 8, "cuda_wmma").to(gpu)
        assert layer.prepare_sliced()
        limits[name] = layer._derived_hit("sliced", layer.packed_indices)[1]
        w = cb[idx].reshape(n, k).float()
        for m in (1, 4):
            _close(layer(x[:m].to(gpu)), x[:m].float() @ w.T)
    cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    assert 1 <= limits["uniform"] <= vqmod._SLICED_MAX_TOKENS  # one token: 8 us against 12 or more
    assert 0 <= limits["zipf"] <= limits["uniform"]
    print("slice-list token limits:", limits, "on", cus, "compute units")


def test_layers_outside_the_mfma_kernels_go_to_decode_and_gemm(gpu, monkeypatch):
    """2-bit group quantization and vector length 2 have no MFMA kernel: the modules decode once and
    call the dense GEMM at every token count instead of the fused entry points (whose element-wise
    kernels decode the weight once per 16 tokens)."""
    import neuropress_amd.nn.np_linear as qmod
    from neuropress_amd import kernels

    calls = []
    for name in ("vq_gemm_tile", "q_gemm_tile", "vq_linear", "q_linear", "vq_dequant", "q_dequant"):
        real = getattr(kernels, name)
        monkeypatch.setattr(kernels, name, lambda *a, _real=real, _name=name, **kw: (calls.append(_name), _real(*a, **kw))[1])
    monkeypatch.setattr(vqmod, "_TILE_MIN_GRID_FRACTION", 0.0)
    monkeypatch.setattr(qmod, "_Q_TILE_MIN_GRID_FRACTION", 0.0)
    Q = cases.q4_layer(81, 96, 256, nbits=2, bias=True)
    qlayer = NPLinear(Q["blob"], Q["scale"], 96, 256, 32, 2, "sym", "cuda", bias=Q["bias"].float()).to(gpu)
    wq = ((Q["codes"].float() - 2).reshape(96, 8, 32) * Q["scale"].float().reshape(96, 8, 1)).reshape(96, 256)
    L = cases.vq_layer(82, 96, 256, 1024, vl=2, bits=10, bias=True, std=0.05)
    layer = NPVQLinear(VQProxy(L["cb"]).to(gpu), L["packed"], 10, 96, 256, 2, "cuda_wmma", bias=L["bias"].float()).to(gpu)
    w = L["cb"][L["idx"]].reshape(96, 256).half().float()
    for m in (3, 40):
        x = (torch.randn(m, 256, generator=cases.gen(m)) * 0.5).half()
        _close(qlayer(x.to(gpu)), torch.nn.functional.linear(x.float(), wq.half().float(), Q["bias"].float()))
        _close(layer(x.to(gpu)), torch.nn.functional.linear(x.float(), w, L["bias"].float()))
    assert calls == ["q_dequant", "vq_dequant"] * 2  # nothing went to a fused entry point


def test_narrow_layers_take_the_split_tile_band(gpu, monkeypatch):
    """A 2048 x 4096 layer has 32 column tiles: up to 32 tokens run the GEMV, and the module still
    routes 33..128 tokens (int4: 33..256) to the tile GEMM (which splits the reduction), and more
    tokens to decode + GEMM."""
    import neuropress_amd.nn.np_linear as qmod

    L = cases.vq_layer(77, 2048, 4096, 4096, bits=12, bias=True, std=0.02)
    layer = NPVQLinear(VQProxy(L["cb"]).to(gpu), L["packed"], 12, 2048, 4096, 8, "cuda_wmma",
                       bias=L["bias"].float()).to(gpu)
    Q = cases.q4_layer(78, 2048, 4096, bias=True)
    qlayer = NPLinear(Q["blob"], Q["scale"], 2048, 4096, 32, 4, "sym", "cuda", bias=Q["bias"].float()).to(gpu)
    calls = []
    from neuropress_amd import kernels

    for name in ("vq_gemm_tile", "q_gemm_tile"):
        real = getattr(kernels, name)
        monkeypatch.setattr(kernels, name,
                            lambda *a, _real=real, _name=name, **kw: (calls.append((_name, a[0].shape[0])), _real(*a, **kw))[1])
    w = L["cb"][L["idx"]].reshape(2048, 4096).half().float()
    wq = ((Q["codes"].float() - 8).reshape(2048, 128, 32) * Q["scale"].float().reshape(2048, 128, 1)).reshape(2048, 4096)
    for m in (17, 32, 33, 128, 129, 257):
        x = (torch.randn(m, 4096, generator=cases.gen(m)) * 0.5).half()
        _close(layer(x.to(gpu)), torch.nn.functional.linear(x.float(), w, L["bias"].float()))
        _close(qlayer(x.to(gpu)), torch.nn.functional.linear(x.float(), wq.half().float(), Q["bias"].float()))
    assert calls == [("vq_gemm_tile", 33), ("q_gemm_tile", 33), ("vq_gemm_tile", 128), ("q_gemm_tile", 128),
                     ("q_gemm_tile", 129)]
    from neuropress_amd import _lib

    assert _lib.load().npamd_gemm_tile_workspace_bytes(17, 2048, 4096) > 0  # the split is in use


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
def test_column_perm_is_folded_into_the_fused_gemv(gpu, act, monkeypatch):
    """A layer with column_perm and a small codebook: up to 16 tokens (while M * K fits the kernel's
    LDS copy of x) the fused GEMV gathers the columns itself; more tokens gather with torch first."""
    from neuropress_amd import kernels

    n, k, nc = 96, 1024, 4096
    L = cases.vq_layer(81, n, k, nc, bits=12, bias=True, std=0.05)
    perm = torch.randperm(k, generator=cases.gen(82))
    layer = NPVQLinear(VQProxy(L["cb"]).to(gpu), L["packed"], 12, n, k, 8, "cuda_wmma", bias=L["bias"].float(),
                       column_perm=perm).to(gpu)
    seen = []
    real = kernels.vq_linear
    monkeypatch.setattr(kernels, "vq_linear",
                        lambda *a, **kw: (seen.append(kw.get("column_perm") is not None), real(*a, **kw))[1])
    w = L["cb"][L["idx"]].reshape(n, k).to(act).float()
    for m in (1, 4, 16):
        x = torch.randn(m, k, generator=cases.gen(m)).to(act)
        _close(layer(x.to(gpu)), torch.nn.functional.linear(x[:, perm].float(), w, L["bias"].float()))
    assert seen == [True, True, True]
    assert layer._perm_i32(gpu).dtype == torch.int32


@pytest.mark.parametrize("kind", ["tiered", "ntier", "zero_escape"])
def test_prefix_coded_layers_run_the_hip_bands(gpu, kind, monkeypatch):
    """A weight stored in a two-tier / n-tier / zero-escape buffer (Zipf-distributed indices, as the
    formats assume): "auto" lowering names the reference's per-format backend and the layer runs the
    slice-list GEMV, the fused GEMV, the tile GEMM and decode + GEMM on its expanded stream."""
    from neuropress_amd import kernels

    monkeypatch.setattr(vqmod, "_SLICED_MIN_INDICES", 1)
    monkeypatch.setattr(vqmod, "_TILE_MAX_TOKENS", 64)
    monkeypatch.setattr(vqmod, "_TILE_WIDE_SMALL_MAX_TOKENS", 64)  # the band of a small layer with a codebook in memory
    monkeypatch.setattr(vqmod, "_TILE_MIN_GRID_FRACTION", 0.0)
    n, k, nc = 128, 512, 20000
    g = cases.gen(91)
    cb = (torch.randn(nc, 8, generator=g) * 0.05).half()
    p = 1.0 / torch.arange(1, nc + 1, dtype=torch.float64) ** 1.1
    idx = torch.multinomial(p / p.sum(), n * k // 8, replacement=True, generator=g)
    kw = {"tiered": dict(use_tiered=True, hot_bits=8), "ntier": dict(tier_bits=[4, 8, 12, 15]),
          "zero_escape": dict(zero_escape=True)}[kind]
    model = nn.Sequential(attach_quantized_weight(nn.Linear(k, n, bias=True),
                                                  VQWeight.from_indices(idx, cb, n, k, bits=15, **kw)))
    bias = model[0].bias.detach().clone()
    model.to(gpu)
    AutoKernelLowering().apply(model)
    model.to(gpu)  # the weight container is not a parameter: the lowered module's buffers move here
    import neuropress_amd

    neuropress_amd.prepare_decode(model)  # slice lists for the buffers where they are now
    layer = model[0]
    assert layer.backend.value == {"tiered": "cuda_tiered", "ntier": "cuda_ntier", "zero_escape": "cuda_zero_escape"}[kind]
    assert layer.bits == 15 and layer.packed_indices.is_cuda
    calls = []
    for name in ("vq_linear_sliced_checked", "vq_linear", "vq_gemm_tile", "vq_dequant"):
        real = getattr(kernels, name)
        monkeypatch.setattr(kernels, name, lambda *a, _r=real, _n=name, **kw_: (calls.append(_n), _r(*a, **kw_))[1])
    w = cb[idx].reshape(n, k).float()
    for m in (1, 12, 40, 100):
        x = torch.randn(m, k, generator=cases.gen(m)).half()
        _close(layer(x.to(gpu)), torch.nn.functional.linear(x.float(), w, bias.float()))
    assert calls == ["vq_linear_sliced_checked", "vq_linear", "vq_gemm_tile", "vq_dequant"]


# ------------------------------------------------------ benchmark full sizes ---


@pytest.fixture(scope="module")
def cfg3(gpu):
    """Config 3, up/gate shape: 14336 x 4096, 65536 x 8 codebook, 16-bit indices, seed 1003."""
    g = cases.gen(1003)
    cb = (torch.randn(65536, 8, generator=g) * 0.02).half()
    idx16 = torch.randint(0, 65536, (14336 * 512,), generator=g, dtype=torch.int32).to(torch.int16)
    return dict(cb=cb.to(gpu), idx16=idx16.to(gpu), packed=idx16.view(torch.uint8).to(gpu), n=14336, k=4096)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_cfg3_decode_equals_device_gather(gpu, cfg3, dtype):
    from neuropress_amd import kernels

    w = kernels.vq_dequant(cfg3["packed"], cfg3["cb"], 16, cfg3["n"], cfg3["k"], dtype)
    idx = cfg3["idx16"].to(torch.int64) & 0xFFFF
    assert torch.equal(w, cfg3["cb"][idx].reshape(cfg3["n"], cfg3["k"]).to(dtype))


@pytest.mark.parametrize("m", [1, 2, 16])
def test_cfg3_gemv_properties(gpu, cfg3, m):
    from neuropress_amd import kernels

    n, k = cfg3["n"], cfg3["k"]
    x = torch.randn(m, k, generator=cases.gen(m)).bfloat16().to(gpu)
    bias = torch.randn(n, generator=cases.gen(9)).to(gpu)
    y = kernels.vq_linear(x, cfg3["packed"], cfg3["cb"], 16, 8, bias, n)
    # against the dense product of the decoded weight (torch matmul = library routine)
    w = kernels.vq_dequant(cfg3["packed"], cfg3["cb"], 16, n, k, torch.bfloat16)
    ref = x.float() @ w.float().T + bias
    _close(y, ref)
    # codebook row permutation + index remap leaves the result bit-identical
    perm = torch.randperm(65536, generator=cases.gen(2)).to(gpu)
    inv = torch.argsort(perm)
    idx = cfg3["idx16"].to(torch.int64) & 0xFFFF
    remapped = inv[idx].to(torch.int16).view(torch.uint8)
    y2 = kernels.vq_linear(x, remapped, cfg3["cb"][perm].contiguous(), 16, 8, bias, n)
    assert torch.equal(y, y2)
    # all-zero codebook -> exactly the bias (rounded once)
    y0 = kernels.vq_linear(x, cfg3["packed"], torch.zeros_like(cfg3["cb"]), 16, 8, bias, n)
    assert torch.equal(y0, bias.bfloat16().expand(m, n))
    # rows of the batch are independent: each row alone gives the same bits
    y_row = kernels.vq_linear(x[:1].contiguous(), cfg3["packed"], cfg3["cb"], 16, 8, bias, n)
    assert torch.equal(y_row, y[:1])


@pytest.mark.parametrize("m", [64, 384])
def test_cfg3_tile_gemm_properties(gpu, cfg3, m):
    from neuropress_amd import kernels

    n, k = cfg3["n"], cfg3["k"]
    x = torch.randn(m, k, generator=cases.gen(m)).bfloat16().to(gpu)
    y = kernels.vq_gemm_tile(x, cfg3["packed"], cfg3["cb"], 16, n)
    w = kernels.vq_dequant(cfg3["packed"], cfg3["cb"], 16, n, k, torch.bfloat16)
    _close(y, x.float() @ w.float().T)
    # splitting M across calls changes nothing (each output row depends on its own x row only)
    y_a = kernels.vq_gemm_tile(x[: m // 2].contiguous(), cfg3["packed"], cfg3["cb"], 16, n)
    assert torch.equal(y_a, y[: m // 2])
    y0 = kernels.vq_gemm_tile(x, cfg3["packed"], torch.zeros_like(cfg3["cb"]), 16, n)
    assert not y0.any()


def test_cfg3_down_proj_shape(gpu):
    """4096 x 14336: K = 224 chunks = 56 steps, exercises the many-waves-per-row split."""
    from neuropress_amd import kernels

    g = cases.gen(1003)
    cb = (torch.randn(65536, 8, generator=g) * 0.02).half().to(gpu)
    packed = torch.randint(0, 65536, (4096 * 1792,), generator=g, dtype=torch.int32).to(torch.int16).view(torch.uint8).to(gpu)
    x = torch.randn(2, 14336, generator=g).bfloat16().to(gpu)
    w = kernels.vq_dequant(packed, cb, 16, 4096, 14336, torch.bfloat16)
    ref = x.float() @ w.float().T
    _close(kernels.vq_linear(x, packed, cb, 16, 8, None, 4096), ref)
    _close(kernels.vq_gemm_tile(x, packed, cb, 16, 4096), ref)
    # mid token counts: 64 column blocks do not fill the GPU, so the reduction is split (workspace in
    # use); the split changes the summation order only, and rows stay independent of each other
    from neuropress_amd import _lib

    for m in (64, 384):
        assert _lib.load().npamd_gemm_tile_workspace_bytes(m, 4096, 14336) > 0
        xm = torch.randn(m, 14336, generator=cases.gen(m)).bfloat16().to(gpu)
        ym = kernels.vq_gemm_tile(xm, packed, cb, 16, 4096)
        _close(ym, xm.float() @ w.float().T)
        assert torch.equal(kernels.vq_gemm_tile(xm[: m // 2].contiguous(), packed, cb, 16, 4096), ym[: m // 2])


def test_cfg5_q4_full_size(gpu):
    from neuropress_amd import kernels

    Q = cases.q4_layer(1005, 14336, 4096)
    blob, sc = Q["blob"].to(gpu), Q["scale"].to(gpu)
    w = kernels.q_dequant(blob, sc, 4, 32, None, torch.float16)
    w_ref = ((Q["codes"].to(gpu).float() - 8).reshape(14336, 128, 32) * sc.float().reshape(14336, 128, 1))
    assert torch.equal(w, w_ref.reshape(14336, 4096).half())
    for m in (1, 16, 256):
        x = torch.randn(m, 4096, generator=cases.gen(m)).half().to(gpu)
        _close(kernels.q_linear(x, blob, sc, 4, 32), x.float() @ w.float().T)


def test_cfg4_residual_full_size(gpu):
    from neuropress_amd import kernels

    L = cases.rvq_layer(1004, 1024, 4096)  # the k/v shape of config 4, Zipf(1.1) indices
    dev = {k: (v.to(gpu) if isinstance(v, torch.Tensor) else v) for k, v in L.items()}
    w = kernels.rvq_dequant(dev["pm"], L["bm"], dev["pr"], L["br"], dev["cbm"], dev["cbr"], dev["scale"],
                            dev["wbias"], 1024, 4096, torch.float16)
    w_ref = (dev["cbm"][dev["im"]] + dev["cbr"][dev["ir"]]).reshape(1024, 4096)
    w_ref = (w_ref * dev["scale"][:, None]) + dev["wbias"][:, None]  # torch fp16 ops round one at a time
    assert torch.equal(w, w_ref)
    for m, tile in ((1, False), (384, True)):
        x = torch.randn(m, 4096, generator=cases.gen(m)).half().to(gpu)
        y = kernels.rvq_linear(x, dev["pm"], L["bm"], dev["pr"], L["br"], dev["cbm"], dev["cbr"], dev["scale"],
                               dev["wbias"], 1024, None, tile=tile)
        _close(y, x.float() @ w.float().T)


# Full sizes anchored in the oracle itself (the C restatement decodes a few million vectors and
# contracts one or two tokens in well under a second), not in the HIP decode.


@pytest.mark.parametrize("name,n,k", [("q/o", 2048, 2048), ("k/v", 512, 2048), ("gate/up", 8192, 2048), ("down", 2048, 8192)])
@pytest.mark.parametrize("bits", [12, 16])
def test_cfg2_layers_full_size_against_the_oracle(gpu, oracle_lib, name, n, k, bits):
    """Config 2's own four layers (4096 x 8 fp16 codebook, fp16, one and two tokens), with the
    index stream as the 12-bit bit stream and as int16: decode bit-exact against the oracle's
    decode, the LDS-codebook GEMV within the bound of the oracle's double-accumulated product."""
    from neuropress_amd import kernels

    from oracle import oracle as orc

    lib = oracle_lib
    L = cases.vq_layer(1002, n, k, 4096, bits=bits, act=torch.float16, m=2, bias=True)
    code = orc.torch_dtype_code(torch.float16)
    w_ref = lib.vq_decode(L["packed"].numpy(), bits, orc.to_bits(L["cb"]), n, k, code)
    dev = {key: L[key].to(gpu) for key in ("x", "packed", "cb", "bias")}
    w = kernels.vq_dequant(dev["packed"], dev["cb"], bits, n, k, torch.float16)
    assert np.array_equal(orc.to_bits(w.cpu()), w_ref)
    for m in (1, 2):
        x = L["x"][:m].contiguous()
        ref = lib.linear_f64(orc.to_bits(x), code, w_ref, code, orc.to_bits(L["bias"]), code)
        y = kernels.vq_linear(x.to(gpu), dev["packed"], dev["cb"], bits, 8, dev["bias"], n)
        ok, max_abs, excess = cases.within_tol(y.float().cpu().numpy(), ref)
        assert ok, f"{name} M={m}: max abs err {max_abs:.3e} = {excess:.2f}x the 1e-2 bound"


def test_cfg4_q_proj_full_size_against_the_oracle(gpu, oracle_lib):
    """Config 4's q/o projection (4096 x 4096, residual VQ, Zipf(1.1) indices): decode bit-exact
    against the oracle, one token through the fused GEMV against the oracle's product, 384 tokens
    through the tile GEMM against the dense product of the (now anchored) decoded weight."""
    from neuropress_amd import kernels

    from oracle import oracle as orc

    lib = oracle_lib
    L = cases.rvq_layer(1004, 4096, 4096)
    code = orc.torch_dtype_code(torch.float16)
    w_ref = lib.rvq_decode(L["pm"].numpy(), L["bm"], L["pr"].numpy(), L["br"], orc.to_bits(L["cbm"]),
                           orc.to_bits(L["cbr"]), orc.to_bits(L["scale"]), orc.to_bits(L["wbias"]), 4096, 4096, code)
    dev = {k: (v.to(gpu) if isinstance(v, torch.Tensor) else v) for k, v in L.items()}
    w = kernels.rvq_dequant(dev["pm"], L["bm"], dev["pr"], L["br"], dev["cbm"], dev["cbr"], dev["scale"],
                            dev["wbias"], 4096, 4096, torch.float16)
    assert np.array_equal(orc.to_bits(w.cpu()), w_ref)
    ref = lib.linear_f64(orc.to_bits(L["x"]), code, w_ref, code)
    y = kernels.rvq_linear(dev["x"], dev["pm"], L["bm"], dev["pr"], L["br"], dev["cbm"], dev["cbr"], dev["scale"],
                           dev["wbias"], 4096, None, tile=False)
    ok, max_abs, excess = cases.within_tol(y.float().cpu().numpy(), ref)
    assert ok, f"max abs err {max_abs:.3e} = {excess:.2f}x the 1e-2 bound"
    x = torch.randn(384, 4096, generator=cases.gen(384)).half().to(gpu)
    y = kernels.rvq_linear(x, dev["pm"], L["bm"], dev["pr"], L["br"], dev["cbm"], dev["cbr"], dev["scale"],
                           dev["wbias"], 4096, None, tile=True)
    _close(y, x.float() @ w.float().T)


def test_cfg5_square_layer_full_size_against_the_oracle(gpu, oracle_lib):
    """Config 5's 4096 x 4096 layer: int4 decode bit-exact against the oracle, one token (the
    row-wise kernel) against the oracle's product, 16 and 256 tokens against the dense product."""
    from neuropress_amd import kernels

    from oracle import oracle as orc

    lib = oracle_lib
    Q = cases.q4_layer(1005, 4096, 4096, bias=True)
    code = orc.torch_dtype_code(torch.float16)
    w_ref = lib.q_decode(Q["blob"].numpy(), orc.to_bits(Q["scale"]), None, 4, 32, code)
    blob, sc, bias = Q["blob"].to(gpu), Q["scale"].to(gpu), Q["bias"].to(gpu)
    w = kernels.q_dequant(blob, sc, 4, 32, None, torch.float16)
    assert np.array_equal(orc.to_bits(w.cpu()), w_ref)
    ref = lib.linear_f64(orc.to_bits(Q["x"]), code, w_ref, code, orc.to_bits(Q["bias"]), code)
    y = kernels.q_linear(Q["x"].to(gpu), blob, sc, 4, 32, None, bias)
    ok, max_abs, excess = cases.within_tol(y.float().cpu().numpy(), ref)
    assert ok, f"max abs err {max_abs:.3e} = {excess:.2f}x the 1e-2 bound"
    for m in (16, 256):
        x = torch.randn(m, 4096, generator=cases.gen(m)).half().to(gpu)
        _close(kernels.q_linear(x, blob, sc, 4, 32, None, bias), x.float() @ w.float().T + bias.float())
