"""Host logic of the drop-in modules on CPU: construction, torch-op forward,
band dispatch (with spies, as the reference tests it), backend resolution,
lowering / unlowering, fallback warning, and the C ABI's exported symbols."""

import ctypes
import logging
import re
from pathlib import Path

import pytest
import torch
import torch.nn as nn

import neuropress_amd.nn.np_vq_linear as vqmod
from neuropress_amd import AutoKernelLowering, LoweringConfig, is_lowered, unlower_model
from neuropress_amd.nn import LinearBackend, NPLinear, NPVQLinear, VQBackend, VQProxy, linearize_vq_weights
from neuropress_amd.nn.backends import Backend
from neuropress_amd.nn.np_linear import _q_dequant_linear, _resolve_backend
from neuropress_amd.nn.np_vq_linear import _resolve_vq_backend
from neuropress_amd.qweights import ScalarQWeight, VQWeight, attach_quantized_weight

ROOT = Path(__file__).resolve().parent.parent


def _make_linear_with_vq(out_features, in_features, num_centroids=8, vector_len=4, bias=False, centroids=None):
    if centroids is None:
        centroids = torch.randn(num_centroids, vector_len, dtype=torch.float16)
    idx = torch.randint(0, centroids.shape[0], (out_features * in_features // centroids.shape[1],))
    lin = nn.Linear(in_features, out_features, bias=bias)
    return attach_quantized_weight(lin, VQWeight.from_indices(idx, centroids, out_features, in_features))


# ---------------------------------------------------------------- proxy / ctor ---


def test_vq_proxy_stores_fp16_centroids_and_refuses_forward():
    proxy = VQProxy(torch.randn(16, 8))
    assert proxy.centroids.dtype == torch.float16 and proxy.centroids.shape == (16, 8)
    assert proxy.num_centroids == 16 and proxy.vector_len == 8
    with pytest.raises(RuntimeError, match="should not be called"):
        proxy(torch.zeros(1))
    assert proxy.centroids_as(torch.bfloat16).dtype == torch.bfloat16
    assert proxy.centroids_as(torch.bfloat16) is proxy.centroids_as(torch.bfloat16)  # cached


def test_from_qtensor_linear():
    lin = _make_linear_with_vq(16, 32, bias=True)
    proxy = VQProxy(lin.weight.qscheme.centroids)
    layer = NPVQLinear.from_qtensor_linear(lin, proxy, backend=Backend.DEFAULT)
    assert (layer.out_features, layer.in_features, layer.bits, layer.n_vectors) == (16, 32, 4, 16 * 8)
    assert layer.bias.shape == (16,)
    assert set(layer.state_dict()) == {"packed_indices", "bias"}  # the proxy is not a sub-module
    with pytest.raises(TypeError, match="QTensorTractVQ"):
        NPVQLinear.from_qtensor_linear(nn.Linear(32, 16), proxy)


def test_constructor_rejects_bad_input():
    proxy = VQProxy(torch.randn(16, 8))
    packed = torch.zeros(64, dtype=torch.uint8)
    with pytest.raises(ValueError, match="prefix-coded buffer holds 0 indices"):
        NPVQLinear(proxy, packed, 4, 16, 64, 8, "default", use_tiered=True)  # an all-zero tiered header
    with pytest.raises(ValueError, match="divisible"):
        NPVQLinear(proxy, packed, 4, 16, 60, 8, "default")
    with pytest.raises(ValueError, match="bytes"):
        NPVQLinear(proxy, packed[:10], 4, 16, 64, 8, "default")
    with pytest.raises(ValueError):
        NPVQLinear(proxy, packed, 4, 16, 64, 8, "gemlite")


@pytest.mark.parametrize("shape", [(4, 32), (2, 5, 32)])
def test_forward_default_matches_dequant(shape):
    lin = _make_linear_with_vq(16, 32, num_centroids=8, vector_len=4, bias=True)
    qs = lin.weight.qscheme
    layer = NPVQLinear.from_qtensor_linear(lin, VQProxy(qs.centroids), backend=Backend.DEFAULT)
    x = torch.randn(*shape)
    y = layer(x)
    ref = torch.nn.functional.linear(x, qs.dequantize(lin.weight.u8_blob, torch.float32), lin.bias)
    assert y.shape == (*shape[:-1], 16) and y.dtype == torch.float32
    assert torch.allclose(y, ref, atol=1e-5)


def test_column_perm_is_applied_to_activations():
    cb = torch.randn(16, 4, dtype=torch.float16)
    idx = torch.randint(0, 16, (8 * 8,))
    perm = torch.randperm(32)
    lin = attach_quantized_weight(nn.Linear(32, 8, bias=False), VQWeight.from_indices(idx, cb, 8, 32, perm))
    layer = NPVQLinear.from_qtensor_linear(lin, VQProxy(cb), "default")
    x = torch.randn(3, 32)
    w_perm = cb[idx].reshape(8, 32).float()
    assert torch.allclose(layer(x), x[:, perm] @ w_perm.T, atol=1e-5)
    # dequantize() undoes the permutation, so F.linear with it equals the layer
    assert torch.allclose(layer(x), x @ lin.weight.qscheme.dequantize(lin.weight.u8_blob, torch.float32).T, atol=1e-5)


def test_residual_layer_torch_path_matches_definition():
    from tests import cases

    L = cases.rvq_layer(3, 12, 64, nc_main=512, nc_res=64, zipf=False)
    layer = NPVQLinear(VQProxy(L["cbm"]), L["pm"], L["bm"], 12, 64, 8, "default",
                       residual_proxy=VQProxy(L["cbr"]), packed_residual=L["pr"], residual_bits=L["br"],
                       row_scale=L["scale"], row_bias=L["wbias"])
    w = (L["cbm"][L["im"]] + L["cbr"][L["ir"]]).reshape(12, 64)
    w = (w * L["scale"][:, None]) + L["wbias"][:, None]
    x = L["x"]
    assert torch.equal(layer(x), torch.nn.functional.linear(x, w))
    assert "residual=True" in repr(layer)


# ------------------------------------------------------------ band dispatch ---


def _fused_layer_with_spies(monkeypatch, backend, lut_max_tokens=16, tile_max_tokens=0, wide_max_tokens=16):
    monkeypatch.setattr(vqmod, "_FUSED_MAX_TOKENS", 16)
    monkeypatch.setattr(vqmod, "_FUSED_WIDE_MAX_TOKENS", wide_max_tokens)  # 16: no 17..32-token GEMV band
    monkeypatch.setattr(vqmod, "_LUT_MAX_TOKENS", lut_max_tokens)
    monkeypatch.setattr(vqmod, "_TILE_MAX_TOKENS", tile_max_tokens)
    monkeypatch.setattr(vqmod, "_TILE_MIN_GRID_FRACTION", 0.0)
    lin = _make_linear_with_vq(16, 32)
    layer = NPVQLinear.from_qtensor_linear(lin, VQProxy(lin.weight.qscheme.centroids), backend=backend)
    calls = []
    fused = {Backend.CUDA_WMMA: "_forward_cuda_wmma", Backend.CUDA_LUT: "_forward_cuda_lut",
             Backend.CUDA: "_forward_cuda"}[backend]
    monkeypatch.setattr(layer, fused, lambda x: calls.append("fused") or x[..., :16])
    monkeypatch.setattr(layer, "_forward_dequant_gemm", lambda x: calls.append("dense") or x[..., :16])
    monkeypatch.setattr(layer, "_forward_tile_gemm", lambda x: calls.append("tile") or x[..., :16])
    return layer, calls


@pytest.mark.parametrize("backend", [Backend.CUDA_WMMA, Backend.CUDA])
def test_mid_sized_batches_use_tile_band(monkeypatch, backend):
    # the sequence asserted at tests/nn/test_np_vq_linear.py:449-456 of the reference
    layer, calls = _fused_layer_with_spies(monkeypatch, backend, tile_max_tokens=64)
    for m in (16, 17, 64, 65):
        layer(torch.randn(m, 32, dtype=torch.float16))
    assert calls == ["fused", "tile", "tile", "dense"]


def test_small_activations_keep_the_gemv_up_to_32_tokens(monkeypatch):
    """17..32 tokens stay in band (a) while tokens x in_features is within the cap."""
    layer, calls = _fused_layer_with_spies(monkeypatch, Backend.CUDA_WMMA, tile_max_tokens=64, wide_max_tokens=32)
    for m in (16, 17, 32, 33):
        layer(torch.randn(m, 32, dtype=torch.float16))
    assert calls == ["fused", "fused", "fused", "tile"]
    del calls[:]
    monkeypatch.setattr(vqmod, "_FUSED_WIDE_MAX_ACTIVATIONS", 20 * 32)
    for m in (17, 20, 21, 32):
        layer(torch.randn(m, 32, dtype=torch.float16))
    assert calls == ["fused", "fused", "tile", "tile"]
    # a raised fused threshold is taken as given
    monkeypatch.setattr(vqmod, "_FUSED_MAX_TOKENS", 24)
    assert layer._gemv_max_tokens(30) == 24


def test_lut_layers_skip_tile_band(monkeypatch):
    layer, calls = _fused_layer_with_spies(monkeypatch, Backend.CUDA_LUT, lut_max_tokens=0, tile_max_tokens=64)
    layer(torch.randn(8, 32, dtype=torch.float16))
    assert calls == ["dense"]


@pytest.mark.parametrize("backend", [Backend.CUDA_WMMA, Backend.CUDA_LUT, Backend.CUDA])
def test_fused_band_up_to_threshold_then_dense(monkeypatch, backend):
    layer, calls = _fused_layer_with_spies(monkeypatch, backend)
    layer(torch.randn(1, 32, dtype=torch.float16))
    layer(torch.randn(2, 8, 32, dtype=torch.float16))  # 16 tokens: leading dims count as tokens
    layer(torch.randn(17, 32, dtype=torch.float16))
    layer(torch.randn(2, 9, 32, dtype=torch.float16))
    assert calls == ["fused", "fused", "dense", "dense"]


def test_lut_backend_uses_dequant_gemm_by_default(monkeypatch):
    layer, calls = _fused_layer_with_spies(monkeypatch, Backend.CUDA_LUT, lut_max_tokens=0)
    layer(torch.randn(1, 32, dtype=torch.float16))
    assert calls == ["dense"]


def test_fp32_activations_take_decode_gemm(monkeypatch):
    layer, calls = _fused_layer_with_spies(monkeypatch, Backend.CUDA_WMMA, tile_max_tokens=64)
    layer(torch.randn(1, 32))
    assert calls == ["dense"]


def test_hip_backend_fails_loudly_without_gpu():
    """No silent fallback: a HIP backend on CPU tensors is an error unless opted in."""
    lin = _make_linear_with_vq(16, 32)
    layer = NPVQLinear.from_qtensor_linear(lin, VQProxy(lin.weight.qscheme.centroids), backend="cuda_wmma")
    with pytest.raises(RuntimeError, match="GPU"):
        layer(torch.randn(1, 32, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="GPU"):
        layer(torch.randn(40, 32, dtype=torch.float16))


def test_opt_in_fallback_warns_once_and_latches(monkeypatch, caplog):
    import neuropress_amd.kernels as K

    monkeypatch.setattr(vqmod, "_ALLOW_FALLBACK", True)
    monkeypatch.setattr(vqmod, "_tile_failed", False)
    monkeypatch.setattr(vqmod, "_TILE_MAX_TOKENS", 64)
    monkeypatch.setattr(vqmod, "_TILE_MIN_GRID_FRACTION", 0.0)
    monkeypatch.setattr(K, "_warned_fallbacks", set())
    lin = _make_linear_with_vq(16, 32)
    layer = NPVQLinear.from_qtensor_linear(lin, VQProxy(lin.weight.qscheme.centroids), backend="cuda_wmma")
    x = torch.randn(40, 32, dtype=torch.bfloat16)
    caplog.set_level(logging.WARNING, logger="neuropress_amd.kernels")
    y1, y2 = layer(x), layer(x)
    ref = NPVQLinear.from_qtensor_linear(lin, VQProxy(lin.weight.qscheme.centroids), backend="default")(x)
    assert torch.equal(y1, ref) and torch.equal(y2, ref)
    assert vqmod._tile_failed is True
    msgs = [r.getMessage() for r in caplog.records]
    assert sum("vq_gemm_tile" in m for m in msgs) == 1 and sum("vq_dequant" in m for m in msgs) == 1


# --------------------------------------------------------- backend resolution ---


def test_backend_resolution():
    assert _resolve_vq_backend(None) == VQBackend.DEFAULT == _resolve_vq_backend("torch")
    assert _resolve_vq_backend(Backend.CUDA_TIERED) == VQBackend.CUDA_TIERED
    with pytest.raises(ValueError, match=r"(?i)gemlite"):
        _resolve_vq_backend(Backend.GEMLITE)
    if not torch.cuda.is_available():
        assert _resolve_vq_backend(Backend.AUTO) == VQBackend.COMPILE
        assert _resolve_backend("auto", 4, 32) == LinearBackend.COMPILE
    assert _resolve_backend(None) == LinearBackend.DEFAULT
    with pytest.raises(ValueError):
        _resolve_backend("nope")
    assert VQBackend.CUDA_WMMA == "cuda_wmma" and f"{VQBackend.CUDA_LUT}" == "cuda_lut"


# ------------------------------------------------------------------ NPLinear ---


def test_nplinear_matches_closed_form_and_round_trips():
    codes = torch.randint(0, 16, (16, 64), dtype=torch.int64).to(torch.uint8)
    scale = (torch.rand(16 * 2) * 0.02 + 0.001).to(torch.float16)
    lin = attach_quantized_weight(nn.Linear(64, 16, bias=True), ScalarQWeight.from_codes(codes, scale, 4, 32))
    layer = NPLinear.from_linear(lin, backend="compile")
    x = torch.randn(4, 64)
    w = ((codes.float() - 8).reshape(16, 2, 32) * scale.float().reshape(16, 2, 1)).reshape(16, 64)
    assert torch.allclose(layer(x), torch.nn.functional.linear(x, w, lin.bias), atol=1e-6)
    restored = layer.to_qtensor()
    assert torch.equal(restored.u8_blob, lin.weight.u8_blob)  # blob preserved bit for bit
    assert torch.equal(restored.decompress_to_u8(), codes)
    assert layer.set_backend("default").backend == LinearBackend.DEFAULT
    with pytest.raises(TypeError):
        NPLinear.from_linear(nn.Linear(4, 4))


def test_nplinear_asym_and_known_answers():
    codes = torch.full((2, 32), 15, dtype=torch.uint8)
    from neuropress_amd.t2n.packing import BitPacking4

    scale = torch.tensor([1e-12, 1.0])
    zp = torch.tensor([2.0, 2.0])
    w = _q_dequant_linear(torch.eye(32), BitPacking4.compress(codes), scale.half(), 4, 32, zp.half(), None).T
    assert torch.all(w[0] == 0) and torch.all(w[1] == 13)


# ------------------------------------------------------------------- lowering ---


class _TwoPath(nn.Module):
    def __init__(self, cb):
        super().__init__()
        self.fc1 = _make_linear_with_vq(16, 32, centroids=cb)
        self.fc2 = _make_linear_with_vq(8, 32, centroids=cb)
        codes = torch.randint(0, 16, (8, 32), dtype=torch.int64).to(torch.uint8)
        self.q = attach_quantized_weight(nn.Linear(32, 8, bias=False),
                                         ScalarQWeight.from_codes(codes, torch.rand(8).half(), 4, 32))
        self.plain = nn.Linear(32, 8)

    def forward(self, x):
        return self.fc2(x) + self.fc1(x)[:, :8] + self.q(x) + self.plain(x)


def test_auto_lowering_swaps_modules_and_shares_proxy(caplog):
    cb = torch.randn(8, 4, dtype=torch.float16)
    model = _TwoPath(cb)
    model.config = type("C", (), {"tie_word_embeddings": True})()
    caplog.set_level(logging.WARNING)
    AutoKernelLowering.from_config({"vq_backend": "default"}).apply(model)
    assert isinstance(model.fc1, NPVQLinear) and isinstance(model.fc2, NPVQLinear) and isinstance(model.q, NPLinear)
    assert isinstance(model.plain, nn.Linear)
    assert model.fc1.proxy is model.fc2.proxy
    assert [n for n, m in model.named_modules() if isinstance(m, VQProxy)] == ["_vq_proxy_0"]
    assert model.config.tie_word_embeddings is False
    assert any("Kernel lowering applied" in r.getMessage() for r in caplog.records)
    assert is_lowered(model)
    keys = set(model.state_dict())
    assert {"fc1.packed_indices", "fc2.packed_indices", "_vq_proxy_0.centroids", "q.u8_blob", "q.scale"} <= keys
    y = model(torch.randn(2, 32))
    assert y.shape == (2, 8)
    unlower_model(model)
    assert not is_lowered(model) and isinstance(model.fc1, nn.Linear)
    assert not any(n.startswith("_vq_proxy_") for n, _ in model.named_children())
    AutoKernelLowering(vq_backend="default", linear_backend="compile").apply(model)  # re-lower
    assert torch.allclose(model(torch.ones(1, 32)), model(torch.ones(1, 32)))


def test_distinct_codebooks_get_distinct_proxies():
    class M(nn.Module):
        def __init__(self):
            super().__init__()
            self.a = _make_linear_with_vq(16, 32)
            self.b = _make_linear_with_vq(8, 32)

    m = linearize_vq_weights(M(), backend="default")
    assert m.a.proxy is not m.b.proxy
    assert len([1 for x in m.modules() if isinstance(x, VQProxy)]) == 2


def test_lowering_config(tmp_path):
    cfg = LoweringConfig.from_dict({"vq_backend": "cuda"})
    assert cfg.vq_backend == "cuda" and cfg.linear_backend == "auto"
    with pytest.raises(ValueError, match="Unknown lowering config"):
        LoweringConfig.from_dict({"bogus": 1})
    cfg.save(tmp_path / "l.yaml")
    assert LoweringConfig.load(tmp_path / "l.yaml") == cfg
    assert LoweringConfig.load(None) == LoweringConfig()
    low = AutoKernelLowering.from_config(tmp_path / "l.yaml")
    assert low.vq_backend == "cuda" and low.norm_backend == "auto"


# -------------------------------------------------------------------- warnings ---


def test_warn_kernel_fallback_once_per_kernel(caplog):
    from neuropress_amd.kernels import warn_kernel_fallback

    caplog.set_level(logging.WARNING, logger="neuropress_amd.kernels")
    for _ in range(3):
        warn_kernel_fallback("test_kernel_a", "slow path", RuntimeError("libnpamd.so does not exist"))
    warn_kernel_fallback("test_kernel_b", "x", RuntimeError("b"))
    a = [r.getMessage() for r in caplog.records if "test_kernel_a" in r.getMessage()]
    assert len(a) == 1 and "does not exist" in a[0] and "slow path" in a[0] and "neuropress_amd.build" in a[0]
    assert any("test_kernel_b" in r.getMessage() for r in caplog.records)


# ------------------------------------------------------------------------ ABI ---


def test_library_exports_every_declared_symbol():
    """Every function include/npamd.h (the drop-in contract) and include/npamd_diag.h (measurement
    aids) declare is exported by the built library and bound by the ctypes layer (no compute calls:
    there is no GPU here)."""
    from neuropress_amd import _lib

    header = (ROOT / "include" / "npamd.h").read_text()
    declared = set(re.findall(r"\b(npamd_[a-z0-9_]+)\s*\(", header))
    assert {"npamd_vq_gemv", "npamd_vq_gemm_tile", "npamd_vq_dequant", "npamd_q_gemv"} <= declared
    assert not any(name.startswith("npamd_diag_") for name in declared), "measurement aids belong in npamd_diag.h"
    diag = set(re.findall(r"\b(npamd_diag_[a-z0-9_]+)\s*\(", (ROOT / "include" / "npamd_diag.h").read_text()))
    assert {"npamd_diag_reload_tuning", "npamd_diag_stream_read", "npamd_diag_mfma"} <= diag
    declared |= diag
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in npamd.h but not exported"
    assert declared - {"npamd_version", "npamd_last_error"} == set(_lib.SIGNATURES)
    loaded = _lib.load()
    assert loaded.npamd_version() == _lib.ABI_VERSION
    assert isinstance(loaded.npamd_last_error(), bytes)  # "" or the last failing call of this thread


def test_c_abi_validates_arguments_without_a_gpu():
    """Argument checks run before any HIP call, so bad calls fail cleanly on a CPU-only host."""
    from neuropress_amd import _lib

    with pytest.raises(RuntimeError, match=r"bits must be in \[4, 20\]"):
        _lib.call("npamd_vq_dequant", None, 0, 3, None, 16, 8, 0, None, 0, None)
    with pytest.raises(RuntimeError, match="too short"):
        _lib.call("npamd_vq_dequant", None, 1, 8, None, 16, 8, 100, None, 0, None)
    with pytest.raises(RuntimeError, match="nbits"):
        _lib.call("npamd_q_dequant", None, None, None, 4, 64, 3, 32, None, 0, None)
    with pytest.raises(RuntimeError, match="not divisible"):
        _lib.call("npamd_vq_gemv", None, 64, None, 0, 8, None, 0, 16, 8, None, None, 4, 1, 4, 60, 0, None)
    with pytest.raises(RuntimeError, match="exceeds the fused limit"):
        _lib.call("npamd_vq_gemv", None, 64, None, 1 << 20, 8, None, 0, 16, 8, None, None, 4, 33, 4, 64, 0, None)
    _lib.call("npamd_vq_dequant", None, 0, 8, None, 16, 8, 0, None, 0, None)  # empty: success, no launch
    # entry points added around the path: same rule
    with pytest.raises(RuntimeError, match="row stride smaller than the row"):
        _lib.call("npamd_rms_norm", None, 8, None, None, 16, 2, 16, 1e-6, 0, None)
    with pytest.raises(RuntimeError, match="bad dtype code"):
        _lib.call("npamd_rms_norm", None, 16, None, None, 16, 2, 16, 1e-6, 7, None)
    _lib.call("npamd_rms_norm", None, 16, None, None, 16, 0, 16, 1e-6, 0, None)  # no rows: success, no launch
    with pytest.raises(RuntimeError, match="16-bit indices"):
        _lib.call("npamd_vq_embedding", None, 1, None, 10, 4, None, 70000, 8, None, 1.0, None, 0, None)
    with pytest.raises(RuntimeError, match="null pointer"):
        _lib.call("npamd_vq_embedding", None, 1, None, 10, 4, None, 256, 8, None, 1.0, None, 0, None)
    with pytest.raises(RuntimeError, match="nbits must be 1, 2, 4 or 8"):
        _lib.call("npamd_q_embedding", None, 1, None, None, None, 3, 32, 10, 64, -1, 1.0, None, 0, None)
    with pytest.raises(RuntimeError, match="bad shape"):
        _lib.call("npamd_q_embedding", None, 1, None, None, None, 4, 48, 10, 64, -1, 1.0, None, 0, None)
    with pytest.raises(RuntimeError, match="column_perm needs"):
        _lib.call("npamd_vq_gemv_perm", 16, 8192, 16, 16, 1 << 20, 16, 16, 0, 65536, 8, None, 16, 64, 9, 64, 8192, 0, None)
    lib = _lib.load()
    assert lib.npamd_vq_gemv_perm_supported(1, 2048, 2048, 4096, 8, 12) == 1
    assert lib.npamd_vq_gemv_perm_supported(1, 2048, 2048, 4096, 4, 12) == 1  # vector length 4
    assert lib.npamd_vq_gemv_perm_supported(1, 2048, 2048, 4096, 6, 12) == 0  # vector length 6
    assert lib.npamd_vq_gemv_perm_supported(5, 2048, 4096, 4096, 8, 12) == 0  # 5 * 4096 elements > 16384
    # which layers the MFMA kernels take (the rest run element-wise kernels; the modules send
    # them to decode + GEMM beyond 16 tokens)
    assert lib.npamd_vq_fused_supported(4096, 8, 12) == 1 and lib.npamd_vq_fused_supported(4096, 8, 16) == 1
    assert lib.npamd_vq_fused_supported(4096, 4, 12) == 1  # vector length 4: two rows per operand
    assert lib.npamd_vq_fused_supported(4096, 2, 12) == 0 and lib.npamd_vq_fused_supported(4096, 16, 12) == 0
    assert lib.npamd_vq_fused_supported(4096, 8, 10) == 0  # 10-bit stream (the module widens it to 16 first)
    assert lib.npamd_vq_fused_supported(4096 + 32, 8, 12) == 0  # K not a multiple of 64
    assert lib.npamd_q_fused_supported(4096, 4, 32) == 1 and lib.npamd_q_fused_supported(4096, 4, 128) == 1
    assert lib.npamd_q_fused_supported(4096, 8, 32) == 1 and lib.npamd_q_fused_supported(4096, 8, 64) == 1
    assert lib.npamd_q_fused_supported(4096, 2, 32) == 0 and lib.npamd_q_fused_supported(4096, 4, 96) == 0
    assert lib.npamd_q_fused_supported(4096, 4, 16) == 0 and lib.npamd_q_fused_supported(4096 + 32, 4, 32) == 0


def test_tile_band_rule_counts_reduction_splits():
    """Layers with few output features take the tile band only while the kernel's
    reduction split can fill the compute units (256 here) and, for short
    reductions, only up to the split band's token limit."""
    from neuropress_amd.nn.backends import tile_band_ok

    def ok(m, n, k):
        return tile_band_ok(m, n, k, 256, 0.7, 128, 8192)

    assert ok(64, 14336, 4096) and ok(256, 14336, 4096)  # grid fills the GPU by itself
    assert ok(64, 4096, 14336) and ok(256, 4096, 14336)  # 64 tiles x 4 splits, long reduction
    assert ok(128, 4096, 4096) and not ok(129, 4096, 4096)  # short reduction: up to 128 tokens
    assert not ok(17, 1024, 4096)  # 16 tiles x 8 splits = half the compute units
    assert not ok(17, 4096, 512)  # no split possible below 1024 input features
    assert ok(17, 2048, 4096)  # 32 tiles x 8 splits


@pytest.mark.parametrize("kind", ["tiered", "tiered_hot8", "ntier", "zero_escape"])
def test_prefix_coded_layers_expand_to_the_fixed_width_stream(kind):
    """A layer built from a two-tier / n-tier / zero-escape buffer (reference:
    np_vq_linear.py:504-511, 573-640) holds the same fixed-width stream, gives the same output and
    packs back to the same bytes as the reference's formats define."""
    from neuropress_amd.transforms.vq_packing import (
        IndexPacking,
        NTieredIndexPacking,
        TieredIndexPacking,
        ZeroEscapePacking,
    )

    n, k, nc = 24, 64, 1024
    g = torch.Generator().manual_seed(11)
    cb = torch.randn(nc, 8, generator=g) * 0.05
    p = 1.0 / torch.arange(1, nc + 1, dtype=torch.float64) ** 1.1
    idx = torch.multinomial(p / p.sum(), n * k // 8, replacement=True, generator=g)
    kw = {"tiered": dict(use_tiered=True), "tiered_hot8": dict(use_tiered=True, hot_bits=8),
          "ntier": dict(tier_bits=[4, 8, 10]), "zero_escape": dict(zero_escape=True)}[kind]
    wq = VQWeight.from_indices(idx, cb, n, k, bits=10, **kw)
    coded = wq.u8_blob
    want = {"tiered": TieredIndexPacking.pack(idx, 10), "tiered_hot8": TieredIndexPacking.pack(idx, 10, 8),
            "ntier": NTieredIndexPacking.pack(idx, [4, 8, 10]), "zero_escape": ZeroEscapePacking.pack(idx, 10)}[kind]
    assert torch.equal(coded, want)
    lin = attach_quantized_weight(nn.Linear(k, n, bias=True), wq)
    plain = NPVQLinear(VQProxy(cb), IndexPacking.pack(idx, 10), 10, n, k, 8, "default", bias=lin.bias.detach())
    layer = NPVQLinear.from_qtensor_linear(lin, VQProxy(cb), backend="default")
    assert layer.bits == 10 and torch.equal(layer.packed_indices, plain.packed_indices)
    assert (layer.use_tiered, layer.tier_bits, layer.zero_escape) == (
        kind.startswith("tiered"), [4, 8, 10] if kind == "ntier" else None, kind == "zero_escape")
    x = torch.randn(5, k, generator=g)
    assert torch.equal(layer(x), plain(x))
    assert {"tiered": "tiered=True(cold=10)", "tiered_hot8": "tiered=True(cold=10)", "ntier": "ntier=[4, 8, 10]",
            "zero_escape": "zero_escape=True"}[kind] in layer.extra_repr()
    back = layer.to_qtensor()
    assert torch.equal(back.u8_blob, coded)  # byte-identical round trip, hot_bits included
    assert (back.qscheme.use_tiered, back.qscheme.tier_bits, back.qscheme.zero_escape) == (
        layer.use_tiered, layer.tier_bits, layer.zero_escape)
    w = cb.half()[idx].reshape(n, k).float()  # the proxy keeps the codebook in fp16
    assert torch.equal(back.qscheme.dequantize(back.u8_blob, torch.float32), w)
    with pytest.raises(ValueError, match="past the end of the codebook"):
        NPVQLinear(VQProxy(cb[:512]), coded, 10, n, k, 8, "default", **{a: b for a, b in kw.items() if a != "hot_bits"})


def test_prefix_coded_backends_resolve_like_the_reference(monkeypatch):
    """"auto" with a format flag: zero-escape > n-tier > tiered when the HIP backend can run
    (np_vq_linear.py:158-163), COMPILE otherwise; the explicit members are accepted."""
    import neuropress_amd.nn.np_vq_linear as vqmod

    res = vqmod._resolve_vq_backend
    assert res("auto", use_tiered=True).value == "compile"  # no GPU here
    monkeypatch.setattr(vqmod.torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(vqmod, "is_hip_backend_available", lambda: True)
    assert res("auto", use_tiered=True, use_ntier=True, use_zero_escape=True).value == "cuda_zero_escape"
    assert res("auto", use_tiered=True, use_ntier=True).value == "cuda_ntier"
    assert res("auto", use_tiered=True).value == "cuda_tiered"
    assert res("auto").value == "cuda_wmma"
    assert res("cuda_tiered").value == "cuda_tiered"


def test_modules_built_under_inference_mode_keep_their_caches_working():
    """Inference tensors raise on ``_version``; the caches of derived tensors (fp32 bias, codebook
    casts) key on device and address for them (the reference quantises under inference mode,
    neuropress/methods/gptq.py:253)."""
    from neuropress_amd.nn import NPLinear, NPVQLinear, VQProxy
    from neuropress_amd.nn.backends import tensor_version
    from tests import cases

    L = cases.vq_layer(5, 32, 64, 256, bits=8, act=torch.float32, m=3, bias=True)
    Q = cases.q4_layer(6, 32, 64, act=torch.float32, m=3, bias=True)
    with torch.inference_mode():
        t = torch.zeros(4)
        assert tensor_version(t) == -1
        vq = NPVQLinear(VQProxy(L["cb"].clone()), L["packed"].clone(), 8, 32, 64, 8, "default", bias=L["bias"].clone())
        ql = NPLinear(Q["blob"].clone(), Q["scale"].clone(), 32, 64, 32, 4, "sym", "default", bias=Q["bias"].clone())
        assert vq._bias_f32().dtype == torch.float32 and vq._bias_f32() is vq._bias_f32()  # cached
        assert ql._bias_f32() is ql._bias_f32()
        assert vq.proxy.centroids_as(torch.bfloat16) is vq.proxy.centroids_as(torch.bfloat16)
        vq.prepare()
        y = vq(L["x"])
        yq = ql(Q["x"])
    w = L["cb"][L["idx"]].reshape(32, 64).float()
    assert torch.allclose(y, L["x"] @ w.T + L["bias"], atol=1e-4)
    wq = ((Q["codes"].float() - 8).reshape(32, 2, 32) * Q["scale"].float().reshape(32, 2, 1)).reshape(32, 64)
    assert torch.allclose(yq, Q["x"] @ wq.T + Q["bias"], atol=1e-3)
    assert tensor_version(torch.zeros(2)) == 0
