"""Checkpoint round trips (safetensors) of quantized models: file layout as the reference's
save_quantized_model / load_quantized_model (neuropress/t2n/model_io.py:55-67, 214-310, 463-596),
component names and metadata as its per-type serdes (neuropress/t2n/qtensors.py:302-548)."""

import json

import pytest
import torch
import torch.nn as nn
from safetensors import safe_open
from safetensors.torch import save_file

from neuropress_amd import AutoKernelLowering, is_lowered
from neuropress_amd.nn import NPLinear, NPVQLinear
from neuropress_amd.qweights import ScalarQWeight, VQWeight, attach_quantized_weight
from neuropress_amd.t2n.model_io import attach_manifest, load_quantized_model, save_quantized_model
from neuropress_amd.transforms.vq_packing import NTieredIndexPacking


def _zipf(n, nc, g):
    p = 1.0 / torch.arange(1, nc + 1, dtype=torch.float64) ** 1.1
    return torch.multinomial(p / p.sum(), n, replacement=True, generator=g)


class Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.norm = nn.LayerNorm(64)
        self.vq_a = nn.Linear(64, 48, bias=True)
        self.vq_b = nn.Linear(64, 32, bias=False)   # shares vq_a's codebook
        self.vq_tier = nn.Linear(64, 16, bias=False)
        self.vq_ntier = nn.Linear(64, 16, bias=False)
        self.vq_zesc = nn.Linear(64, 16, bias=False)
        self.q4 = nn.Linear(64, 24, bias=True)
        self.q4zp = nn.Linear(64, 24, bias=False)
        self.plain = nn.Linear(64, 8)

    def forward(self, x):
        x = self.norm(x)
        return torch.cat([m(x) for m in (self.vq_a, self.vq_b, self.vq_tier, self.vq_ntier, self.vq_zesc,
                                         self.q4, self.q4zp, self.plain)], dim=-1)


def _quantized_net(seed=3):
    g = torch.Generator().manual_seed(seed)
    torch.manual_seed(seed)
    net = Net()
    cb = (torch.randn(512, 8, generator=g) * 0.05).half()
    cb_big = (torch.randn(2048, 8, generator=g) * 0.05).half()
    perm = torch.randperm(64, generator=g)
    attach_quantized_weight(net.vq_a, VQWeight.from_indices(_zipf(48 * 8, 512, g), cb, 48, 64, column_permutation=perm))
    attach_quantized_weight(net.vq_b, VQWeight.from_indices(_zipf(32 * 8, 512, g), cb, 32, 64))
    attach_quantized_weight(net.vq_tier, VQWeight.from_indices(_zipf(128, 2048, g), cb_big, 16, 64, use_tiered=True, hot_bits=8))
    attach_quantized_weight(net.vq_ntier, VQWeight.from_indices(_zipf(128, 2048, g), cb_big, 16, 64, tier_bits=[4, 8, 11]))
    attach_quantized_weight(net.vq_zesc, VQWeight.from_indices(_zipf(128, 2048, g), cb_big, 16, 64, zero_escape=True))
    codes = torch.randint(0, 16, (24, 64), generator=g, dtype=torch.uint8)
    scale = (torch.rand(24 * 2, generator=g) * 0.02 + 0.001).half()
    attach_quantized_weight(net.q4, ScalarQWeight.from_codes(codes, scale, 4, 32))
    zp = torch.randint(0, 16, (24 * 2,), generator=g).half()
    attach_quantized_weight(net.q4zp, ScalarQWeight.from_codes(codes, scale, 4, 32, zero_point=zp))
    return net


def _same_weight(a, b):
    assert type(a) is type(b)
    assert torch.equal(a.u8_blob, b.u8_blob)
    qa, qb = a.qscheme, b.qscheme
    if isinstance(a, VQWeight):
        assert torch.equal(qa.centroids, qb.centroids) and tuple(qa.original_shape) == tuple(qb.original_shape)
        assert (qa.is_packed_indices, qa.use_tiered, qa.tier_bits, qa.zero_escape) == (
            qb.is_packed_indices, qb.use_tiered, qb.tier_bits, qb.zero_escape)
        assert (qa.column_permutation is None) == (qb.column_permutation is None)
        if qa.column_permutation is not None:
            assert torch.equal(qa.column_permutation, qb.column_permutation)
    else:
        assert (qa.n_bits, qa.group_size) == (qb.n_bits, qb.group_size) and torch.equal(qa.scale, qb.scale)
        assert (qa.zero_point is None) == (qb.zero_point is None)
        if qa.zero_point is not None:
            assert torch.equal(qa.zero_point, qb.zero_point)
        assert [c.nbits for c in a.u8_compressors] == [c.nbits for c in b.u8_compressors]


def test_file_layout_matches_the_reference_convention(tmp_path):
    net = _quantized_net()
    path = tmp_path / "ckpt.safetensors"
    save_quantized_model(net, path, recipe_config_json=json.dumps({"name": "unit"}))
    with safe_open(str(path), framework="pt") as f:
        keys, meta = set(f.keys()), f.metadata()
    assert {"vq_a.weight::u8_blob", "vq_a.weight::centroids", "vq_a.weight::column_permutation", "vq_a.bias",
            "vq_b.weight::u8_blob", "q4.weight::u8_blob", "q4.weight::scale", "q4zp.weight::zero_point",
            "norm.weight", "plain.weight", "plain.bias"} <= keys
    assert "vq_b.weight::column_permutation" not in keys and "vq_a.weight" not in keys
    manifest = json.loads(meta["__neuropress_manifest__"])
    assert manifest["format_version"] == "2" and manifest["recipe_config"] == {"name": "unit"}
    (assign,) = [t for t in manifest["transforms"] if t["type"] == "qtensor_assignment"]
    entry = assign["qtensor_params"]["vq_a.weight"]
    assert entry["type"] == "QTensorTractVQ" and entry["tensor_keys"] == ["u8_blob", "centroids", "column_permutation"]
    assert set(entry["metadata"]) == {"proxy_selector", "original_shape", "bits_per_index", "dequant_to_dtype",
                                      "proxy_content_hash", "has_column_perm", "use_tiered", "zero_escape"}
    assert entry["metadata"]["original_shape"] == "48,64" and entry["metadata"]["bits_per_index"] == "9"
    assert entry["metadata"]["has_column_perm"] == "1" and len(entry["metadata"]["proxy_content_hash"]) == 64
    assert assign["qtensor_params"]["vq_tier.weight"]["metadata"]["use_tiered"] == "1"
    assert assign["qtensor_params"]["vq_zesc.weight"]["metadata"]["zero_escape"] == "1"
    assert json.loads(assign["qtensor_params"]["vq_ntier.weight"]["metadata"]["tier_bits"]) == [4, 8, 11]
    q4 = assign["qtensor_params"]["q4.weight"]
    assert q4["type"] == "QTensorTractScaleOnly" and q4["tensor_keys"] == ["u8_blob", "scale"]
    assert q4["metadata"] == {"shape": "[24, 64]", "packing": "[4]", "n_bits": "4", "group_size": "32",
                              "dequant_to_dtype": "float16", "nnef_name": ""}
    assert assign["qtensor_params"]["q4zp.weight"]["type"] == "QTensorScaleZp"


def test_round_trip_without_lowering_restores_every_weight(tmp_path):
    net = _quantized_net()
    path = tmp_path / "ckpt.safetensors"
    save_quantized_model(net, path)
    fresh = Net()
    manifest = load_quantized_model(fresh, path, kernel_lowering=None)
    assert manifest.qtensor_params["q4zp.weight"] == "QTensorScaleZp" and len(manifest.qtensor_params) == 7
    for name in ("vq_a", "vq_b", "vq_tier", "vq_ntier", "vq_zesc", "q4", "q4zp"):
        _same_weight(getattr(net, name).weight, getattr(fresh, name).weight)
    # layers saved with one codebook share one tensor object again: lowering then shares one proxy
    assert fresh.vq_a.weight.qscheme.centroids is fresh.vq_b.weight.qscheme.centroids
    assert fresh.vq_a.weight.qscheme.centroids is not fresh.vq_tier.weight.qscheme.centroids
    assert torch.equal(fresh.plain.weight, net.plain.weight) and torch.equal(fresh.vq_a.bias, net.vq_a.bias)
    assert not is_lowered(fresh)


def test_load_lowers_and_a_lowered_model_saves_the_same_file(tmp_path):
    net = _quantized_net()
    p1, p2 = tmp_path / "a.safetensors", tmp_path / "b.safetensors"
    save_quantized_model(net, p1)
    loaded = Net()
    load_quantized_model(loaded, p1)  # kernel_lowering="auto"
    assert is_lowered(loaded) and isinstance(loaded.vq_a, NPVQLinear) and isinstance(loaded.q4, NPLinear)
    assert loaded.vq_a.proxy is loaded.vq_b.proxy
    ref = Net()
    load_quantized_model(ref, p1, kernel_lowering=None)
    AutoKernelLowering(vq_backend="default", linear_backend="compile").apply(ref)
    x = torch.randn(3, 64)
    assert torch.allclose(loaded(x), ref(x), atol=1e-5)
    save_quantized_model(loaded, p2)  # unlowers, saves, lowers again
    assert is_lowered(loaded)
    with safe_open(str(p1), framework="pt") as fa, safe_open(str(p2), framework="pt") as fb:
        assert set(fa.keys()) == set(fb.keys())
        for k in fa.keys():
            assert torch.equal(fa.get_tensor(k), fb.get_tensor(k)), k
        ma, mb = (json.loads(f.metadata()["__neuropress_manifest__"]) for f in (fa, fb))
    assert ma == mb


def test_files_written_without_this_backends_additions_still_load(tmp_path):
    """A writer that records neither tier_bits (the reference's) nor shape / packing (its older
    files): n-tier buffers are recognised by their header, scalar layouts by the blob size."""
    net = _quantized_net()
    attach_manifest(net)
    path = tmp_path / "old.safetensors"
    save_quantized_model(net, path)
    with safe_open(str(path), framework="pt") as f:
        tensors = {k: f.get_tensor(k) for k in f.keys()}
        manifest = json.loads(f.metadata()["__neuropress_manifest__"])
    params = manifest["transforms"][0]["qtensor_params"]
    del params["vq_ntier.weight"]["metadata"]["tier_bits"]
    for name in ("q4.weight", "q4zp.weight"):
        del params[name]["metadata"]["shape"], params[name]["metadata"]["packing"]
    save_file(tensors, str(path), metadata={"__neuropress_manifest__": json.dumps(manifest)})
    fresh = Net()
    load_quantized_model(fresh, path, kernel_lowering=None)
    assert fresh.vq_ntier.weight.qscheme.tier_bits == [4, 8, 11]
    assert NTieredIndexPacking.is_ntier_buffer(fresh.vq_ntier.weight.u8_blob)
    assert [c.nbits for c in fresh.q4.weight.u8_compressors] == [4]
    _same_weight(net.q4zp.weight, fresh.q4zp.weight)


def test_load_errors(tmp_path):
    path = tmp_path / "plain.safetensors"
    save_file({"w": torch.zeros(2)}, str(path))
    with pytest.raises(ValueError, match="missing the '__neuropress_manifest__' metadata key"):
        load_quantized_model(Net(), path)
    manifest = {"format_version": "2", "transforms": [{"type": "qtensor_assignment", "qtensor_params": {
        "q4.weight": {"type": "QTensorMystery", "tensor_keys": [], "metadata": {}}}}], "recipe_config": None}
    save_file({"w": torch.zeros(2)}, str(path), metadata={"__neuropress_manifest__": json.dumps(manifest)})
    with pytest.raises(ValueError, match="No QTensorSerde registered for type 'QTensorMystery'"):
        load_quantized_model(Net(), path)
    with pytest.raises(ValueError, match="kernel_lowering must be 'auto' or None"):
        load_quantized_model(Net(), path, kernel_lowering="fast")
    split = {"format_version": "2", "recipe_config": None, "transforms": [
        {"type": "mixed_precision_split", "modules": {"vq_a": {"out_features": 48, "split_sizes": [32, 32]}}}]}
    save_file({"w": torch.zeros(2)}, str(path), metadata={"__neuropress_manifest__": json.dumps(split)})
    with pytest.raises(ValueError, match="mixed_precision_split"):  # changes the module tree: refused, not skipped
        load_quantized_model(Net(), path)


@pytest.mark.gpu
def test_checkpoint_loaded_onto_the_gpu_runs_the_hip_kernels(tmp_path):
    """save_quantized_model -> load_quantized_model(kernel_lowering="auto") into a model that lives on
    the GPU -> forward: every quantized layer computes with the HIP kernels and matches the
    unlowered model's torch-op forward of the same checkpoint (fp16, 1 and 40 tokens)."""
    from neuropress_amd import kernels

    gpu = torch.device("cuda:0")
    src = _quantized_net()
    attach_manifest(src)
    path = tmp_path / "net.safetensors"
    save_quantized_model(src, path)
    ref = Net()
    load_quantized_model(ref, path, kernel_lowering=None)
    AutoKernelLowering(vq_backend="default", linear_backend="compile").apply(ref)  # torch-op paths on the CPU
    model = Net().half().to(gpu)
    calls = []
    patched = {}
    for name in ("vq_linear", "q_linear", "vq_gemm_tile", "q_gemm_tile", "vq_dequant", "q_dequant"):
        real = getattr(kernels, name)
        patched[name] = real
        setattr(kernels, name, lambda *a, _r=real, _n=name, **kw: (calls.append(_n), _r(*a, **kw))[1])
    try:
        load_quantized_model(model, path)  # kernel_lowering="auto"
        assert is_lowered(model) and model.vq_a.packed_indices.is_cuda and model.q4.u8_blob.is_cuda
        assert model.vq_a.backend.value.startswith("cuda") and model.q4.backend.value == "cuda"
        for m in (1, 40):
            x = torch.randn(m, 64, generator=torch.Generator().manual_seed(m))
            y = model(x.half().to(gpu)).float().cpu()
            want = ref.float()(x.half().float())
            assert (y - want).abs().max().item() <= 1e-2 + 1e-2 * want.abs().max().item()
    finally:
        for name, real in patched.items():
            setattr(kernels, name, real)
    assert "vq_linear" in calls and "q_linear" in calls  # the HIP entry points did the work
