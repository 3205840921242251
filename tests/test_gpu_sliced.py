"""Parity of the slice-list decode GEMV against the CPU oracle, through the C ABI.

Bar: outputs within 1e-2 abs + 1e-2 rel of the oracle's double-accumulated
contraction of the oracle-decoded weight; results identical from run to run.
"""

import numpy as np
import pytest
import torch

from oracle import oracle as orc
from tests import cases

pytestmark = pytest.mark.gpu


def _vq_ref(oracle_lib, L, act):
    code = orc.torch_dtype_code(act)
    w = oracle_lib.vq_decode(L["packed"].numpy(), L["bits"], orc.to_bits(L["cb"]), L["n"], L["k"], code)
    bias = None if L["bias"] is None else orc.to_bits(L["bias"])
    return oracle_lib.linear_f64(orc.to_bits(L["x"]), code, w, code, bias, code)


def _check(y: torch.Tensor, ref: np.ndarray):
    ok, max_abs, excess = cases.within_tol(y.float().cpu().numpy(), ref)
    assert ok, f"max abs err {max_abs:.3e}, {excess:.2f}x the 1e-2 bound"


def _run(gpu, L, act, **kw):
    from neuropress_amd import kernels

    sl = kernels.vq_slice_indices(L["packed"], L["bits"], L["n"], L["k"], 8, L["nc"], device=gpu)
    bias = None if L["bias"] is None else L["bias"].to(gpu)
    return kernels.vq_linear_sliced(L["x"].to(gpu), sl, L["cb"].to(act).to(gpu), bias, **kw), sl


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize(
    "n,k,nc,bits",
    [
        (72, 96, 300, None),  # one slice
        (130, 8, 9000, None),  # a single group, two slices
        (1000, 64, 20000, None),  # short last slice
        (1100, 256, 65536, 16),  # two row blocks
        (300, 128, 4096, 12),
        (96, 12296, 65536, 16),  # K / 8 = 1537 groups: two group ranges are forced
    ],
)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 9, 16])
def test_sliced_gemv_matches_oracle(gpu, oracle_lib, act, n, k, nc, bits, m):
    L = cases.vq_layer(900 + n + m, n, k, nc, bits=bits, act=act, m=m, bias=True, std=0.05)
    y, _ = _run(gpu, L, act)
    assert y.shape == (m, n) and y.dtype == act
    _check(y, _vq_ref(oracle_lib, L, act))


def test_sliced_gemv_zipf_indices(gpu, oracle_lib):
    """Config-4-like index statistics: slice 0 receives most entries and gets more group ranges."""
    from neuropress_amd.transforms.vq_packing import IndexPacking

    n, k, nc, act = 517, 1024, 65536, torch.float16
    L = cases.vq_layer(77, n, k, nc, bits=16, act=act, m=2, bias=False, std=0.05)
    idx = cases.zipf_indices(cases.gen(78), nc, n * (k // 8))
    L["idx"], L["packed"] = idx, IndexPacking.pack(idx, 16)
    y, sl = _run(gpu, L, act)
    assert sl.n_partials > sl.n_slices  # the hot slice was split over several group ranges
    _check(y, _vq_ref(oracle_lib, L, act))


def test_sliced_gemv_full_size_and_fused_gemv_agree(gpu, oracle_lib):
    """The headline benchmark shape (14336 x 4096, 65536 x 8 codebook, bf16), one token: against the
    oracle, against the fused GEMV (same f32-accumulated sum in another order), run to run,
    and the workspace comes back zero-filled."""
    from neuropress_amd import kernels

    act = torch.bfloat16
    L = cases.vq_layer(1003, 14336, 4096, 65536, bits=16, act=act, m=1, bias=True, std=0.02)
    ws = torch.zeros(64 * 14336, device=gpu, dtype=torch.float32)
    y, sl = _run(gpu, L, act, workspace=ws)
    assert sl.n_workgroups <= 2 * torch.cuda.get_device_properties(gpu).multi_processor_count
    assert sl.n_partials < 256  # one kernel: every lane adds its partial sum with one atomic
    _check(y, _vq_ref(oracle_lib, L, act))
    cb = L["cb"].to(act).to(gpu)
    y_fused = kernels.vq_linear(L["x"].to(gpu), L["packed"].to(gpu), cb, 16, 8, L["bias"].to(gpu), 14336)
    assert (y.float() - y_fused.float()).abs().max().item() <= 2 ** -6  # one bf16 ulp at |y| < 4
    for _ in range(3):
        assert not ws.any()  # handed back zero-filled
        again = kernels.vq_linear_sliced(L["x"].to(gpu), sl, cb, L["bias"].to(gpu), workspace=ws)
        assert torch.equal(again, y)


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 3])
def test_sliced_gemv_partial_sums_outside_the_fixed_point_range(gpu, oracle_lib, act, m):
    """Partial sums of magnitude 2^15 or more, infinities and NaNs bypass the fixed-point word
    (float accumulator): large finite results, an overflowing row, a NaN row, and the rows
    around them come out as the oracle's; the workspace is zero-filled afterwards."""
    from neuropress_amd import kernels

    n, k, nc = 96, 256, 9000
    L = cases.vq_layer(31 + m, n, k, nc, act=act, m=m, bias=True, std=0.05)
    cb = L["cb"].clone()
    x = L["x"].clone()
    cb *= 20.0  # entries ~ N(0, 1)
    x[:, :8] = 1.0e4  # group 0 of every row contributes 1e4 * (sum of eight entries) ~ N(0, 2.8e4)
    L["cb"], L["x"] = cb, x
    ws = torch.zeros(64 * n * m, device=gpu, dtype=torch.float32)
    sl = kernels.vq_slice_indices(L["packed"], L["bits"], n, k, 8, nc, device=gpu)
    y = kernels.vq_linear_sliced(x.to(gpu), sl, cb.to(act).to(gpu), L["bias"].to(gpu), workspace=ws)
    assert not ws.any()
    code = orc.torch_dtype_code(act)
    w = oracle_lib.vq_decode(L["packed"].numpy(), L["bits"], orc.to_bits(cb), n, k, code)
    ref = oracle_lib.linear_f64(orc.to_bits(x), code, w, code, orc.to_bits(L["bias"]), code)
    got = y.float().cpu().numpy().astype(np.float64)
    lim = float(torch.finfo(act).max)
    finite = np.abs(ref) < lim
    assert np.abs(ref[finite]).max() > 2.0**15  # the case does leave the fixed-point range
    assert np.all(np.abs(got[finite] - ref[finite]) <= 1e-2 + 1e-2 * np.abs(ref[finite]))
    assert np.all(np.isinf(got[~finite]) & (np.sign(got[~finite]) == np.sign(ref[~finite])))
    # NaN and infinity in the activations: the rows they reach are NaN / inf, as torch's would be.
    x2 = L["x"].clone()
    x2[0, 8] = float("nan")
    y2 = kernels.vq_linear_sliced(x2.to(gpu), sl, cb.to(act).to(gpu), None, workspace=ws)
    assert torch.isnan(y2[0]).any()
    assert not ws.any()


def test_sliced_gemv_two_kernel_finish(gpu, oracle_lib):
    """A codebook of 2^20 rows has 256 slices: a row has more partial sums than the fused finish
    counts, so the partial sums are written out and added by a second kernel."""
    from neuropress_amd import kernels

    n, k, nc, act = 40, 64, 1 << 20, torch.float16
    L = cases.vq_layer(77, n, k, nc, bits=20, act=act, m=2, bias=True, std=0.05)
    ws = torch.zeros(300 * n * 2 * 8, device=gpu, dtype=torch.float32)
    y, sl = _run(gpu, L, act, workspace=ws)
    assert sl.n_partials >= 256
    _check(y, _vq_ref(oracle_lib, L, act))
    assert not ws.any()
    again, _ = _run(gpu, L, act, workspace=ws)
    assert torch.equal(again, y)


def test_sliced_wrapper_errors(gpu):
    from neuropress_amd import kernels

    L = cases.vq_layer(6, 64, 64, 20000, act=torch.float16, m=1)
    sl = kernels.vq_slice_indices(L["packed"], L["bits"], 64, 64, 8, 20000, device=gpu)
    x, cb = L["x"].to(gpu), L["cb"].to(gpu)
    with pytest.raises(RuntimeError, match="x's dtype"):
        kernels.vq_linear_sliced(x.to(torch.bfloat16), sl, cb)
    with pytest.raises(RuntimeError, match="built for"):
        kernels.vq_linear_sliced(x[:, :32].contiguous(), sl, cb)
    with pytest.raises(RuntimeError, match="must be float16 or bfloat16"):
        kernels.vq_linear_sliced(x.float(), sl, cb.float())
    with pytest.raises(RuntimeError, match="workspace of"):
        kernels.vq_linear_sliced(x, sl, cb, workspace=torch.zeros(4, device=gpu))
    with pytest.raises(RuntimeError, match="VL = 8"):
        kernels.vq_slice_indices(L["packed"], L["bits"], 64, 64, 4, 20000, device=gpu)


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
def test_module_routes_decode_steps_through_the_slice_lists(gpu, oracle_lib, act, monkeypatch):
    """NPVQLinear: up to 7 tokens on a layer with a large codebook use the slice lists, more
    tokens the fused GEMV; both match the oracle; a HIP graph captured after
    prepare_sliced() replays to the same bits."""
    from neuropress_amd import kernels
    from neuropress_amd.nn import np_vq_linear as mod

    monkeypatch.setattr(mod, "_SLICED_MIN_INDICES", 1)
    n, k, nc = 384, 512, 20000
    L = cases.vq_layer(41, n, k, nc, act=act, m=9, bias=True, std=0.05)
    proxy = mod.VQProxy(L["cb"]).to(gpu)
    layer = mod.NPVQLinear(proxy, L["packed"], L["bits"], n, k, 8, "cuda_wmma", bias=L["bias"].float()).to(gpu)
    assert layer.prepare_sliced()  # forward never builds the lists itself
    calls = []
    real = kernels.vq_linear_sliced_checked
    monkeypatch.setattr(kernels, "vq_linear_sliced_checked", lambda *a, **kw: (calls.append(a[0].shape[0]), real(*a, **kw))[1])
    # a layer's later calls go through the plan its first call left behind
    real_run = kernels.SlicedCallPlan.run

    def run(plan, xx):
        yy = real_run(plan, xx)
        if yy is not None:
            calls.append(xx.numel() // k)
        return yy

    monkeypatch.setattr(kernels.SlicedCallPlan, "run", run)
    x = L["x"].to(gpu)
    ref = _vq_ref(oracle_lib, L, act)
    y1 = layer(x[:1])
    y2 = layer(x[:2].reshape(1, 2, k))
    y7 = layer(x[:7])
    y9 = layer(x)
    assert calls == [1, 2, 7] and y2.shape == (1, 2, n)
    _check(y1, ref[:1])
    _check(y2.reshape(2, n), ref[:2])
    _check(y7, ref[:7])
    _check(y9, ref)
    # Graph capture: no host work may happen inside; the lists already exist.
    static_x = x[:1].clone()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        layer(static_x)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            static_y = layer(static_x)
    for i in range(3):
        static_x.copy_(x[i : i + 1])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, layer(x[i : i + 1]))


def test_forward_never_builds_slice_lists(gpu, monkeypatch, caplog):
    """An eligible layer that was not prepared runs the fused GEMV -- eagerly and when its very
    first call is inside a graph capture -- without any host work (no build, no device-to-host
    copy), and says so once; after prepare_sliced() the same calls take the slice lists."""
    import logging

    from neuropress_amd import kernels
    from neuropress_amd.nn import np_vq_linear as mod

    monkeypatch.setattr(mod, "_SLICED_MIN_INDICES", 1)
    monkeypatch.setattr(mod, "_unprepared_warned", False)
    monkeypatch.setattr(mod, "_PREPARE_ON_MOVE", False)  # as for a layer built from tensors already on the GPU
    L = cases.vq_layer(42, 128, 256, 20000, bits=15, act=torch.float16, m=1, bias=True, std=0.05)  # 15 bits: widened stream
    proxy = mod.VQProxy(L["cb"]).to(gpu)
    layer = mod.NPVQLinear(proxy, L["packed"], L["bits"], 128, 256, 8, "cuda_wmma", bias=L["bias"].float()).to(gpu)
    x = L["x"].to(gpu)

    def no_build(*a, **kw):
        raise AssertionError("forward() must not build slice lists")

    monkeypatch.setattr(kernels, "vq_slice_indices", no_build)
    caplog.set_level(logging.WARNING, logger=mod.__name__)
    # First call of the module inside the capture: nothing it derives may be cached from there.
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            y = layer(x)
    assert layer._derived_hit("sliced", layer.packed_indices) is None
    assert not any(isinstance(v, tuple) for v in layer._derived.values())  # no tensor made inside the capture was kept
    eager_before_replay = layer(x)  # must not read tensors that only exist inside the graph
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, eager_before_replay)
    layer(x)
    assert sum("prepare_decode" in r.getMessage() for r in caplog.records) == 1
    monkeypatch.undo()
    monkeypatch.setattr(mod, "_SLICED_MIN_INDICES", 1)
    assert layer.prepare_sliced()
    seen = []
    real = kernels.vq_linear_sliced_checked
    monkeypatch.setattr(kernels, "vq_linear_sliced_checked", lambda *a, **kw: (seen.append(1), real(*a, **kw))[1])
    y2 = layer(x)
    assert seen == [1]
    assert (y2.float() - y.float()).abs().max().item() < 1e-2


@pytest.mark.parametrize("m", [1, 16, 64])
def test_reloaded_buffers_invalidate_everything_derived_from_them(gpu, oracle_lib, monkeypatch, m):
    """load_state_dict (an in-place copy into packed_indices and bias) after a first forward: the
    slice lists, the widened stream and the fp32 bias made from the old buffers must not be
    used again -- every band has to compute with the new indices and bias."""
    from neuropress_amd.nn import np_vq_linear as mod

    monkeypatch.setattr(mod, "_SLICED_MIN_INDICES", 1)
    monkeypatch.setattr(mod, "_PREPARE_ON_MOVE", False)  # the reload leaves the layer unprepared: fused paths first
    act = torch.float16
    n, k, nc = 192, 512, 20000
    A = cases.vq_layer(71, n, k, nc, bits=15, act=act, m=m, bias=True, std=0.05)
    B = cases.vq_layer(72, n, k, nc, bits=15, act=act, m=m, bias=True, std=0.05)
    layer = mod.NPVQLinear(mod.VQProxy(A["cb"]).to(gpu), A["packed"], 15, n, k, 8, "cuda_wmma",
                           bias=A["bias"].float()).to(gpu)
    layer.prepare_sliced()
    x = A["x"].to(gpu)
    _check(layer(x), _vq_ref(oracle_lib, A, act))
    state = {"packed_indices": B["packed"], "bias": B["bias"].float()}
    layer.load_state_dict(state, strict=False)
    Bx = dict(B, x=A["x"], cb=A["cb"])
    _check(layer(x), _vq_ref(oracle_lib, Bx, act))  # unprepared: the fused paths, new buffers
    layer.prepare_sliced()
    _check(layer(x), _vq_ref(oracle_lib, Bx, act))  # and through the rebuilt lists at m <= 7


@pytest.mark.parametrize("m", [1, 12])
def test_column_permutation_with_indices_wider_than_16_bits(gpu, oracle_lib, m):
    """A codebook of 70000 rows has 17-bit indices, which the fused GEMV with the permutation
    folded in does not stream: the layer must permute with torch and take decode + GEMM, not fail."""
    from neuropress_amd.nn import np_vq_linear as mod

    act = torch.float16
    n, k, nc = 64, 256, 70000
    L = cases.vq_layer(81, n, k, nc, act=act, m=m, bias=True, std=0.05)
    assert L["bits"] == 17
    perm = torch.randperm(k, generator=cases.gen(82))
    layer = mod.NPVQLinear(mod.VQProxy(L["cb"]).to(gpu), L["packed"], 17, n, k, 8, "cuda_wmma",
                           bias=L["bias"].float(), column_perm=perm).to(gpu)
    y = layer(L["x"].to(gpu))
    _check(y, _vq_ref(oracle_lib, dict(L, x=L["x"][:, perm].contiguous()), act))


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 3, 6, 10])
def test_column_permutation_is_applied_inside_the_sliced_kernel(gpu, oracle_lib, act, m, monkeypatch):
    """x[..., column_perm] (reference: np_vq_linear.py:1027-1028): the slice-list GEMV reads the
    permuted columns itself (m <= 7); larger m permutes with torch first.  Both must equal the
    oracle fed with the permuted activations."""
    from neuropress_amd import kernels
    from neuropress_amd.nn import np_vq_linear as mod

    monkeypatch.setattr(mod, "_SLICED_MIN_INDICES", 1)
    n, k, nc = 200, 384, 20000
    L = cases.vq_layer(51, n, k, nc, act=act, m=m, bias=True, std=0.05)
    perm = torch.randperm(k, generator=cases.gen(52))
    layer = mod.NPVQLinear(mod.VQProxy(L["cb"]).to(gpu), L["packed"], L["bits"], n, k, 8, "cuda_wmma",
                           bias=L["bias"].float(), column_perm=perm).to(gpu)
    assert layer.prepare_sliced()
    seen = []
    real = kernels.vq_linear_sliced_checked
    monkeypatch.setattr(kernels, "vq_linear_sliced_checked",
                        lambda *a, **kw: (seen.append(a[4] is not None), real(*a, **kw))[1])
    y = layer(L["x"].to(gpu))
    assert seen == ([True] if m <= 7 else [])
    Lp = dict(L, x=L["x"][:, perm].contiguous())
    _check(y, _vq_ref(oracle_lib, Lp, act))


def test_prepare_decode_builds_the_lists_of_every_eligible_layer(gpu, monkeypatch):
    import neuropress_amd
    from neuropress_amd.nn import np_vq_linear as mod

    monkeypatch.setattr(mod, "_SLICED_MIN_INDICES", 1)
    big = cases.vq_layer(61, 128, 256, 20000, act=torch.float16)
    small = cases.vq_layer(62, 128, 256, 256, act=torch.float16)  # 256-row codebook: stays on the fused GEMV
    model = torch.nn.Sequential(
        mod.NPVQLinear(mod.VQProxy(big["cb"]), big["packed"], big["bits"], 128, 256, 8, "cuda_wmma"),
        mod.NPVQLinear(mod.VQProxy(small["cb"]), small["packed"], small["bits"], 128, 256, 8, "cuda_wmma"),
    )
    assert neuropress_amd.prepare_decode(model) == 0  # still on the CPU
    model.to(gpu)
    assert neuropress_amd.prepare_decode(model) == 1
    assert model[0]._derived_hit("sliced", model[0].packed_indices) is not None
    assert "sliced" not in model[1]._derived
