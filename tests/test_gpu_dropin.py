"""Drop-in behaviour of the lowered modules on the GPU, and the benchmark configurations at their
own shapes where the other files only had look-alikes.

* a model lowered on the CPU and moved with ``.to("cuda")`` (or reloaded with ``load_state_dict``)
  reaches the slice-list decode kernel with no further call;
* buffers created or moved under ``torch.inference_mode()`` (the reference quantises there,
  neuropress/methods/gptq.py:253) work in every band;
* the slice-list GEMV's shared workspace when the first call on a stream is inside a graph capture;
* config 1 (2048 x 640, 256-entry codebook, uint8 indices, fp16, seed 1001) at 1 and 16 tokens and
  config 3's down projection (4096 x 14336) through the slice-list kernel, both against the oracle;
* config 3's up/gate layer through the module at 1024 and 4096 tokens (band c), by properties.
"""

import numpy as np
import pytest
import torch

import neuropress_amd.nn.np_vq_linear as vqmod
from neuropress_amd.nn import NPLinear, NPVQLinear, VQProxy
from oracle import oracle as orc
from tests import cases

pytestmark = pytest.mark.gpu


def _check(y, ref):
    ok, max_abs, excess = cases.within_tol(y.float().cpu().numpy(), ref)
    assert ok, f"max abs err {max_abs:.3e}, {excess:.2f}x the 1e-2 bound"


def _vq_ref(oracle_lib, L, act, x=None):
    code = orc.torch_dtype_code(act)
    w = oracle_lib.vq_decode(L["packed"].numpy(), L["bits"], orc.to_bits(L["cb"]), L["n"], L["k"], code)
    bias = None if L["bias"] is None else orc.to_bits(L["bias"])
    return oracle_lib.linear_f64(orc.to_bits(L["x"] if x is None else x), code, w, code, bias, code)


class _Root(torch.nn.Module):
    """A lowered model in miniature: the layer first, its shared codebook on the root after it."""

    def __init__(self, layer, proxy):
        super().__init__()
        self.proj = layer
        self._vq_proxy_0 = proxy

    def forward(self, x):
        return self.proj(x)


def _spy(monkeypatch, names):
    from neuropress_amd import kernels

    calls = []
    for name in names:
        real = getattr(kernels, name)
        monkeypatch.setattr(kernels, name, lambda *a, _r=real, _n=name, **kw: (calls.append(_n), _r(*a, **kw))[1])
    return calls


def test_a_model_lowered_on_the_cpu_and_moved_reaches_the_slice_list_kernel(gpu, oracle_lib, monkeypatch):
    """lower (CPU) -> .to("cuda") -> forward(one token): the slice lists are built by the move, not by
    forward and not by an API the reference lacks; load_state_dict() into the moved module rebuilds
    them for the new indices."""
    monkeypatch.setattr(vqmod, "_SLICED_MIN_INDICES", 1)
    act = torch.bfloat16
    L = cases.vq_layer(31, 256, 512, 20000, bits=15, act=act, m=1, bias=True, std=0.05)
    proxy = VQProxy(L["cb"])
    layer = NPVQLinear(proxy, L["packed"], L["bits"], 256, 512, 8, "cuda_wmma", bias=L["bias"].float())
    model = _Root(layer, proxy)
    assert layer._derived_hit("sliced", layer.packed_indices) is None  # nothing on the CPU
    calls = _spy(monkeypatch, ("vq_slice_indices",))
    model.to(gpu)  # the layer moves before its codebook
    assert calls == ["vq_slice_indices"]
    assert layer._derived_hit("sliced", layer.packed_indices) is not None
    model.to(gpu)  # nothing moves: nothing is rebuilt
    assert calls == ["vq_slice_indices"]
    assert layer._derived_hit("sliced", layer.packed_indices) is not None
    calls = _spy(monkeypatch, ("vq_linear_sliced_checked", "vq_linear", "vq_slice_indices"))
    y = model(L["x"].to(gpu))
    assert calls == ["vq_linear_sliced_checked"]
    _check(y, _vq_ref(oracle_lib, L, act))
    # new indices through load_state_dict: the old lists are stale, new ones are made by the load
    L2 = cases.vq_layer(32, 256, 512, 20000, bits=15, act=act, m=1, bias=True, std=0.05)
    state = {k: v.clone() for k, v in model.state_dict().items()}
    state["proj.packed_indices"] = L2["packed"].to(gpu)
    state["_vq_proxy_0.centroids"] = L2["cb"].to(gpu)
    state["proj.bias"] = L2["bias"].float().to(gpu)
    calls.clear()
    model.load_state_dict(state)
    assert calls == ["vq_slice_indices"]
    calls.clear()
    y2 = model(L2["x"].to(gpu))
    assert calls == ["vq_linear_sliced_checked"]
    _check(y2, _vq_ref(oracle_lib, L2, act))


def test_modules_built_and_moved_under_inference_mode(gpu, oracle_lib, monkeypatch):
    """Inference tensors keep no version counter: the caches of derived tensors must not ask for one."""
    monkeypatch.setattr(vqmod, "_SLICED_MIN_INDICES", 1)
    act = torch.float16
    L = cases.vq_layer(33, 256, 512, 20000, bits=15, act=act, m=40, bias=True, std=0.05)
    Q = cases.q4_layer(34, 128, 256, act=act, m=40, bias=True)
    with torch.inference_mode():
        proxy = VQProxy(L["cb"].clone())
        vq = NPVQLinear(proxy, L["packed"].clone(), L["bits"], 256, 512, 8, "cuda_wmma",
                        bias=L["bias"].float().clone()).to(gpu)
        proxy.to(gpu)  # the layer's lists are made when its codebook arrives
        assert vq._derived_hit("sliced", vq.packed_indices) is not None
        ql = NPLinear(Q["blob"].clone(), Q["scale"].clone(), 128, 256, 32, 4, "sym", "cuda",
                      bias=Q["bias"].float().clone()).to(gpu)
        vq.prepare()
        for m in (1, 12, 40):  # slice-list GEMV, fused GEMV, tile GEMM / decode + GEMM
            _check(vq(L["x"][:m].to(gpu)), _vq_ref(oracle_lib, L, act, x=L["x"][:m]))
        code = orc.DT_F16
        wq = oracle_lib.q_decode(Q["blob"].numpy(), orc.to_bits(Q["scale"]), None, 4, 32, code)
        for m in (1, 40):
            ref = oracle_lib.linear_f64(orc.to_bits(Q["x"][:m]), code, wq, code, orc.to_bits(Q["bias"]), code)
            _check(ql(Q["x"][:m].to(gpu)), ref)
    # and called outside inference mode afterwards
    _check(vq(L["x"][:1].to(gpu)), _vq_ref(oracle_lib, L, act, x=L["x"][:1]))


def test_sliced_workspace_made_inside_a_capture_is_not_kept(gpu):
    """First slice-list call on a fresh stream inside a graph capture, then an eager call on that
    stream before the first replay: the eager call must not get the capture's buffer, whose
    zero-fill has not run yet."""
    from neuropress_amd import kernels

    L = cases.vq_layer(12, 300, 256, 20000, act=torch.float16, m=1, std=0.05)
    sl = kernels.vq_slice_indices(L["packed"], L["bits"], 300, 256, 8, 20000, device=gpu)
    cb, x = L["cb"].to(gpu), L["x"].to(gpu)
    expect = kernels.vq_linear_sliced(x, sl, cb, None)
    s = torch.cuda.Stream()
    key = (gpu.index if gpu.index is not None else torch.cuda.current_device(), s.cuda_stream)
    with torch.cuda.stream(s):
        torch.cuda.synchronize()
        assert key not in kernels._SLICED_WORKSPACES
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            y_graph = kernels.vq_linear_sliced(x, sl, cb, None)
        assert key not in kernels._SLICED_WORKSPACES  # the capture's buffer was not cached
        y_eager = kernels.vq_linear_sliced(x, sl, cb, None)  # before the first replay
        torch.cuda.synchronize()
        assert torch.equal(y_eager, expect)
        for _ in range(3):
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_graph, expect)
            assert torch.equal(kernels.vq_linear_sliced(x, sl, cb, None), expect)  # eager work between the replays


@pytest.mark.parametrize("m", [1, 16])
def test_cfg1_at_its_own_shape_against_the_oracle(gpu, oracle_lib, m):
    """Config 1: 2048 x 640, one 256-entry fp16 codebook ~N(0, 0.02), uint8 indices [2048, 80], fp16
    activations, no bias, seed 1001.  K = 640 is two and a half of the GEMV's 256-k steps and 2048
    rows take the plan that trades rows of the MFMA tile for parts of k."""
    from neuropress_amd import kernels

    L = cases.vq_layer(1001, 2048, 640, 256, bits=8, act=torch.float16, m=m, bias=False, std=0.02)
    assert L["packed"].numel() == 2048 * 80  # one byte per index
    pk, cb = L["packed"].to(gpu), L["cb"].to(gpu)
    code = orc.DT_F16
    w_ref = oracle_lib.vq_decode(L["packed"].numpy(), 8, orc.to_bits(L["cb"]), 2048, 640, code)
    assert np.array_equal(orc.to_bits(kernels.vq_dequant(pk, cb, 8, 2048, 640, torch.float16)), w_ref)
    ref = oracle_lib.linear_f64(orc.to_bits(L["x"]), code, w_ref, code, None, code)
    _check(kernels.vq_linear(L["x"].to(gpu), pk, cb, 8, 8, None, 2048), ref)
    layer = NPVQLinear(VQProxy(L["cb"]).to(gpu), L["packed"], 8, 2048, 640, 8, "auto").to(gpu)
    _check(layer(L["x"].to(gpu)), ref)


@pytest.mark.parametrize("m", [1, 2])
def test_cfg3_down_projection_through_the_slice_lists_against_the_oracle(gpu, oracle_lib, m):
    """Config 3's down projection, 4096 x 14336 (1792 groups: several group ranges per slice), bf16."""
    from neuropress_amd import kernels

    act = torch.bfloat16
    L = cases.vq_layer(1003, 4096, 14336, 65536, bits=16, act=act, m=m, bias=True, std=0.02)
    sl = kernels.vq_slice_indices(L["packed"], 16, 4096, 14336, 8, 65536, device=gpu)
    assert sl.n_partials > sl.n_slices  # more than one group range per slice
    cb = L["cb"].to(act).to(gpu)
    y = kernels.vq_linear_sliced(L["x"].to(gpu), sl, cb, L["bias"].to(gpu))
    _check(y, _vq_ref(oracle_lib, L, act))
    assert torch.equal(y, kernels.vq_linear_sliced(L["x"].to(gpu), sl, cb, L["bias"].to(gpu)))


def test_sliced_gemv_outputs_of_small_magnitude(gpu, oracle_lib):
    """Weights of standard deviation 1e-4: every partial sum is rounded to 2^-24 before it is added, so
    the absolute error is bounded by (partial sums per row) x 2^-25 -- here 16 x 2^-25 = 4.8e-7 --
    whatever the output's magnitude; outputs of magnitude 1e-3 keep three digits."""
    from neuropress_amd import kernels

    act = torch.float16
    L = cases.vq_layer(77, 512, 2048, 65536, bits=16, act=act, m=2, bias=False, std=1e-4)
    sl = kernels.vq_slice_indices(L["packed"], 16, 512, 2048, 8, 65536, device=gpu)
    y = kernels.vq_linear_sliced(L["x"].to(gpu), sl, L["cb"].to(gpu), None).float().cpu().numpy()
    ref = _vq_ref(oracle_lib, L, act)
    bound = sl.n_partials * 2.0 ** -25 + np.abs(ref) * 2.0 ** -10  # fixed-point roundings + the fp16 store
    assert np.all(np.abs(y - ref) <= bound), float(np.max(np.abs(y - ref) / bound))


@pytest.mark.parametrize("m", [1024, 4096])
def test_cfg3_through_the_module_in_band_c(gpu, m, monkeypatch):
    """Config 3's up/gate layer at 1024 and 4096 tokens through NPVQLinear: decode + dense GEMM.
    Properties: equals the dense product of the decoded weight, rows of the batch are independent
    of the batch they are in, an all-zero codebook returns exactly the bias."""
    g = cases.gen(1003)
    n, k = 14336, 4096
    cb = (torch.randn(65536, 8, generator=g) * 0.02).half()
    packed = torch.randint(0, 65536, (n * k // 8,), generator=g, dtype=torch.int32).to(torch.int16).view(torch.uint8)
    bias = torch.randn(n, generator=cases.gen(9))
    layer = NPVQLinear(VQProxy(cb).to(gpu), packed.to(gpu), 16, n, k, 8, "cuda_wmma", bias=bias.to(gpu))
    calls = _spy(monkeypatch, ("vq_dequant", "vq_gemm_tile", "vq_linear"))
    x = torch.randn(m, k, generator=cases.gen(m)).bfloat16().to(gpu)
    y = layer(x)
    assert calls == ["vq_dequant"]
    from neuropress_amd import kernels

    w = kernels.vq_dequant(layer.packed_indices, layer.proxy.centroids, 16, n, k, torch.bfloat16)
    # the band is the reference's own: the dense product of the decoded weight with the bias in the
    # activation dtype (neuropress/nn/np_vq_linear.py:1148), so the same call gives the same bits
    assert torch.equal(y, torch.nn.functional.linear(x, w, bias.to(gpu).bfloat16()))
    xw = x.float() @ w.float().T
    ref = xw + bias.to(gpu)
    # bf16 roundings of the product, of the bias and of their sum: relative to the terms, not to a sum that cancels
    err = (y.float() - ref).abs()
    assert bool((err <= 1e-2 + 1e-2 * (xw.abs() + bias.to(gpu).abs())).all()), float(err.max())
    part = layer(x[100:612])  # 512 rows: still band c, another GEMM tiling: a few output ulps (2^-8 relative each)
    diff = (part.float() - y[100:612].float()).abs()
    assert bool((diff <= 2.0 ** -6 * (1 + xw[100:612].abs() + bias.to(gpu).abs())).all()), float(diff.max())
    zero = NPVQLinear(VQProxy(torch.zeros_like(cb)).to(gpu), layer.packed_indices, 16, n, k, 8, "cuda_wmma", bias=bias.to(gpu))
    assert torch.equal(zero(x), bias.to(gpu).bfloat16().expand(m, n))


def test_the_staging_predicate_names_the_kernel_the_launcher_takes(gpu):
    """npamd_gemv_stages_activations decides how far the modules keep the fused GEMV ahead of the tile
    GEMM; it restates the launcher's choice, so every shape class is launched once and asked about."""
    from neuropress_amd import _lib, kernels

    lib = _lib.load()
    g = cases.gen(3)
    seen = set()
    for nc, bits in ((256, 8), (4096, 12), (65536, 16)):
        cb = (torch.randn(nc, 8, generator=g) * 0.05).half().to(gpu)
        for n, k in ((256, 512), (512, 4096), (1024, 1024), (2048, 640), (2048, 8192), (6144, 4096), (14336, 4096), (4096, 14336)):
            L = cases.vq_layer(n + k, n, k, nc, bits=bits, act=torch.float16, m=1, std=0.05)
            pk = L["packed"].to(gpu)
            for m in (1, 2, 7, 8, 9, 16, 17, 24, 32):
                x = torch.randn(m, k, generator=g).half().to(gpu)
                kernels.vq_linear(x, pk, cb, bits, 8, None, n)
                launched = lib.npamd_diag_last_gemv_staged()
                said = lib.npamd_gemv_stages_activations(m, n, k, nc)
                assert launched in (0, 1)
                what = f"{n} x {k}, {nc}-row codebook, {m} tokens: said {said}, launched {launched}"
                assert said == launched, what
                seen.add(launched)
    Q = cases.q4_layer(5, 6144, 4096, act=torch.float16, m=32)
    blob, sc = Q["blob"].to(gpu), Q["scale"].to(gpu)
    for m in (2, 8, 16, 17, 32):  # one fp16 token takes the row-wise int4 kernel, not this launcher
        kernels.q_linear(Q["x"][:m].to(gpu), blob, sc, 4, 32, None, None)
        said, launched = lib.npamd_gemv_stages_activations(m, 6144, 4096, 0), lib.npamd_diag_last_gemv_staged()
        assert said == launched, (m, said, launched)
    assert seen == {0, 1}


def test_planned_decode_calls_follow_the_buffers(gpu, oracle_lib, monkeypatch):
    """A layer's second decode call reuses the arguments of its first.  Writing into a buffer,
    replacing one, or calling with another dtype, shape or stride must not reuse what no longer holds."""
    from neuropress_amd import kernels

    monkeypatch.setattr(vqmod, "_SLICED_MIN_INDICES", 1)
    act = torch.bfloat16
    n, k = 256, 512
    A = cases.vq_layer(41, n, k, 20000, bits=15, act=act, m=3, bias=True, std=0.05)
    B = cases.vq_layer(42, n, k, 20000, bits=15, act=act, m=3, bias=True, std=0.05)
    proxy = VQProxy(A["cb"]).to(gpu)
    layer = NPVQLinear(proxy, A["packed"], 15, n, k, 8, "cuda_wmma", bias=A["bias"].float()).to(gpu)
    planned = []
    real_run = kernels.SlicedCallPlan.run
    monkeypatch.setattr(kernels.SlicedCallPlan, "run",
                        lambda p, xx: (lambda yy: (planned.append(yy is not None), yy)[1])(real_run(p, xx)))
    x = A["x"].to(gpu)
    ref = _vq_ref(oracle_lib, A, act)
    _check(layer(x), ref)
    assert planned == []  # the first call makes the plan
    _check(layer(x), ref)
    _check(layer(x[:1]), ref[:1])
    _check(layer(x.reshape(1, 3, k)).reshape(3, n), ref)  # leading dimensions are kept
    wide = torch.zeros(3, 2 * k, dtype=act, device=gpu)
    wide[:, :k] = x
    _check(layer(wide[:, :k]), ref)  # a row stride that is not K
    assert planned == [True] * 4
    A16 = dict(A, x=A["x"].half(), bias=A["bias"].half())  # bf16 values are fp16 values at these magnitudes
    _check(layer(x.half()), _vq_ref(oracle_lib, A16, torch.float16))  # another dtype: its own first call
    planned.clear()
    # written in place: bias first, then the indices (the lists are stale: fused GEMV until they are rebuilt)
    layer.bias.copy_(B["bias"].float())
    _check(layer(x), _vq_ref(oracle_lib, dict(A, bias=B["bias"]), act))
    assert planned == []
    layer.packed_indices.copy_(B["packed"])
    Bx = dict(B, x=A["x"], cb=A["cb"])
    _check(layer(x), _vq_ref(oracle_lib, Bx, act))
    layer.prepare_sliced()
    _check(layer(x), _vq_ref(oracle_lib, Bx, act))
    _check(layer(x), _vq_ref(oracle_lib, Bx, act))
    assert planned == [True]
    # the codebook written in place, then replaced by moving the proxy
    proxy.centroids.copy_(B["cb"])
    Bb = dict(B, x=A["x"])
    _check(layer(x), _vq_ref(oracle_lib, Bb, act))
    _check(layer(x), _vq_ref(oracle_lib, Bb, act))
    proxy.to("cpu")
    proxy.centroids.copy_(A["cb"])
    proxy.to(gpu)
    _check(layer(x), _vq_ref(oracle_lib, Bx, act))
    # eight tokens are past the lists' band: the plan declines, the fused GEMV answers
    x8 = torch.randn(8, k, generator=cases.gen(8)).to(act)
    _check(layer(x8.to(gpu)), _vq_ref(oracle_lib, Bx, act, x=x8))
