"""Every entry point inside a HIP graph: replays (with eager work and synchronisation between
them) must reproduce the eager result bit for bit.  The library launches plain kernels only
(no allocation, no memset, no synchronisation), which is what makes the calls capturable."""

import pytest
import torch

from tests import cases

pytestmark = pytest.mark.gpu


def _capture_and_replay(gpu, fn, make_inputs, n_replays=3):
    """fn(inputs) -> tensor.  Captures fn on static inputs, then for each replay copies fresh
    inputs in, replays, and compares with fn run eagerly on the same inputs."""
    static = make_inputs(0)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        fn(static)  # warm up outside the capture (lazy module state, LDS attribute calls)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            out = fn(static)
    for i in range(1, n_replays + 1):
        fresh = make_inputs(i)
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        eager = fn(fresh)
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i} differs from the eager call"
        _ = torch.randn(1024, device=gpu).sum().item()  # unrelated eager work between replays


@pytest.mark.parametrize("m,tile", [(1, False), (16, False), (40, True)])
def test_vq_fused_kernels_in_a_graph(gpu, m, tile):
    from neuropress_amd import kernels

    L = cases.vq_layer(11, 200, 512, 65536, bits=16, act=torch.bfloat16, m=m, bias=True, std=0.05)
    packed, cb, bias = L["packed"].to(gpu), L["cb"].to(torch.bfloat16).to(gpu), L["bias"].to(gpu)
    mk = lambda i: [torch.randn(m, 512, generator=cases.gen(100 + i)).to(torch.bfloat16).to(gpu)]
    if tile:
        fn = lambda inp: kernels.vq_gemm_tile(inp[0], packed, cb, 16, 200, bias)
    else:
        fn = lambda inp: kernels.vq_linear(inp[0], packed, cb, 16, 8, bias, 200)
    _capture_and_replay(gpu, fn, mk)


def test_vq_dequant_and_widen_in_a_graph(gpu):
    from neuropress_amd import kernels
    from neuropress_amd.transforms.vq_packing import IndexPacking

    cb = (torch.randn(1024, 8, generator=cases.gen(3)) * 0.05).to(torch.float16).to(gpu)

    def mk(i):
        idx = torch.randint(0, 1024, (64 * 32,), generator=cases.gen(200 + i))
        return [IndexPacking.pack(idx, 10).to(gpu)]

    _capture_and_replay(gpu, lambda inp: kernels.vq_dequant(inp[0], cb, 10, 64, 256, torch.bfloat16), mk)
    _capture_and_replay(gpu, lambda inp: kernels.widen_indices_u16(inp[0], 64 * 32, 10), mk)


@pytest.mark.parametrize("m", [1, 3])
def test_sliced_gemv_in_a_graph(gpu, m):
    from neuropress_amd import kernels

    L = cases.vq_layer(12, 300, 256, 20000, act=torch.float16, m=m, std=0.05)
    sl = kernels.vq_slice_indices(L["packed"], L["bits"], 300, 256, 8, 20000, device=gpu)
    cb = L["cb"].to(gpu)
    ws = torch.zeros(sl.workspace_bytes(m) // 4, device=gpu, dtype=torch.float32)
    mk = lambda i: [torch.randn(m, 256, generator=cases.gen(300 + i)).to(torch.float16).to(gpu)]
    _capture_and_replay(gpu, lambda inp: kernels.vq_linear_sliced(inp[0], sl, cb, None, workspace=ws), mk)


@pytest.mark.parametrize("m", [1, 4, 40])
def test_rvq_in_a_graph(gpu, m):
    from neuropress_amd import kernels

    L = cases.rvq_layer(13, 80, 256, act=torch.float16, m=m)
    a = [L[k].to(gpu) for k in ("pm", "pr", "cbm", "cbr", "scale", "wbias")]
    mk = lambda i: [torch.randn(m, 256, generator=cases.gen(400 + i)).to(torch.float16).to(gpu)]
    fn = lambda inp: kernels.rvq_linear(inp[0], a[0], L["bm"], a[1], L["br"], a[2], a[3], a[4], a[5], 80, None)
    _capture_and_replay(gpu, fn, mk)


@pytest.mark.parametrize("act", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m", [1, 4, 40])
def test_q4_in_a_graph(gpu, act, m):
    """One fp16 token: the row-wise kernel; otherwise the MFMA GEMV (m <= 16) or the tile GEMM."""
    from neuropress_amd import kernels

    L = cases.q4_layer(14, 136, 512, gs=32, act=act, m=m, bias=True)
    blob, sc, bias = L["blob"].to(gpu), L["scale"].to(gpu), L["bias"].to(gpu)
    mk = lambda i: [torch.randn(m, 512, generator=cases.gen(500 + i)).to(act).to(gpu)]
    _capture_and_replay(gpu, lambda inp: kernels.q_linear(inp[0], blob, sc, 4, 32, None, bias), mk)


def test_q_dequant_in_a_graph(gpu):
    from neuropress_amd import kernels
    from neuropress_amd.t2n.packing import BitPacking4

    sc = (torch.rand(64 * 8, generator=cases.gen(5)) * 0.02).to(torch.float16).to(gpu)
    mk = lambda i: [BitPacking4.compress(
        torch.randint(0, 16, (64, 256), generator=cases.gen(600 + i), dtype=torch.int64).to(torch.uint8)).to(gpu)]
    _capture_and_replay(gpu, lambda inp: kernels.q_dequant(inp[0], sc, 4, 32, None, torch.float16), mk)


def test_split_k_tile_gemm_and_permuted_gemv_in_a_graph(gpu):
    """The tile GEMM with a workspace (K split over blockIdx.z plus its reduction kernel) and the GEMV
    that gathers x[..., column_perm] itself."""
    from neuropress_amd import kernels

    L = cases.vq_layer(14, 128, 4096, 4096, bits=12, act=torch.float16, m=24, bias=True, std=0.02)
    packed, cb, bias = L["packed"].to(gpu), L["cb"].to(gpu), L["bias"].to(gpu)
    mk = lambda i: [torch.randn(24, 4096, generator=cases.gen(500 + i)).half().to(gpu)]
    _capture_and_replay(gpu, lambda inp: kernels.vq_gemm_tile(inp[0], packed, cb, 12, 128, bias), mk)
    perm = torch.randperm(4096, generator=cases.gen(1)).to(torch.int32).to(gpu)
    mk2 = lambda i: [torch.randn(2, 4096, generator=cases.gen(600 + i)).half().to(gpu)]
    _capture_and_replay(gpu, lambda inp: kernels.vq_linear(inp[0], packed, cb, 12, 8, bias, 128, column_perm=perm), mk2)


def test_rms_norm_and_embedding_lookups_in_a_graph(gpu):
    from neuropress_amd import kernels
    from neuropress_amd.t2n.packing import BitPacking4

    g = cases.gen(15)
    w = (torch.rand(512, generator=g) + 0.5).to(torch.bfloat16).to(gpu)
    mk = lambda i: [torch.randn(9, 512, generator=cases.gen(700 + i)).to(torch.bfloat16).to(gpu)]
    _capture_and_replay(gpu, lambda inp: kernels.rms_norm(inp[0], w, 1e-6), mk)
    cb = (torch.randn(4096, 8, generator=g) * 0.05).half().to(gpu)
    tab = torch.randint(0, 4096, (300, 64), generator=g).to(torch.int16).to(gpu)
    inv = torch.argsort(torch.randperm(512, generator=g)).to(torch.int32).to(gpu)
    mk_ids = lambda i: [torch.randint(0, 300, (4, 5), generator=cases.gen(800 + i)).to(gpu)]
    _capture_and_replay(gpu, lambda inp: kernels.vq_embedding(inp[0], tab, cb, 22.6, inv, torch.bfloat16), mk_ids)
    blob = BitPacking4.compress(torch.randint(0, 16, (300, 512), generator=g, dtype=torch.int64).to(torch.uint8)).to(gpu)
    sc = (torch.rand(300 * 16, generator=g) * 0.02 + 0.001).half().to(gpu)
    _capture_and_replay(gpu, lambda inp: kernels.q_embedding(inp[0], blob, sc, 4, 32, None, 7, 22.6, torch.float16), mk_ids)
