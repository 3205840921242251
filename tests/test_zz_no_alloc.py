"""``npamd_vq_gemv_sliced_static``: the slice-list GEMV with the library's own device workspace.

The entry point allocates nothing; its results must equal ``npamd_vq_gemv_sliced``'s bit for
bit (same kernels, another workspace), on calls that follow each other and share the array.
"""

import ctypes

import pytest
import torch

from tests import cases

pytestmark = pytest.mark.gpu


def _both(gpu, L, act, m, perm=None):
    """y from npamd_vq_gemv_sliced (own workspace) and from npamd_vq_gemv_sliced_static."""
    from neuropress_amd import _lib, kernels

    sl = kernels.vq_slice_indices(L["packed"], L["bits"], L["n"], L["k"], 8, L["nc"], device=gpu)
    x = L["x"][:m].to(gpu).contiguous()
    cb = L["cb"].to(act).to(gpu)
    bias = L["bias"].float().to(gpu)
    ref = kernels.vq_linear_sliced(x, sl, cb, bias, workspace=torch.zeros(sl.workspace_bytes(m) // 4, device=gpu),
                                   column_perm=perm)
    y = torch.full((m, L["n"]), float("nan"), device=gpu, dtype=act)
    code = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}[act]
    _lib.call(
        "npamd_vq_gemv_sliced_static", x.data_ptr(), x.stride(0), None if perm is None else perm.data_ptr(),
        sl.header_ptr, sl.blob.data_ptr(), cb.data_ptr(), code, bias.data_ptr(), y.data_ptr(), L["n"], m, code,
        torch.cuda.current_stream(gpu).cuda_stream,
    )  # fmt: skip
    torch.cuda.synchronize(gpu)
    return y, ref


@pytest.mark.parametrize("act", [torch.bfloat16, torch.float16])
def test_static_workspace_equals_caller_workspace_on_consecutive_calls(gpu, act):
    big = cases.vq_layer(501, 1100, 512, 65536, bits=16, act=act, m=5, bias=True, std=0.05)
    small = cases.vq_layer(502, 200, 128, 20000, act=act, m=2, bias=True, std=0.05)
    for L, m in ((big, 5), (small, 2), (big, 1), (small, 1)):  # a smaller input right after a larger one
        y, ref = _both(gpu, L, act, m)
        assert torch.equal(y, ref)


def test_static_workspace_with_column_permutation(gpu):
    act = torch.float16
    L = cases.vq_layer(503, 300, 256, 9000, act=act, m=3, bias=True, std=0.05)
    perm = torch.randperm(256, generator=cases.gen(9)).to(torch.int32).to(gpu)
    y, ref = _both(gpu, L, act, 3, perm)
    assert torch.equal(y, ref)


def test_static_workspace_rejects_requests_beyond_its_size(gpu):
    """A layer whose workspace need exceeds the built-in array is refused before anything is launched."""
    from neuropress_amd import _lib, kernels

    act = torch.float16
    L = cases.vq_layer(504, 64, 64, 20000, act=act, m=1, bias=True)
    sl = kernels.vq_slice_indices(L["packed"], L["bits"], 64, 64, 8, 20000, device=gpu)
    # Same blob, header edited to claim a layer of 2^20 output rows: 32 tokens x 12 bytes x 2^20 rows > 4 MiB.
    hdr = bytearray(sl.header)
    hdr[8:12] = (1 << 20).to_bytes(4, "little")
    buf = ctypes.create_string_buffer(bytes(hdr), len(hdr))
    x, cb = L["x"].to(gpu), L["cb"].to(gpu)
    y = torch.empty((1, 1 << 20), device=gpu, dtype=act)
    with pytest.raises(RuntimeError, match="the built-in one holds"):
        _lib.call("npamd_vq_gemv_sliced_static", x.data_ptr(), x.stride(0), None, ctypes.addressof(buf),
                  sl.blob.data_ptr(), cb.data_ptr(), _lib.F16, None, y.data_ptr(), 1 << 20, 1, _lib.F16,
                  torch.cuda.current_stream(gpu).cuda_stream)  # fmt: skip
