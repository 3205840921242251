"""Kernel wrappers: torch tensors in, HIP kernels through the C ABI, torch tensors out.

Mirrors the function surface of the reference's ``neuropress.kernels``
(neuropress/kernels/__init__.py): ``vq_linear`` (:209-216), ``vq_linear_wmma``
(:335-342), ``vq_dequant`` (:497-504), ``dequantize_vq_weight`` (:248-255),
``q_linear`` (:109-117), ``unpack_indices`` (:947), ``warn_kernel_fallback``
(:436-453) -- same names, argument order and error type (``RuntimeError``).
``vq_gemm_tile`` takes the place of the reference's Triton GEMM
(neuropress/kernels/vq_triton.py:119-179); ``q_dequant`` / ``q_gemm_tile`` and
the ``rvq_*`` functions have no reference counterpart.

Every function here launches on torch's current stream, allocates its output
with torch, and raises if the HIP library is missing: there is no CPU fallback
at this level (callers that want one catch ``RuntimeError`` and say so through
:func:`warn_kernel_fallback`).
"""

from __future__ import annotations

import logging

import torch

from .. import _lib

log = logging.getLogger(__name__)

_DT = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}


def _dt(dtype: torch.dtype, what: str) -> int:
    try:
        return _DT[dtype]
    except KeyError:
        raise RuntimeError(f"{what}: dtype must be bfloat16, float16 or float32, got {dtype}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """Handle of torch's current stream on ``t``'s device (the raw query costs a few tenths of a
    microsecond, ``torch.cuda.current_stream`` about four)."""
    if _raw_stream is not None:
        return _raw_stream(t.get_device())
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _check_device(what: str, *tensors: torch.Tensor | None) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(f"{what}: all tensors must be on the GPU (got a {t.device} tensor)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"{what}: tensors are on different devices ({dev} vs {t.device})")
    assert dev is not None
    return dev


def _packed_u8(packed: torch.Tensor, what: str) -> torch.Tensor:
    if packed.dtype != torch.uint8:
        raise RuntimeError(f"{what}: packed indices must be uint8, got {packed.dtype}")
    return packed.contiguous().reshape(-1)


def _centroids_f16(centroids: torch.Tensor, what: str) -> torch.Tensor:
    if centroids.dim() != 2:
        raise RuntimeError(f"{what}: centroids must be [NC, VL]")
    return centroids.contiguous()


def _bias_f32(bias: torch.Tensor | None) -> torch.Tensor | None:
    if bias is None:
        return None
    return bias.contiguous() if bias.dtype == torch.float32 else bias.to(torch.float32).contiguous()


def _x2d(x: torch.Tensor, what: str) -> torch.Tensor:
    if x.dim() != 2:
        raise RuntimeError(f"{what}: x must be 2-D [M, K]")
    if x.stride(1) != 1:
        x = x.contiguous()
    return x


def _tile_workspace(entry: str, m: int, n: int, k: int, device) -> tuple[int | None, int]:
    """Scratch for the tile GEMM's split-K (layers with few output features); (None, 0) for the
    other entry points and for shapes the library does not split.  Allocated per call from
    torch's caching allocator, so it is stream-ordered and capturable like the output."""
    if not entry.endswith("_gemm_tile"):
        return None, 0
    need = int(_lib.load().npamd_gemm_tile_workspace_bytes(int(m), int(n), int(k)))
    if need <= 0:
        return None, 0
    ws = torch.empty(need // 4, device=device, dtype=torch.float32)
    return ws, need


# ---------------------------------------------------------------------------
# VQ
# ---------------------------------------------------------------------------


def vq_dequant(
    packed_indices: torch.Tensor,
    centroids: torch.Tensor,
    bits: int,
    out_features: int,
    in_features: int,
    dtype: torch.dtype,
) -> torch.Tensor:
    """Decode a packed VQ weight to a dense ``[out_features, in_features]`` tensor.

    Same contract as the reference's ``vq_dequant`` (neuropress/kernels/__init__.py:497-529,
    neuropress/kernels/vq_dequant.cu:105-146); the result equals
    ``centroids[idx].reshape(N, K).to(dtype)`` bit for bit.
    """
    what = "vq_dequant"
    _check_device(what, packed_indices, centroids)
    packed = _packed_u8(packed_indices, what)
    cb = _centroids_f16(centroids, what)
    if cb.dtype != torch.float16:
        raise RuntimeError(f"{what}: centroids must be float16")
    vl = cb.shape[1]
    numel = out_features * in_features
    if numel % vl:
        raise RuntimeError(f"{what}: weight size not divisible by VL={vl}")
    out = torch.empty((out_features, in_features), device=packed.device, dtype=dtype)
    _lib.call(
        "npamd_vq_dequant", packed.data_ptr(), packed.numel(), int(bits), cb.data_ptr(),
        cb.shape[0], vl, numel // vl, out.data_ptr(), _dt(dtype, what), _stream(out),
    )  # fmt: skip
    return out


def dequantize_vq_weight(
    packed_indices: torch.Tensor,
    centroids: torch.Tensor,
    bits: int,
    vector_len: int,
    out_features: int,
    in_features: int,
) -> torch.Tensor:
    """fp16 decode (reference: neuropress/kernels/__init__.py:248-283); no tail padding needed."""
    if centroids.shape[1] != vector_len:
        raise RuntimeError("dequantize_vq_weight: vector_len does not match the codebook")
    return vq_dequant(packed_indices, centroids, bits, out_features, in_features, torch.float16)


def unpack_indices(packed: torch.Tensor, n_indices: int, bits: int) -> torch.Tensor:
    """Bit-stream -> int64 indices on the GPU (reference: neuropress/kernels/__init__.py:947)."""
    return widen_indices_u16(packed, n_indices, bits).view(torch.int16).to(torch.int64) & 0xFFFF


def widen_indices_u16(packed: torch.Tensor, n_indices: int, bits: int) -> torch.Tensor:
    """Bit-stream -> one uint16 per index, returned as a uint8 view (a 16-bit stream)."""
    what = "widen_indices_u16"
    _check_device(what, packed)
    p = _packed_u8(packed, what)
    out = torch.empty(2 * n_indices, device=p.device, dtype=torch.uint8)
    _lib.call("npamd_vq_widen_u16", p.data_ptr(), p.numel(), int(bits), int(n_indices),
              out.data_ptr(), _stream(out))  # fmt: skip
    return out


def _vq_fused(
    entry: str,
    x: torch.Tensor,
    packed_indices: torch.Tensor,
    centroids: torch.Tensor,
    bits: int,
    out_features: int | None,
    bias: torch.Tensor | None,
    column_perm: torch.Tensor | None = None,
) -> torch.Tensor:
    _check_device(entry, x, packed_indices, centroids, bias)
    x = _x2d(x, entry)
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"{entry}: x must be float16 or bfloat16, got {x.dtype}")
    packed = _packed_u8(packed_indices, entry)
    cb = _centroids_f16(centroids, entry)
    if cb.dtype not in (torch.float16, x.dtype):
        raise RuntimeError(f"{entry}: centroids must be float16 or x's dtype")
    m, k = x.shape
    vl = cb.shape[1]
    if k % vl:
        raise RuntimeError(f"{entry}: K={k} not divisible by VL={vl}")
    groups = k // vl
    if out_features is None:
        # N from the stream length, as the reference kernels do (vq_linear_wmma.cu:501-506).
        total = packed.numel() * 8 // bits
        if groups == 0 or total % groups:
            raise RuntimeError(f"{entry}: packed_indices size does not evenly divide into rows")
        out_features = total // groups
    y = torch.empty((m, out_features), device=x.device, dtype=x.dtype)
    b32 = _bias_f32(bias)
    ws, ws_bytes = _tile_workspace(entry, m, out_features, k, x.device)
    extra = (_ptr(ws), ws_bytes) if entry.endswith("_gemm_tile") else ()
    perm = ()
    if column_perm is not None:
        if column_perm.dtype != torch.int32 or column_perm.numel() != k or not column_perm.is_contiguous():
            raise RuntimeError(f"{entry}: column_perm must be a contiguous int32 tensor of K={k} entries")
        if column_perm.device != x.device:
            raise RuntimeError(f"{entry}: column_perm must live on x's device")
        perm = (column_perm.data_ptr(),)
    _lib.call(
        entry, x.data_ptr(), x.stride(0), *perm, packed.data_ptr(), packed.numel(), int(bits),
        cb.data_ptr(), _DT[cb.dtype], cb.shape[0], vl, _ptr(b32), y.data_ptr(), y.stride(0),
        m, out_features, k, _DT[x.dtype], *extra, _stream(x),
    )  # fmt: skip
    return y


def vq_linear(
    x: torch.Tensor,
    packed_indices: torch.Tensor,
    centroids: torch.Tensor,
    bits: int,
    vector_len: int,
    bias: torch.Tensor | None = None,
    out_features: int | None = None,
    column_perm: torch.Tensor | None = None,
) -> torch.Tensor:
    """Fused decode GEMV, ``M <= 32`` (reference: neuropress/kernels/__init__.py:209-245).

    ``column_perm`` (int32 ``[K]``, optional, not in the reference's signature): compute
    ``vq_linear(x[..., column_perm], ...)`` with the gather done inside the kernel; see
    :func:`vq_linear_perm_supported` for the shapes that take it.
    """
    if centroids.dim() == 2 and centroids.shape[1] != vector_len:
        raise RuntimeError("vq_linear: vector_len does not match the codebook")
    if column_perm is not None:
        return _vq_fused("npamd_vq_gemv_perm", x, packed_indices, centroids, bits, out_features, bias,
                         column_perm)  # fmt: skip
    return _vq_fused("npamd_vq_gemv", x, packed_indices, centroids, bits, out_features, bias)


def vq_linear_perm_supported(m: int, n: int, k: int, num_centroids: int, vector_len: int, bits: int) -> bool:
    """Whether :func:`vq_linear` should be given ``column_perm`` for this shape: the kernel takes it
    (``M <= 16``, ``M * K <= 16384``, VL 8 or 4, 4/8/12/16-bit indices, ``K % 64 == 0``) and its LDS copy of x
    does not reduce the workgroups per compute unit."""
    return bool(_lib.load().npamd_vq_gemv_perm_supported(int(m), int(n), int(k), int(num_centroids),
                                                         int(vector_len), int(bits)))  # fmt: skip


def gemv_stages_activations(m: int, n: int, k: int, num_centroids: int) -> bool:
    """Whether a fused GEMV call of *m* tokens on an ``n x k`` layer runs the kernel that stages its
    activations through LDS (``npamd_gemv_stages_activations``): then the GEMV stays ahead of the
    tile GEMM up to its 32 tokens at any ``k``.  *num_centroids*: rows of the layer's codebook of
    eight-element vectors, 0 for a group-quantized layer."""
    return bool(_lib.load().npamd_gemv_stages_activations(int(m), int(n), int(k), int(num_centroids)))


def vq_fused_supported(in_features: int, vector_len: int, bits: int) -> bool:
    """Whether the MFMA GEMV / tile GEMM take a VQ layer of this shape (``npamd_vq_fused_supported``).
    Other shapes run an element-wise kernel that decodes the weight once per 16 tokens."""
    return bool(_lib.load().npamd_vq_fused_supported(int(in_features), int(vector_len), int(bits)))


def q_fused_supported(in_features: int, nbits: int, group_size: int) -> bool:
    """The same question for group-quantized layers (``npamd_q_fused_supported``)."""
    return bool(_lib.load().npamd_q_fused_supported(int(in_features), int(nbits), int(group_size)))


class SlicedIndices:
    """Slice-list form of one layer's indices: the blob on the GPU plus a host copy of its header.

    Built by :func:`vq_slice_indices`, consumed by :func:`vq_linear_sliced`.
    """

    _FIELDS = ("magic", "version", "n", "k", "vl", "nc", "slice_rows", "n_slices", "n_workgroups",
               "n_partials", "groups_max", "flags", "n_quads", "n_entries", "off_workgroups",
               "off_rowmap", "off_entries", "total_bytes")  # fmt: skip

    def __init__(self, blob: torch.Tensor, header: bytes):
        import ctypes
        import struct

        if len(header) != _lib.SLICED_HEADER_BYTES:
            raise RuntimeError("SlicedIndices: header must be 128 bytes")
        self.blob = blob
        self.header = header
        self._header_buf = ctypes.create_string_buffer(header, len(header))
        values = struct.unpack("<2I9iI6q", header[:96])
        for name, value in zip(self._FIELDS, values):
            setattr(self, name, value)
        self.wave_quads = struct.unpack("<16H", header[96:128])
        self._workspace_bytes: dict[int, int] = {}  # per token count (asked on every call)

    @property
    def header_ptr(self) -> int:
        import ctypes

        return ctypes.addressof(self._header_buf)

    def workspace_bytes(self, m: int) -> int:
        need = self._workspace_bytes.get(m)
        if need is None:
            need = self._workspace_bytes[m] = int(_lib.load().npamd_vq_sliced_workspace_bytes(self.header_ptr, int(m)))
        return need

    def to(self, device) -> "SlicedIndices":
        return SlicedIndices(self.blob.to(device), self.header)


def vq_slice_indices(
    packed_indices: torch.Tensor,
    bits: int,
    out_features: int,
    in_features: int,
    vector_len: int,
    num_centroids: int,
    device: torch.device | str | None = None,
    target_workgroups: int = 0,
) -> SlicedIndices:
    """Re-lay a packed index stream into the slice-list form (host work, once per layer).

    The stream is copied to the host, filed by codebook slice there
    (``npamd_vq_sliced_build``), checked (``npamd_vq_sliced_check``) and uploaded to
    *device* (default: where *packed_indices* lives).  No reference counterpart.
    """
    import ctypes

    what = "vq_slice_indices"
    if packed_indices.dtype != torch.uint8:
        raise RuntimeError(f"{what}: packed indices must be uint8, got {packed_indices.dtype}")
    dev = torch.device(device) if device is not None else packed_indices.device
    host = packed_indices.detach().to("cpu").contiguous().reshape(-1)
    if target_workgroups <= 0 and dev.type == "cuda":
        target_workgroups = torch.cuda.get_device_properties(dev).multi_processor_count
    size = ctypes.c_int64(0)
    args = (host.data_ptr(), host.numel(), int(bits), int(out_features), int(in_features),
            int(vector_len), int(num_centroids), int(target_workgroups))  # fmt: skip
    # One build into a buffer sized for the usual case (3 bytes per index, a third of padding,
    # the tables); only if that is too small is the size asked for and the build repeated.
    n_idx = int(out_features) * (int(in_features) // max(int(vector_len), 1))
    blob = torch.empty(4 * n_idx + (2 << 20), dtype=torch.uint8)
    lib = _lib.load()
    rc = lib.npamd_vq_sliced_build(*args, blob.data_ptr(), blob.numel(), ctypes.byref(size))
    if rc != 0 and size.value > blob.numel():
        blob = torch.empty(size.value, dtype=torch.uint8)
        rc = lib.npamd_vq_sliced_build(*args, blob.data_ptr(), blob.numel(), ctypes.byref(size))
    if rc != 0:
        raise RuntimeError(f"npamd_vq_sliced_build failed (code {rc}): {lib.npamd_last_error().decode('utf-8', 'replace')}")
    blob = blob[: size.value]
    _lib.call("npamd_vq_sliced_check", blob.data_ptr(), blob.numel())
    header = bytes(blob[: _lib.SLICED_HEADER_BYTES].numpy().tobytes())
    return SlicedIndices(blob.to(dev), header)


_SLICED_WORKSPACES: dict = {}


def sliced_workspace(device: torch.device, nbytes: int, stream: int | None = None) -> torch.Tensor:
    """The zero-filled scratch of :func:`vq_linear_sliced` for the current stream of *device*.

    Every call hands its workspace back zero-filled, so one buffer per (device, stream) serves
    all layers whose calls follow each other on that stream.  Grown (and zero-filled again) on
    demand; allocate it before a graph capture starts, e.g. through ``NPVQLinear.prepare_sliced``.
    """
    if stream is None:
        stream = torch.cuda.current_stream(device).cuda_stream
    key = (device.index, stream)
    ws = _SLICED_WORKSPACES.get(key)
    if ws is None or ws.numel() * 4 < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 20) // 4 + 4, device=device, dtype=torch.float32)
        # A buffer made inside a graph capture lives in the graph's private pool and is zero-filled
        # only when the graph is replayed: it serves this capture and is not kept (an eager call, or
        # another capture on the same stream, before the first replay would start from garbage).
        if not torch.cuda.is_current_stream_capturing():
            _SLICED_WORKSPACES[key] = ws
    return ws


def drop_sliced_workspace(device: torch.device, stream: int) -> None:
    """Forget the cached workspace of (*device*, *stream*): after a failed call it may not be
    zero-filled any more, and the kernels count on that."""
    _SLICED_WORKSPACES.pop((device.index, stream), None)


def vq_linear_sliced(
    x: torch.Tensor,
    sliced: SlicedIndices,
    centroids: torch.Tensor,
    bias: torch.Tensor | None = None,
    workspace: torch.Tensor | None = None,
    column_perm: torch.Tensor | None = None,
) -> torch.Tensor:
    """Decode GEMV over the slice-list form, ``M <= 32`` (``npamd_vq_gemv_sliced``).

    *centroids* must already be in ``x.dtype`` (the modules cache that copy).
    *workspace*: optional float32 scratch of at least ``sliced.workspace_bytes(M) / 4``
    elements, zero-filled before its first use (every call leaves it zero-filled); by
    default the per-stream buffer of :func:`sliced_workspace`.
    *column_perm*: int32 ``[K]``; the kernel then computes with ``x[:, column_perm]``
    (the reference's input permutation, np_vq_linear.py:1027-1028) without materialising it.
    """
    what = "vq_linear_sliced"
    _check_device(what, x, sliced.blob, centroids, bias, workspace)
    x = _x2d(x, what)
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"{what}: x must be float16 or bfloat16, got {x.dtype}")
    cb = _centroids_f16(centroids, what)
    if cb.dtype != x.dtype:
        raise RuntimeError(f"{what}: centroids must be in x's dtype ({x.dtype}), got {cb.dtype}")
    m, k = x.shape
    if column_perm is not None:
        if column_perm.dtype != torch.int32 or column_perm.numel() != sliced.k or not column_perm.is_contiguous():
            raise RuntimeError(f"{what}: column_perm must be a contiguous int32 tensor of K={sliced.k} entries")
        _check_device(what, x, column_perm)
    if k != sliced.k or cb.shape[0] != sliced.nc or cb.shape[1] != sliced.vl:
        raise RuntimeError(f"{what}: slice lists were built for K={sliced.k}, codebook [{sliced.nc}, {sliced.vl}]")
    if workspace is not None and (workspace.dtype != torch.float32 or not workspace.is_contiguous()):
        raise RuntimeError(f"{what}: workspace must be a contiguous float32 tensor")
    return vq_linear_sliced_checked(x, sliced, cb, _bias_f32(bias), column_perm, workspace)


def vq_linear_sliced_checked(x, sliced, cb, bias_f32, column_perm, workspace=None) -> torch.Tensor:
    """:func:`vq_linear_sliced` without the argument checks, for callers that have made them
    (``NPVQLinear``, whose tensors come out of its own caches): *x* 2-D with unit inner stride,
    fp16 / bf16, *cb* in ``x.dtype``, *bias_f32* float32 or None, *column_perm* int32 or None, all
    on ``x``'s device.  The library still validates sizes and pointers."""
    m = x.shape[0]
    stream = _stream(x)
    own = workspace is None
    if own:
        workspace = sliced_workspace(x.device, sliced.workspace_bytes(max(m, 1)), stream)
    y = torch.empty((m, sliced.n), device=x.device, dtype=x.dtype)
    dt = _DT[x.dtype]
    try:
        _lib.call(
            "npamd_vq_gemv_sliced", x.data_ptr(), x.stride(0), _ptr(column_perm), sliced.header_ptr, sliced.blob.data_ptr(),
            cb.data_ptr(), dt, _ptr(bias_f32), y.data_ptr(), sliced.n, m, dt,
            workspace.data_ptr(), workspace.numel() * 4, stream,
        )  # fmt: skip
    except RuntimeError:
        if own:  # a launch of a multi-pass call may have run: the shared buffer is not known to be zero
            drop_sliced_workspace(x.device, stream)
        raise
    return y


class SlicedCallPlan:
    """One layer's :func:`vq_linear_sliced_checked` call with everything that does not change from
    call to call worked out once: the entry point, the addresses of the codebook, bias, permutation,
    header and blob, the workspace need per token count.  ``run`` does per call only what depends on
    the call (x's shape and address, the output tensor, the current stream and its workspace) and
    returns None whenever anything is not as planned -- the caller then takes the ordinary route,
    which checks and reports.  The host time to issue a one-token decode call is Python's, not the
    kernel's: 14 us through the ordinary route against an 11 us kernel."""

    __slots__ = ("fn", "sliced", "cb", "bias_f32", "perm", "device", "index", "dtype", "dt", "n", "k", "limit",
                 "cb_ptr", "bias_ptr", "perm_ptr", "header_ptr", "blob_ptr", "need", "ws", "ws_ptr", "ws_bytes")

    def __init__(self, sliced: SlicedIndices, cb: torch.Tensor, bias_f32, perm, dtype: torch.dtype, limit: int):
        self.fn = getattr(_lib.load(), "npamd_vq_gemv_sliced")
        self.sliced, self.cb, self.bias_f32, self.perm = sliced, cb, bias_f32, perm  # kept alive
        self.device = sliced.blob.device
        self.index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self.dtype, self.dt = dtype, _DT[dtype]
        self.n, self.k = sliced.n, sliced.k
        self.limit = min(int(limit), _lib.GEMV_MAX_M)
        self.cb_ptr, self.bias_ptr, self.perm_ptr = cb.data_ptr(), _ptr(bias_f32), _ptr(perm)
        self.header_ptr, self.blob_ptr = sliced.header_ptr, sliced.blob.data_ptr()
        self.need = [0] + [sliced.workspace_bytes(m) for m in range(1, self.limit + 1)]
        self.ws, self.ws_ptr, self.ws_bytes = None, 0, 0

    def run(self, x: torch.Tensor):
        if x.dtype != self.dtype or x.device != self.device:
            return None
        shape = x.shape
        k, n = self.k, self.n
        if len(shape) == 2:
            m, ldx = shape[0], x.stride(0)
            if shape[1] != k or x.stride(1) != 1:
                return None
            out_shape = (m, n)
        else:
            if not shape or shape[-1] != k or not x.is_contiguous():
                return None
            m, ldx = x.numel() // k, k
            out_shape = (*shape[:-1], n)
        if not 1 <= m <= self.limit or _raw_stream is None:
            return None
        stream = _raw_stream(self.index)
        ws = _SLICED_WORKSPACES.get((self.index, stream))
        if ws is not self.ws:
            if ws is None:
                return None
            self.ws, self.ws_ptr, self.ws_bytes = ws, ws.data_ptr(), ws.numel() * 4
        if self.ws_bytes < self.need[m]:
            return None
        y = torch.empty(out_shape, dtype=self.dtype, device=self.device)
        rc = self.fn(x.data_ptr(), ldx, self.perm_ptr, self.header_ptr, self.blob_ptr, self.cb_ptr, self.dt,
                     self.bias_ptr, y.data_ptr(), n, m, self.dt, self.ws_ptr, self.ws_bytes, stream)  # fmt: skip
        if rc != 0:
            drop_sliced_workspace(self.device, stream)  # it may not be zero-filled any more
            self.ws = None
            return None
        return y


def _vq_linear_coded(what, x, flat, class_streams, payload_streams, payload_bits, payload_base, row_offsets,
                     centroids, vector_len, bias):
    """Shared body of the three prefix-coded GEMV wrappers (``npamd_vq_gemv_coded``)."""
    import ctypes

    streams = [*class_streams, *payload_streams, *row_offsets]
    _check_device(what, x, centroids, bias, *streams)
    x = _x2d(x, what)
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"{what}: x must be float16 or bfloat16, got {x.dtype}")
    cb = _centroids_f16(centroids, what).to(x.dtype)
    if cb.shape[1] != vector_len:
        raise RuntimeError(f"{what}: vector_len does not match the codebook")
    m, k = x.shape
    if k % vector_len:
        raise RuntimeError(f"{what}: K={k} not divisible by vector_len={vector_len}")
    if m > _lib.GEMV_MAX_M:
        raise RuntimeError(f"{what}: M={m} exceeds the fused limit {_lib.GEMV_MAX_M}")
    n_classes = len(payload_streams)
    if len(row_offsets) != n_classes or len(payload_bits) != n_classes or len(payload_base) != n_classes:
        raise RuntimeError(f"{what}: one payload stream, width, base and row-offset table per class")
    for t in (*class_streams, *payload_streams):
        if t.dtype != torch.uint8 or not t.is_contiguous():
            raise RuntimeError(f"{what}: streams must be contiguous uint8 tensors")
    for t in row_offsets:
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise RuntimeError(f"{what}: row offsets must be contiguous int32 tensors")
    n = int(row_offsets[0].numel()) - 1
    if n < 0 or any(int(t.numel()) != n + 1 for t in row_offsets):
        raise RuntimeError(f"{what}: row offsets must all have N + 1 entries")
    ptr_array = lambda ts: (ctypes.c_void_p * max(len(ts), 1))(*[t.data_ptr() if t.numel() else None for t in ts])
    cls_ptrs, pay_ptrs, off_ptrs = ptr_array(class_streams), ptr_array(payload_streams), ptr_array(row_offsets)
    cls_bytes = (ctypes.c_int64 * max(len(class_streams), 1))(*[t.numel() for t in class_streams])
    pay_bytes = (ctypes.c_int64 * n_classes)(*[t.numel() for t in payload_streams])
    bits = (ctypes.c_int * n_classes)(*[int(b) for b in payload_bits])
    base = (ctypes.c_uint32 * n_classes)(*[int(b) for b in payload_base])
    y = torch.empty((m, n), device=x.device, dtype=x.dtype)
    b32 = _bias_f32(bias)
    _lib.call(
        "npamd_vq_gemv_coded", x.data_ptr(), x.stride(0), int(flat), n_classes,
        ctypes.addressof(cls_ptrs), ctypes.addressof(cls_bytes), ctypes.addressof(pay_ptrs), ctypes.addressof(pay_bytes),
        ctypes.addressof(bits), ctypes.addressof(base), ctypes.addressof(off_ptrs),
        cb.data_ptr(), _DT[cb.dtype], cb.shape[0], int(vector_len), _ptr(b32), y.data_ptr(), n, m, n, k,
        _DT[x.dtype], _stream(x),
    )  # fmt: skip
    return y


def vq_linear_tiered(
    x: torch.Tensor,
    prefix_stream: torch.Tensor,
    hot_stream: torch.Tensor,
    cold_stream: torch.Tensor,
    hot_row_off: torch.Tensor,
    cold_row_off: torch.Tensor,
    centroids: torch.Tensor,
    cold_bits: int,
    hot_bits: int,
    vector_len: int,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """Decode GEMV over a two-tier prefix-coded buffer, ``M <= 32`` (reference:
    neuropress/kernels/__init__.py:589-659).  The caller splits the buffer into its streams and
    passes ``TieredIndexPacking.compute_row_offsets`` (on the device)."""
    return _vq_linear_coded("vq_linear_tiered", x, 0, [prefix_stream], [hot_stream, cold_stream],
                            [hot_bits, cold_bits], [0, 0], [hot_row_off, cold_row_off], centroids, vector_len, bias)


def vq_linear_ntier(
    x: torch.Tensor,
    prefix_streams: list[torch.Tensor],
    tier_streams: list[torch.Tensor],
    row_offsets: list[torch.Tensor],
    centroids: torch.Tensor,
    tier_bits: list[int],
    vector_len: int,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """Decode GEMV over an n-tier (cascaded prefix) buffer, ``M <= 32`` (reference:
    neuropress/kernels/__init__.py:711-762)."""
    base = [0] + [1 << int(b) for b in tier_bits[:-1]]
    return _vq_linear_coded("vq_linear_ntier", x, 0, list(prefix_streams), list(tier_streams), list(tier_bits), base,
                            list(row_offsets), centroids, vector_len, bias)


def vq_linear_zero_escape(
    x: torch.Tensor,
    prefix_stream: torch.Tensor,
    hot_stream: torch.Tensor,
    warm_stream: torch.Tensor,
    cold_stream: torch.Tensor,
    row_off_zero: torch.Tensor,
    row_off_hot: torch.Tensor,
    row_off_warm: torch.Tensor,
    row_off_cold: torch.Tensor,
    centroids: torch.Tensor,
    cold_bits: int,
    vector_len: int,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """Decode GEMV over a zero-escape buffer (two class bits per index), ``M <= 32`` (reference:
    neuropress/kernels/__init__.py:974-1049)."""
    empty = prefix_stream.new_empty(0)
    return _vq_linear_coded("vq_linear_zero_escape", x, 1, [prefix_stream], [empty, hot_stream, warm_stream, cold_stream],
                            [0, 4, 8, cold_bits], [0, 1, 17, 257],
                            [row_off_zero, row_off_hot, row_off_warm, row_off_cold], centroids, vector_len, bias)


def vq_lut_gather(
    lut: torch.Tensor,
    packed_indices: torch.Tensor,
    bits: int,
    out_features: int,
) -> torch.Tensor:
    """LUT gather phase: ``y[m, j] = sum_g lut[m, g, idx[j, g]]`` (``npamd_vq_lut_gather``).

    Same signature as the reference's wrapper (neuropress/kernels/__init__.py:405-433):
    *lut* is the float32 ``[M, n_groups, NC]`` table the caller built as
    ``(x.reshape(M * n_groups, VL) @ centroids.T).reshape(M, n_groups, NC)``, the index of
    output ``j``, group ``g`` sits at position ``j * n_groups + g`` of the bit-stream;
    returns float32 ``[M, N]``.
    """
    what = "vq_lut_gather"
    _check_device(what, lut, packed_indices)
    if lut.dim() != 3 or lut.dtype != torch.float32:
        raise RuntimeError(f"{what}: lut must be a float32 [M, n_groups, NC] tensor, got {lut.dtype} {tuple(lut.shape)}")
    lut = lut.contiguous()
    packed = _packed_u8(packed_indices, what)
    m, groups, nc = lut.shape
    y = torch.empty((m, int(out_features)), device=lut.device, dtype=torch.float32)
    _lib.call("npamd_vq_lut_gather", lut.data_ptr(), packed.data_ptr(), packed.numel(), int(bits), y.data_ptr(),
              m, int(out_features), groups, nc, _stream(lut))  # fmt: skip
    return y


def vq_linear_wmma(
    x: torch.Tensor,
    packed_indices: torch.Tensor,
    centroids: torch.Tensor,
    bits: int,
    vector_len: int,
    bias: torch.Tensor | None = None,
    out_features: int | None = None,
) -> torch.Tensor:
    """GEMV/GEMM auto-dispatch on M (reference: neuropress/kernels/__init__.py:335-354).

    ``M <= 32`` runs the fused GEMV, larger M the tile-decode MFMA GEMM.
    """
    if centroids.dim() == 2 and centroids.shape[1] != vector_len:
        raise RuntimeError("vq_linear_wmma: vector_len does not match the codebook")
    entry = "npamd_vq_gemv" if x.shape[0] <= _lib.GEMV_MAX_M else "npamd_vq_gemm_tile"
    return _vq_fused(entry, x, packed_indices, centroids, bits, out_features, bias)


def vq_gemm_tile(
    x: torch.Tensor,
    packed_indices: torch.Tensor,
    centroids: torch.Tensor,
    bits: int,
    out_features: int,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """``x @ W.T (+ bias)`` with W decoded tile by tile inside an MFMA GEMM.

    Signature of the reference's ``vq_gemm_triton`` (neuropress/kernels/vq_triton.py:119-126).
    """
    return _vq_fused("npamd_vq_gemm_tile", x, packed_indices, centroids, bits, out_features, bias)


# ---------------------------------------------------------------------------
# Residual VQ (two codebooks, per-row scale / bias)
# ---------------------------------------------------------------------------


def _f16_or_none(t: torch.Tensor | None, what: str) -> torch.Tensor | None:
    if t is None:
        return None
    if t.dtype != torch.float16:
        raise RuntimeError(f"{what}: per-row scale / bias must be float16")
    return t.contiguous()


def rvq_dequant(
    packed_main: torch.Tensor,
    bits_main: int,
    packed_res: torch.Tensor,
    bits_res: int,
    centroids_main: torch.Tensor,
    centroids_res: torch.Tensor,
    row_scale: torch.Tensor | None,
    row_bias: torch.Tensor | None,
    out_features: int,
    in_features: int,
    dtype: torch.dtype,
) -> torch.Tensor:
    what = "rvq_dequant"
    _check_device(what, packed_main, packed_res, centroids_main, centroids_res, row_scale, row_bias)
    pm, pr = _packed_u8(packed_main, what), _packed_u8(packed_res, what)
    cm, cr = _centroids_f16(centroids_main, what), _centroids_f16(centroids_res, what)
    if cm.dtype != torch.float16 or cr.dtype != torch.float16 or cm.shape[1] != cr.shape[1]:
        raise RuntimeError(f"{what}: codebooks must be float16 with the same vector length")
    sc, rb = _f16_or_none(row_scale, what), _f16_or_none(row_bias, what)
    out = torch.empty((out_features, in_features), device=pm.device, dtype=dtype)
    _lib.call(
        "npamd_rvq_dequant", pm.data_ptr(), pm.numel(), int(bits_main), pr.data_ptr(), pr.numel(),
        int(bits_res), cm.data_ptr(), cm.shape[0], cr.data_ptr(), cr.shape[0], _ptr(sc), _ptr(rb),
        cm.shape[1], out_features, in_features, out.data_ptr(), _dt(dtype, what), _stream(out),
    )  # fmt: skip
    return out


def rvq_linear(
    x: torch.Tensor,
    packed_main: torch.Tensor,
    bits_main: int,
    packed_res: torch.Tensor,
    bits_res: int,
    centroids_main: torch.Tensor,
    centroids_res: torch.Tensor,
    row_scale: torch.Tensor | None,
    row_bias: torch.Tensor | None,
    out_features: int,
    bias: torch.Tensor | None = None,
    tile: bool | None = None,
) -> torch.Tensor:
    """Fused residual-VQ linear; ``tile=None`` picks GEMV for ``M <= 32`` else the tile GEMM."""
    what = "rvq_linear"
    _check_device(what, x, packed_main, packed_res, centroids_main, centroids_res)
    x = _x2d(x, what)
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"{what}: x must be float16 or bfloat16, got {x.dtype}")
    pm, pr = _packed_u8(packed_main, what), _packed_u8(packed_res, what)
    cm, cr = _centroids_f16(centroids_main, what), _centroids_f16(centroids_res, what)
    if cm.dtype != torch.float16 or cr.dtype != torch.float16 or cm.shape[1] != cr.shape[1]:
        raise RuntimeError(f"{what}: codebooks must be float16 with the same vector length")
    sc, rb = _f16_or_none(row_scale, what), _f16_or_none(row_bias, what)
    m, k = x.shape
    if tile is None:
        tile = m > _lib.GEMV_MAX_M
    y = torch.empty((m, out_features), device=x.device, dtype=x.dtype)
    b32 = _bias_f32(bias)
    entry = "npamd_rvq_gemm_tile" if tile else "npamd_rvq_gemv"
    ws, ws_bytes = _tile_workspace(entry, m, out_features, k, x.device)
    extra = (_ptr(ws), ws_bytes) if tile else ()
    _lib.call(
        entry,
        x.data_ptr(), x.stride(0), pm.data_ptr(), pm.numel(), int(bits_main), pr.data_ptr(),
        pr.numel(), int(bits_res), cm.data_ptr(), cm.shape[0], cr.data_ptr(), cr.shape[0],
        _ptr(sc), _ptr(rb), cm.shape[1], _ptr(b32), y.data_ptr(), y.stride(0), m, out_features, k,
        _DT[x.dtype], *extra, _stream(x),
    )  # fmt: skip
    return y


# ---------------------------------------------------------------------------
# Group-affine n-bit
# ---------------------------------------------------------------------------


def _q_args(what, w_pack, scale, zero_point, nbits, group_size):
    if w_pack.dtype != torch.uint8 or w_pack.dim() != 2:
        raise RuntimeError(f"{what}: w_pack must be a 2-D uint8 tensor [N, K/vpb]")
    if scale.dtype != torch.float16:
        raise RuntimeError(f"{what}: scale must be float16")
    if zero_point is not None and zero_point.dtype != torch.float16:
        raise RuntimeError(f"{what}: zero_point must be float16")
    if nbits not in (1, 2, 4, 8):
        raise RuntimeError(f"{what}: nbits must be one of {{1, 2, 4, 8}}, got {nbits}")
    n = w_pack.shape[0]
    k = w_pack.shape[1] * (8 // nbits)
    if group_size <= 0 or k % group_size:
        raise RuntimeError(f"{what}: K={k} not divisible by group_size={group_size}")
    sc = scale.contiguous().reshape(-1)
    if sc.numel() != n * (k // group_size):
        raise RuntimeError(f"{what}: scale has {sc.numel()} entries, expected {n * (k // group_size)}")
    zp = None
    if zero_point is not None:
        zp = zero_point.contiguous().reshape(-1)
        if zp.numel() != sc.numel():
            raise RuntimeError(f"{what}: zero_point must have the same number of entries as scale")
    return w_pack.contiguous(), sc, zp, n, k


def q_dequant(
    w_pack: torch.Tensor,
    scale: torch.Tensor,
    nbits: int,
    group_size: int,
    zero_point: torch.Tensor | None = None,
    dtype: torch.dtype = torch.float16,
) -> torch.Tensor:
    """Decode ``[N, K/vpb]`` packed codes to a dense ``[N, K]`` weight of *dtype*."""
    what = "q_dequant"
    _check_device(what, w_pack, scale, zero_point)
    wp, sc, zp, n, k = _q_args(what, w_pack, scale, zero_point, nbits, group_size)
    out = torch.empty((n, k), device=wp.device, dtype=dtype)
    _lib.call("npamd_q_dequant", wp.data_ptr(), sc.data_ptr(), _ptr(zp), n, k, int(nbits),
              int(group_size), out.data_ptr(), _dt(dtype, what), _stream(out))  # fmt: skip
    return out


def _q_fused(entry, x, w_pack, scale, nbits, group_size, zero_point, bias):
    _check_device(entry, x, w_pack, scale, zero_point, bias)
    wp, sc, zp, n, k = _q_args(entry, w_pack, scale, zero_point, nbits, group_size)
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"{entry}: x must be float16 or bfloat16, got {x.dtype}")
    if x.shape[-1] != k:
        raise RuntimeError(f"{entry}: x has K={x.shape[-1]}, the packed weight has K={k}")
    lead = x.shape[:-1]
    x2 = _x2d(x.reshape(-1, k), entry)
    m = x2.shape[0]
    y = torch.empty((m, n), device=x.device, dtype=x.dtype)
    b32 = _bias_f32(bias)
    ws, ws_bytes = _tile_workspace(entry, m, n, k, x.device)
    extra = (_ptr(ws), ws_bytes) if entry.endswith("_gemm_tile") else ()
    _lib.call(entry, x2.data_ptr(), x2.stride(0), wp.data_ptr(), sc.data_ptr(), _ptr(zp), _ptr(b32),
              y.data_ptr(), y.stride(0), m, n, k, int(nbits), int(group_size), _DT[x.dtype],
              *extra, _stream(x))  # fmt: skip
    return y.reshape(*lead, n)


def q_linear(
    x: torch.Tensor,
    w_pack: torch.Tensor,
    scale: torch.Tensor,
    nbits: int,
    group_size: int,
    zero_point: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """Fused group-quantized dequant + linear (reference: neuropress/kernels/__init__.py:109-151).

    ``M <= 32`` runs the fused GEMV, larger M the fused MFMA GEMM; the reference
    runs its GEMV at every M (neuropress/kernels/q4_linear.cu:137-139).
    """
    m = x.numel() // x.shape[-1] if x.shape[-1] else 0
    entry = "npamd_q_gemv" if m <= _lib.GEMV_MAX_M else "npamd_q_gemm_tile"
    return _q_fused(entry, x, w_pack, scale, nbits, group_size, zero_point, bias)


def q_gemm_tile(x, w_pack, scale, nbits, group_size, zero_point=None, bias=None) -> torch.Tensor:
    """Fused dequant MFMA GEMM at any M."""
    return _q_fused("npamd_q_gemm_tile", x, w_pack, scale, nbits, group_size, zero_point, bias)


# ---------------------------------------------------------------------------
# Fallback reporting
# ---------------------------------------------------------------------------

_warned_fallbacks: set[str] = set()


def warn_kernel_fallback(kernel: str, fallback: str, exc: BaseException) -> None:
    """Warn once per *kernel* that it is unavailable and *fallback* runs instead.

    Same behaviour as the reference (neuropress/kernels/__init__.py:436-453):
    one WARNING per kernel name carrying the cause and the fix; later calls for
    the same kernel are silent.
    """
    if kernel in _warned_fallbacks:
        return
    _warned_fallbacks.add(kernel)
    log.warning(
        "HIP kernel %s unavailable (%s); using %s instead, which can be much slower. "
        "Build the library with `python -m neuropress_amd.build` (needs hipcc from ROCm) "
        "and run on a gfx950 GPU.",
        kernel,
        exc,
        fallback,
    )


# ---------------------------------------------------------------------------
# Neighbours of the linear on a decode step: RMSNorm, embedding lookups
# ---------------------------------------------------------------------------


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """Fused RMSNorm over the last dimension of a 2-D ``x`` (reference: neuropress/kernels/__init__.py
    ``rms_norm``, kernels/rms_norm.cu:79-118: same checks, same signature)."""
    what = "rms_norm"
    _check_device(what, x, weight)
    if x.dim() != 2:
        raise RuntimeError(f"{what}: x must be 2-D [M, H]")
    if weight.dim() != 1 or weight.shape[0] != x.shape[1]:
        raise RuntimeError(f"{what}: weight must be 1-D [H] matching x.size(1)")
    if x.dtype != weight.dtype:
        raise RuntimeError(f"{what}: x and weight must share dtype")
    if x.stride(1) != 1:
        x = x.contiguous()
    weight = weight.contiguous()
    out = torch.empty((x.shape[0], x.shape[1]), device=x.device, dtype=x.dtype)
    _lib.call("npamd_rms_norm", x.data_ptr(), x.stride(0), weight.data_ptr(), out.data_ptr(), out.stride(0),
              x.shape[0], x.shape[1], float(eps), _dt(x.dtype, what), _stream(x))  # fmt: skip
    return out


def vq_embedding(
    input_ids: torch.Tensor,
    all_indices: torch.Tensor,
    centroids: torch.Tensor,
    scale: float = 1.0,
    inv_perm: torch.Tensor | None = None,
    out_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    """Rows of a VQ-compressed embedding table: ``[..., groups * VL]`` for ids of any shape.

    ``all_indices``: ``[vocab, groups]`` int16 (bit pattern of the unsigned index); ``centroids``:
    fp16 ``[NC, VL]``; ``inv_perm``: optional int32 ``[groups * VL]``.  One kernel in place of the
    gather / gather / permute / scale / cast sequence of neuropress/nn/np_vq_embedding.py:120-142.
    """
    what = "vq_embedding"
    _check_device(what, input_ids, all_indices, centroids, inv_perm)
    if all_indices.dtype != torch.int16 or all_indices.dim() != 2:
        raise RuntimeError(f"{what}: all_indices must be int16 [vocab, groups]")
    cb = _centroids_f16(centroids, what)
    if cb.dtype != torch.float16:
        raise RuntimeError(f"{what}: centroids must be float16")
    vocab, groups = all_indices.shape
    dim = groups * cb.shape[1]
    if inv_perm is not None and (inv_perm.dtype != torch.int32 or inv_perm.numel() != dim):
        raise RuntimeError(f"{what}: inv_perm must be int32 with {dim} entries")
    ids = input_ids.reshape(-1).to(torch.int64).contiguous()
    dtype = out_dtype or torch.float16
    out = torch.empty((ids.numel(), dim), device=ids.device, dtype=dtype)
    _lib.call("npamd_vq_embedding", ids.data_ptr(), ids.numel(), all_indices.contiguous().data_ptr(), vocab, groups,
              cb.data_ptr(), cb.shape[0], cb.shape[1], _ptr(None if inv_perm is None else inv_perm.contiguous()),
              float(scale), out.data_ptr(), _dt(dtype, what), _stream(out))  # fmt: skip
    return out.reshape(*input_ids.shape, dim)


def q_embedding(
    input_ids: torch.Tensor,
    u8_blob: torch.Tensor,
    scale: torch.Tensor,
    nbits: int,
    group_size: int,
    zero_point: torch.Tensor | None = None,
    padding_idx: int | None = None,
    embed_scale: float = 1.0,
    out_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    """Rows of a group-affine n-bit embedding table, dequantized: gather, unpack, ``(q - zp) * scale``,
    padding row, dtype cast and ``embed_scale`` of neuropress/nn/np_embedding.py:120-183, 455-473 in one kernel."""
    what = "q_embedding"
    _check_device(what, input_ids, u8_blob, scale, zero_point)
    if u8_blob.dtype != torch.uint8 or u8_blob.dim() != 2:
        raise RuntimeError(f"{what}: u8_blob must be uint8 [vocab, dim * nbits / 8]")
    if nbits not in (1, 2, 4, 8):
        raise RuntimeError(f"{what}: nbits must be 1, 2, 4 or 8, got {nbits}")
    vocab = u8_blob.shape[0]
    dim = u8_blob.shape[1] * (8 // nbits)
    if dim % group_size:
        raise RuntimeError(f"{what}: dim={dim} not divisible by group_size={group_size}")
    sc = scale.reshape(-1).to(torch.float16).contiguous()
    if sc.numel() != vocab * (dim // group_size):
        raise RuntimeError(f"{what}: scale has {sc.numel()} entries, expected {vocab * (dim // group_size)}")
    zp = None
    if zero_point is not None:
        zp = zero_point.reshape(-1).to(torch.float16).contiguous()
        if zp.numel() != sc.numel():
            raise RuntimeError(f"{what}: zero_point must have one entry per group")
    ids = input_ids.reshape(-1).to(torch.int64).contiguous()
    dtype = out_dtype or torch.float16
    out = torch.empty((ids.numel(), dim), device=ids.device, dtype=dtype)
    _lib.call("npamd_q_embedding", ids.data_ptr(), ids.numel(), u8_blob.contiguous().data_ptr(), sc.data_ptr(),
              _ptr(zp), int(nbits), int(group_size), vocab, dim, -1 if padding_idx is None else int(padding_idx),
              float(embed_scale), out.data_ptr(), _dt(dtype, what), _stream(out))  # fmt: skip
    return out.reshape(*input_ids.shape, dim)
