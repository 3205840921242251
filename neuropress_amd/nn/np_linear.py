"""NPLinear: ``nn.Linear`` replacement with a packed n-bit group-quantized weight.

Same surface as the reference (neuropress/nn/np_linear.py:426-871):
``NPLinear(u8_blob, scale, out_features, in_features, group_size, nbits, qtype,
backend, bias, zero_point, ...)``, ``from_linear``, ``set_backend``,
``to_qtensor``, ``linearize_qtensor_weights`` and the helpers ``_unpack_u8`` /
``_pack_u8`` / ``_q_dequant_linear``.

Dequantisation rule (neuropress/nn/np_linear.py:333-353):

    ``q = (blob[n, k // vpb] >> ((k % vpb) * nbits)) & mask``
    ``w = (float(q) - zp) * float(scale[n, k // group_size])``   (f32),
    ``zp = 2**(nbits-1)`` when symmetric

The ``cuda`` backend runs the HIP kernels: a fused dequant GEMV up to 16
tokens, a fused dequant MFMA GEMM up to ``_Q_TILE_MAX_TOKENS``, and decode +
dense GEMM above.  bf16 activations are computed natively (the reference casts
them to fp16 first, np_linear.py:748-749).
"""

from __future__ import annotations

import logging
import os

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..qweights import ScalarQScheme, ScalarQWeight, is_scalar_qweight
from ..t2n.packing import BitPacking
from .backends import Backend, LinearBackend, is_hip_backend_available, tensor_version, tile_band_ok

log = logging.getLogger(__name__)

# Upper end of the fused-GEMM band for the int4 path; above it decode + GEMM.
# Measured on one MI355X (14336 x 4096, group 32): fused GEMM 35-40 us up to 128
# tokens and 56 us at 256 against 56-64 / 80 us for decode + GEMM; 83-84 vs 78-84 us at
# 320-384, 158 vs 93 us at 512.
_Q_TILE_MAX_TOKENS: int = int(os.environ.get("NEUROPRESS_Q_TILE_MAX_TOKENS", "256"))
# Long reductions (K >= _Q_TILE_SPLIT_LONG_K), where the dense GEMM is slow, keep the fused
# GEMM up to this many tokens: 4096 x 14336 80 vs 105-109 us at 320-384, 148 vs 120 us at 512.
_Q_TILE_LONG_K_MAX_TOKENS: int = 384
# Layers of at least _Q_TILE_WIDE_MIN_FEATURES output or input features run the 128-column fused GEMM
# (256-row blocks past 384 tokens): 14336 x 4096 61 us at 384 tokens and 78-82 at 512 against 86 and 93 us
# for decode + GEMM, 150 against about 140 at 1024; 4096 x 14336 68 / 82 us at 384 / 512.
_Q_TILE_WIDE_MAX_TOKENS: int = int(os.environ.get("NEUROPRESS_Q_TILE_WIDE_MAX_TOKENS", "512"))
_Q_TILE_WIDE_MIN_FEATURES: int = 8192
# As for the VQ path: the fused GEMM splits the reduction when the layer has few
# output features; a layer that still leaves most compute units idle takes decode +
# GEMM.  Measured (fused vs decode + GEMM): 4096 x 14336 41-57 vs 93-115 us from 128 to
# 256 tokens; 4096 x 4096 24-31 vs 37-45 us from 128 to 256, 39-41 vs 39-40 us at
# 320-384; 1024 x 4096 (not enough workgroups even when split) 17-19 vs 16-20 us.
_Q_TILE_MIN_GRID_FRACTION: float = 0.7
_Q_TILE_SPLIT_MAX_TOKENS: int = 256
_Q_TILE_SPLIT_LONG_K: int = 8192
_Q_FUSED_MAX_TOKENS: int = 16
# 17..32 tokens: the GEMV reuses every dequantized operand for two 16-token tiles, and each
# workgroup reads all of x from L2, so it beats the fused GEMM while x is small.  Measured
# (GEMV vs fused GEMM, 17 / 24 / 32 tokens): int4 14336 x 4096 17.0 / 17.8 / 19.9 vs 26-28 us,
# 4096 x 14336 25.5 / 29.5 / 33.8 vs 28 us; with zero points 21-24 vs 41-43 us and 29-37 vs 41 us;
# int8 14336 x 4096 22-25 vs 25-27 us, 4096 x 14336 28-37 vs 26-27 us.
_Q_FUSED_WIDE_MAX_TOKENS: int = 32
_Q_FUSED_WIDE_MAX_ACTIVATIONS = {4: 1 << 18, 8: 1 << 17}  # tokens x in_features, by bit width

_ALLOW_FALLBACK: bool = os.environ.get("NEUROPRESS_ALLOW_KERNEL_FALLBACK", "").strip() in (
    "1", "true", "yes",
)  # fmt: skip


def _unpack_u8(u8_blob: torch.Tensor, nbits: int) -> torch.Tensor:
    """``[N, K/vpb]`` packed bytes -> ``[N, K]`` one value per byte (np_linear.py:78-97)."""
    return BitPacking(nbits).decompress(u8_blob)


def _pack_u8(values: torch.Tensor, nbits: int) -> torch.Tensor:
    """Inverse of :func:`_unpack_u8` (np_linear.py:100-118)."""
    return BitPacking(nbits).compress(values.to(torch.uint8))


def _kernel_blob(weight_q) -> torch.Tensor:
    """The weight's codes in the kernels' ``[N, K // vpb]`` layout (np_linear.py:121-138).

    A blob already bit-packed at the scheme's width has that layout and is reused.
    """
    nbits = weight_q.qscheme.n_bits
    comps = getattr(weight_q, "u8_compressors", None) or []
    if (
        len(comps) == 1
        and getattr(comps[0], "nbits", None) == nbits
        and weight_q.u8_blob.dim() == 2
    ):
        return weight_q.u8_blob
    return _pack_u8(weight_q.decompress_to_u8(), nbits)


def _resolve_backend(
    backend: str | LinearBackend | None,
    nbits: int | None = None,
    group_size: int | None = None,
) -> LinearBackend:
    """Resolve an alias to a concrete :class:`LinearBackend` (np_linear.py:166-213).

    ``"auto"``: ``CUDA`` (the HIP kernels) when a GPU and the kernel library
    are available, else ``COMPILE``.  The third-party GemLite backend the
    reference prefers is not part of this package; asking for it explicitly
    raises ``ValueError`` at construction.
    """
    if backend is None or backend == "torch":
        return LinearBackend.DEFAULT
    if isinstance(backend, (LinearBackend, Backend)):
        backend = backend.value
    if backend != "auto":
        return LinearBackend(backend)  # ValueError for unknown strings
    if torch.cuda.is_available() and is_hip_backend_available():
        return LinearBackend.CUDA
    return LinearBackend.COMPILE


def _q_dequant_weight(
    u8_blob: torch.Tensor,
    scale: torch.Tensor,
    nbits: int,
    group_size: int,
    zero_point: torch.Tensor | None,
) -> torch.Tensor:
    """f32 ``[N, K]`` weight with torch ops (the decode half of np_linear.py:333-351)."""
    n = u8_blob.shape[0]
    vals = _unpack_u8(u8_blob, nbits).to(torch.float32)
    k = vals.shape[1]
    g = k // group_size
    vals = vals.reshape(n, g, group_size)
    sc = scale.to(torch.float32).reshape(n, g, 1)
    zp = (
        zero_point.to(torch.float32).reshape(n, g, 1)
        if zero_point is not None
        else float(1 << (nbits - 1))
    )
    return ((vals - zp) * sc).reshape(n, k)


def _q_dequant_linear(
    x: torch.Tensor,
    u8_blob: torch.Tensor,
    scale: torch.Tensor,
    nbits: int,
    group_size: int,
    zero_point: torch.Tensor | None,
    bias: torch.Tensor | None,
) -> torch.Tensor:
    """Generic n-bit group-quantized dequant + linear with torch ops (np_linear.py:298-353)."""
    w = _q_dequant_weight(u8_blob, scale, nbits, group_size, zero_point)
    return F.linear(x, w.to(x.dtype), bias)


class NPLinear(nn.Module):
    """Linear layer with a packed n-bit quantized weight and a pluggable backend."""

    def __init__(
        self,
        u8_blob: torch.Tensor,
        scale: torch.Tensor,
        out_features: int,
        in_features: int,
        group_size: int,
        nbits: int,
        qtype: str,
        backend: str | LinearBackend | None,
        bias: torch.Tensor | None = None,
        zero_point: torch.Tensor | None = None,
        weight_q=None,
        qtensor_meta: dict[str, str] | None = None,
        compute_dtype: torch.dtype = torch.float16,
    ) -> None:
        super().__init__()
        if qtype not in ("sym", "asym"):
            raise ValueError(f"qtype must be 'sym' or 'asym', got {qtype!r}")
        self._qtensor_meta = qtensor_meta
        self.out_features = out_features
        self.in_features = in_features
        self.group_size = group_size
        self.nbits = nbits
        self.qtype = qtype
        self.backend = _resolve_backend(backend, nbits=nbits, group_size=group_size)
        if self.backend == LinearBackend.GEMLITE:
            raise ValueError("backend 'gemlite' is a third-party kernel not included in this package")
        self._compute_dtype = compute_dtype
        if weight_q is not None:
            object.__setattr__(self, "_weight_q", weight_q)

        self.register_buffer("u8_blob", u8_blob.contiguous())
        self.register_buffer("scale", scale.to(torch.float16).reshape(-1).contiguous())
        if zero_point is not None:
            self.register_buffer("zero_point", zero_point.to(torch.float16).reshape(-1).contiguous())
        else:
            self.zero_point = None
        if bias is not None:
            self.register_buffer("bias", bias.contiguous())
        else:
            self.bias = None
        self._derived: dict = {}

    def _apply(self, fn, recurse: bool = True):
        result = super()._apply(fn, recurse)
        self._derived = {}
        return result

    @classmethod
    def from_linear(
        cls, linear: nn.Linear, backend: str | LinearBackend | None = LinearBackend.AUTO
    ) -> NPLinear:
        """Build from an ``nn.Linear`` with a scalar-quantized weight (np_linear.py:539-607)."""
        wq = linear.weight
        if not is_scalar_qweight(wq):
            raise TypeError(
                f"Unsupported weight type {type(wq).__name__!r}. Expected a scale-only "
                "(symmetric) or scale+zero-point (asymmetric) quantized weight."
            )
        qs = wq.qscheme
        zp = None
        if getattr(qs, "zero_point", None) is not None:
            zp = qs.per_group_zero_point().detach() if hasattr(qs, "per_group_zero_point") else qs.zero_point
        bias = linear.bias.detach().clone() if linear.bias is not None else None
        return cls(
            u8_blob=_kernel_blob(wq),
            scale=qs.scale.detach().clone(),
            out_features=linear.out_features,
            in_features=linear.in_features,
            group_size=qs.group_size,
            nbits=qs.n_bits,
            qtype="sym" if zp is None else "asym",
            backend=backend,
            bias=bias,
            zero_point=zp,
            weight_q=wq,
            qtensor_meta={"dequant_to_dtype": str(getattr(wq, "dequant_to_dtype", torch.float16))},
            compute_dtype=getattr(wq, "dequant_to_dtype", torch.float16),
        )

    def to_qtensor(self) -> ScalarQWeight:
        """Rebuild the quantized weight; the packed blob is preserved bit for bit
        (the property tested at tests/test_quantized_weight_regressions.py:79-92 of the reference)."""
        if self._qtensor_meta is None:
            raise RuntimeError(
                "Cannot reconstruct QTensor: no serde metadata stored. "
                "Build via NPLinear.from_linear() to enable to_qtensor()."
            )
        scheme = ScalarQScheme(self.nbits, self.group_size, self.scale, self.zero_point)
        return ScalarQWeight(self.u8_blob, scheme, self._compute_dtype)

    def set_backend(self, backend: str | LinearBackend | None) -> NPLinear:
        """Switch backend in place; ``"auto"`` re-resolves now (np_linear.py:651-696)."""
        bk = _resolve_backend(backend, nbits=self.nbits, group_size=self.group_size)
        if bk == LinearBackend.GEMLITE:
            raise RuntimeError("backend 'gemlite' is not available in this package")
        self.backend = bk
        return self

    # ------------------------------------------------------------------

    def _bias_f32(self) -> torch.Tensor | None:
        if self.bias is None:
            return None
        # Keyed on the buffer's device, address and version counter: load_state_dict or an in-place
        # copy_ into `bias` makes a new fp32 copy.  Not stored inside a graph capture (a tensor made
        # there holds data only after a replay).
        src = self.bias
        key = (src.device, src.data_ptr(), tensor_version(src))
        hit = self._derived.get("bias_f32")
        if hit is not None and hit[0] == key:
            return hit[1]
        b = src.detach().to(torch.float32).contiguous()
        if not (src.is_cuda and torch.cuda.is_current_stream_capturing()):
            self._derived["bias_f32"] = (key, b)
        return b

    def _bias_as(self, dtype: torch.dtype) -> torch.Tensor | None:
        if self.bias is None or self.bias.dtype == dtype:
            return self.bias
        return self.bias.to(dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.backend == LinearBackend.CUDA:
            return self._forward_cuda(x)
        # default / compile: the torch-op specification of the layer.
        return self._forward_compile(x)

    def _forward_compile(self, x: torch.Tensor) -> torch.Tensor:
        return _q_dequant_linear(
            x, self.u8_blob, self.scale, self.nbits, self.group_size, self.zero_point,
            self._bias_as(x.dtype),
        )

    def _mfma_layer(self) -> bool:
        ok = self._derived.get("mfma_layer")
        if ok is None:
            from .. import kernels

            ok = kernels.q_fused_supported(self.in_features, self.nbits, self.group_size)
            self._derived["mfma_layer"] = ok
        return ok

    def _tile_grid_fills_gpu(self, x: torch.Tensor, m: int) -> bool:
        cus = self._derived.get("cus")
        if cus is None:
            cus = torch.cuda.get_device_properties(x.device).multi_processor_count
            self._derived["cus"] = cus
        return tile_band_ok(
            m, self.out_features, self.in_features, cus,
            _Q_TILE_MIN_GRID_FRACTION, _Q_TILE_SPLIT_MAX_TOKENS, _Q_TILE_SPLIT_LONG_K,
        )  # fmt: skip

    def _gemv_max_tokens(self, m: int) -> int:
        """End of the GEMV band for a call of *m* tokens: 16, or 32 while x stays small."""
        if _Q_FUSED_MAX_TOKENS < m <= _Q_FUSED_WIDE_MAX_TOKENS:
            cap = _Q_FUSED_WIDE_MAX_ACTIVATIONS.get(self.nbits, 0)
            if self.zero_point is not None and self.nbits == 4:
                cap = 1 << 30  # the fused GEMM pays for the zero points per tile: GEMV at any K
            if m * self.in_features <= cap:
                return _Q_FUSED_WIDE_MAX_TOKENS
            # One row tile per workgroup: the GEMV stages its activations through LDS and stays
            # ahead of the tile GEMM at any K (int4, GEMV vs tile GEMM at 17 / 24 / 32 tokens:
            # 4096 x 14336 23.6 / 24.4 / 25.6 vs 29.5-29.9 us, 4096 x 8192 15.2 / 15.0 / 15.6 vs 21.8-22.5 us).
            if self.nbits == 4:
                from .. import kernels

                if kernels.gemv_stages_activations(m, self.out_features, self.in_features, 0):
                    return _Q_FUSED_WIDE_MAX_TOKENS
        return _Q_FUSED_MAX_TOKENS

    def _forward_cuda(self, x: torch.Tensor) -> torch.Tensor:
        """HIP path by token count; takes the place of np_linear.py:731-761."""
        if not x.is_cuda:
            return self._forward_compile(x)
        from .. import kernels

        m = x.numel() // self.in_features
        try:
            # Layers the MFMA kernels do not take (1 / 2 / 8 bits, odd group sizes) would run an
            # element-wise kernel, slower at every token count than decoding once and calling the
            # dense GEMM (14336 x 4096, 8 bits: 99 us against 57 us at one token, 452 against 57 at 16).
            fused_ok = x.dtype in (torch.float16, torch.bfloat16) and self._mfma_layer()
            gemv_max = self._gemv_max_tokens(m)
            if fused_ok and m > gemv_max:
                limit = _Q_TILE_MAX_TOKENS
                if self.in_features >= _Q_TILE_SPLIT_LONG_K:
                    limit = max(limit, _Q_TILE_LONG_K_MAX_TOKENS)
                if limit > 0 and max(self.in_features, self.out_features) >= _Q_TILE_WIDE_MIN_FEATURES:
                    limit = max(limit, _Q_TILE_WIDE_MAX_TOKENS)
                fused_ok = m <= limit and self._tile_grid_fills_gpu(x, m)
            if fused_ok:
                if m <= gemv_max:
                    return kernels.q_linear(
                        x, self.u8_blob, self.scale, self.nbits, self.group_size,
                        self.zero_point, self._bias_f32(),
                    )  # fmt: skip
                return kernels.q_gemm_tile(
                    x, self.u8_blob, self.scale, self.nbits, self.group_size,
                    self.zero_point, self._bias_f32(),
                )  # fmt: skip
            w = kernels.q_dequant(
                self.u8_blob, self.scale, self.nbits, self.group_size, self.zero_point, x.dtype
            )
        except RuntimeError as exc:
            if not _ALLOW_FALLBACK:
                raise
            kernels.warn_kernel_fallback("q_linear", "torch dequant + matmul", exc)
            return self._forward_compile(x)
        return F.linear(x, w, self._bias_as(x.dtype))

    def extra_repr(self) -> str:
        return (
            f"in={self.in_features}, out={self.out_features}, "
            f"nbits={self.nbits}, group_size={self.group_size}, "
            f"qtype={self.qtype}, backend={self.backend.value}"
        )


def linearize_qtensor_weights(
    model: nn.Module,
    backend: str | LinearBackend | None = LinearBackend.AUTO,
) -> nn.Module:
    """Replace every ``nn.Linear`` carrying a scalar-quantized weight with an :class:`NPLinear`.

    Follows neuropress/nn/np_linear.py:796-871; VQ weights are left to
    :func:`~neuropress_amd.nn.np_vq_linear.linearize_vq_weights`.
    """
    replacements: list[tuple[str, NPLinear]] = []
    for name, module in model.named_modules():
        if not isinstance(module, nn.Linear) or not is_scalar_qweight(module.weight):
            continue
        try:
            layer = NPLinear.from_linear(module, backend)
        except (TypeError, ValueError) as exc:
            log.warning("linearize_qtensor_weights: skipping %s — %s", name, exc)
            continue
        replacements.append((name, layer))

    for name, layer in replacements:
        if "." in name:
            parent_name, attr = name.rsplit(".", 1)
            parent = model.get_submodule(parent_name)
        else:
            parent, attr = model, name
        setattr(parent, attr, layer)

    counts: dict[str, int] = {}
    for _, layer in replacements:
        counts[layer.backend.value] = counts.get(layer.backend.value, 0) + 1
    summary = ", ".join(f"{v}x{k}" for k, v in sorted(counts.items()))
    log.info(
        "linearize_qtensor_weights: replaced %d layer(s) [%s]", len(replacements), summary or "none"
    )
    return model
