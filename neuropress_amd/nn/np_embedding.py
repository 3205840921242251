"""NPEmbedding: ``nn.Embedding`` over a group-affine n-bit table.

Module surface of the reference (neuropress/nn/np_embedding.py:193-526): backends
``default`` (decode the whole table, ``F.embedding``), ``compile`` (gather the queried rows in
packed form, unpack and dequantize them with torch ops) and ``cuda``.  Here ``cuda`` is one HIP
kernel (``kernels.q_embedding``) doing gather, unpack, ``(q - zp) * scale``, padding row, dtype
cast and ``embed_scale``; ``"auto"`` picks it when a GPU and the kernel library are there, else
``compile``.  ``compile`` runs the same torch ops eagerly (no tracing compiler in this package).
"""

from __future__ import annotations

import logging

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..qweights import ScalarQScheme, ScalarQWeight, is_scalar_qweight
from .backends import Backend, EmbeddingBackend, is_hip_backend_available
from .np_linear import _kernel_blob, _q_dequant_weight

log = logging.getLogger(__name__)


def _resolve_backend_emb(backend, nbits: int | None = None, group_size: int | None = None) -> EmbeddingBackend:
    """Alias -> concrete :class:`EmbeddingBackend` (np_embedding.py:84-112); ``"gemlite"`` is a ``ValueError``."""
    if backend is None or backend == "torch":
        return EmbeddingBackend.DEFAULT
    if isinstance(backend, (EmbeddingBackend, Backend)):
        backend = backend.value
    if backend == "auto":
        if torch.cuda.is_available() and is_hip_backend_available():
            return EmbeddingBackend.CUDA
        return EmbeddingBackend.COMPILE
    return EmbeddingBackend(backend)


def _emb_dequant(x, u8_blob, scale, nbits: int, group_size: int, zero_point) -> torch.Tensor:
    """Rows ``x`` of the table, dequantized with torch ops: the specification (np_embedding.py:120-183)."""
    vpb = 8 // nbits
    vocab, dim = u8_blob.shape[0], u8_blob.shape[1] * vpb
    groups = dim // group_size
    flat = x.reshape(-1)
    shifts = torch.arange(vpb, device=u8_blob.device, dtype=torch.int32) * nbits
    codes = ((u8_blob[flat].to(torch.int32).unsqueeze(-1) >> shifts) & ((1 << nbits) - 1)).reshape(flat.numel(), dim)
    sc = scale.reshape(vocab, groups)[flat].to(torch.float32).unsqueeze(-1)
    zp = (
        zero_point.reshape(vocab, groups)[flat].to(torch.float32).unsqueeze(-1)
        if zero_point is not None
        else float(1 << (nbits - 1))
    )
    out = (codes.to(torch.float32).reshape(flat.numel(), groups, group_size) - zp) * sc
    return out.reshape(flat.numel(), dim).to(scale.dtype).reshape(*x.shape, dim)


class NPEmbedding(nn.Module):
    """Embedding layer over packed n-bit codes + per-group fp16 scales (and zero points)."""

    def __init__(
        self,
        u8_blob: torch.Tensor,
        scale: torch.Tensor,
        num_embeddings: int,
        embedding_dim: int,
        group_size: int,
        nbits: int,
        qtype: str,
        backend,
        padding_idx: int | None = None,
        zero_point: torch.Tensor | None = None,
        weight_q=None,
        qtensor_meta: dict | None = None,
        embed_scale: float = 1.0,
        out_dtype: torch.dtype | None = None,
    ) -> None:
        super().__init__()
        if qtype not in ("sym", "asym"):
            raise ValueError(f"qtype must be 'sym' or 'asym', got {qtype!r}")
        self._qtensor_meta = qtensor_meta
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.group_size = group_size
        self.nbits = nbits
        self.qtype = qtype
        self.padding_idx = padding_idx
        self.embed_scale = embed_scale
        self.out_dtype = out_dtype
        self.backend = _resolve_backend_emb(backend, nbits=nbits, group_size=group_size)
        if self.backend == EmbeddingBackend.DEFAULT and weight_q is None:
            raise ValueError("weight_q is required when backend='default'.")
        if weight_q is not None:
            object.__setattr__(self, "_weight_q", weight_q)
        self.register_buffer("u8_blob", u8_blob.contiguous())
        self.register_buffer("scale", scale.reshape(-1).contiguous())
        if zero_point is not None:
            self.register_buffer("zero_point", zero_point.reshape(-1).contiguous())
        else:
            self.zero_point = None

    @classmethod
    def from_embedding(cls, embedding: nn.Embedding, backend=EmbeddingBackend.AUTO) -> NPEmbedding:
        """Build from an ``nn.Embedding`` whose weight is a scalar-quantized container (np_embedding.py:301-377)."""
        weight_q = embedding.__dict__.get("weight", None)
        if weight_q is None:
            weight_q = embedding._parameters.get("weight")
        if not is_scalar_qweight(weight_q):
            raise TypeError(
                f"Unsupported weight type {type(weight_q).__name__!r}. "
                "Expected QTensorTractScaleOnly (symmetric) or QTensorScaleZp (asymmetric)."
            )
        qs = weight_q.qscheme
        zp = getattr(qs, "zero_point", None)
        if zp is not None:
            zp = qs.per_group_zero_point().detach()
        bk = _resolve_backend_emb(backend, nbits=qs.n_bits, group_size=qs.group_size)
        scale_buf = getattr(embedding, "embed_scale", None)
        embed_scale = 1.0 if scale_buf is None else float(scale_buf.item() if torch.is_tensor(scale_buf) else scale_buf)
        return cls(
            u8_blob=_kernel_blob(weight_q),
            scale=qs.scale.detach().clone(),
            num_embeddings=embedding.num_embeddings,
            embedding_dim=embedding.embedding_dim,
            group_size=qs.group_size,
            nbits=qs.n_bits,
            qtype="sym" if zp is None else "asym",
            backend=bk,
            padding_idx=embedding.padding_idx,
            zero_point=zp,
            weight_q=weight_q if bk == EmbeddingBackend.DEFAULT else None,
            qtensor_meta={"dequant_to_dtype": getattr(weight_q, "dequant_to_dtype", torch.float16)},
            embed_scale=embed_scale,
            out_dtype=getattr(weight_q, "dequant_to_dtype", None),
        )

    def to_qtensor(self) -> ScalarQWeight:
        """Rebuild the quantized weight; the packed codes are kept bit for bit."""
        if self._qtensor_meta is None:
            raise RuntimeError(
                "Cannot reconstruct QTensor: no serde metadata stored. "
                "Build via NPEmbedding.from_embedding() to enable to_qtensor()."
            )
        if hasattr(self, "_weight_q"):
            return self._weight_q
        scheme = ScalarQScheme(self.nbits, self.group_size, self.scale, self.zero_point)
        return ScalarQWeight(self.u8_blob, scheme, self._qtensor_meta["dequant_to_dtype"])

    def set_backend(self, backend) -> NPEmbedding:
        bk = _resolve_backend_emb(backend, nbits=self.nbits, group_size=self.group_size)
        if bk == EmbeddingBackend.DEFAULT and not hasattr(self, "_weight_q"):
            raise RuntimeError(
                "Cannot switch to EmbeddingBackend.DEFAULT: the original QTensor was "
                "not retained.  Reconstruct NPEmbedding with backend='default'."
            )
        self.backend = bk
        return self

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.backend == EmbeddingBackend.CUDA and x.is_cuda and self.u8_blob.is_cuda:
            from .. import kernels

            return kernels.q_embedding(x, self.u8_blob, self.scale, self.nbits, self.group_size, self.zero_point,
                                       self.padding_idx, self.embed_scale, self.out_dtype or self.scale.dtype)  # fmt: skip
        if self.backend == EmbeddingBackend.DEFAULT:
            table = _q_dequant_weight(self.u8_blob, self.scale, self.nbits, self.group_size, self.zero_point)
            out = F.embedding(x, table.to(self.scale.dtype), padding_idx=self.padding_idx)
        else:
            out = _emb_dequant(x, self.u8_blob, self.scale, self.nbits, self.group_size, self.zero_point)
            if self.padding_idx is not None:
                out = out.clone()
                out[x == self.padding_idx] = 0.0
        if self.out_dtype is not None:
            out = out.to(self.out_dtype)
        if self.embed_scale != 1.0:
            out = out * self.embed_scale
        return out

    def extra_repr(self) -> str:
        parts = [
            f"num_embeddings={self.num_embeddings}", f"embedding_dim={self.embedding_dim}", f"nbits={self.nbits}",
            f"group_size={self.group_size}", f"qtype={self.qtype}", f"backend={self.backend.value}",
        ]  # fmt: skip
        if self.padding_idx is not None:
            parts.append(f"padding_idx={self.padding_idx}")
        return ", ".join(parts)


def linearize_qtensor_embeddings(model: nn.Module, backend=EmbeddingBackend.AUTO) -> nn.Module:
    """Replace every ``nn.Embedding`` carrying a scalar-quantized weight with an :class:`NPEmbedding`
    (np_embedding.py:528-595).  The model is changed in place and returned."""
    replacements: list[tuple[str, NPEmbedding]] = []
    for name, module in model.named_modules():
        if not isinstance(module, nn.Embedding):
            continue
        weight = module.__dict__.get("weight", None)
        if weight is None:
            weight = module._parameters.get("weight")
        if not is_scalar_qweight(weight):
            continue
        try:
            replacements.append((name, NPEmbedding.from_embedding(module, backend)))
        except (TypeError, ValueError) as exc:
            log.warning("linearize_qtensor_embeddings: skipping %s - %s", name, exc)
    for name, emb in replacements:
        parent_name, _, attr = name.rpartition(".")
        setattr(model.get_submodule(parent_name) if parent_name else model, attr, emb)
    log.info("linearize_qtensor_embeddings: replaced %d layer(s)", len(replacements))
    return model
