"""NPVQEmbedding: lookup in a VQ-compressed embedding table.

Module surface of the reference (neuropress/nn/np_vq_embedding.py:60-142, 166-289): the
indices of the whole table are unpacked once into a ``[vocab, groups]`` int16 buffer; a
forward call gathers the queried tokens' index rows and their codebook rows, undoes the
column permutation, applies the embedding scale and casts.  On a GPU that whole sequence is
one kernel (``kernels.vq_embedding``).

Two differences from the reference, both on inputs it mishandles or refuses: the 16-bit
indices are read as unsigned (its ``.long()`` of an int16 turns indices above 32767 into
negative ones, which only happen to land on the right row when the codebook has exactly
65536 rows), and tables stored in a prefix-coded format are expanded instead of skipped.
"""

from __future__ import annotations

import logging

import torch
import torch.nn as nn

from ..qweights import is_vq_weight
from ..transforms.vq_packing import IndexPacking
from .np_vq_linear import VQProxy

log = logging.getLogger(__name__)


class _WeightProxy:
    """What ``NPVQEmbedding.weight`` returns: row indexing without materialising the table."""

    __slots__ = ("_emb",)

    def __init__(self, emb: NPVQEmbedding) -> None:
        self._emb = emb

    @property
    def shape(self) -> tuple[int, int]:
        return (self._emb.all_indices.shape[0], self._emb.embedding_dim)

    def __getitem__(self, key: object) -> torch.Tensor:
        row_key, rest = (key[0], key[1:]) if isinstance(key, tuple) else (key, ())
        scalar = isinstance(row_key, int)
        ids = torch.tensor([row_key] if scalar else list(row_key), dtype=torch.long,
                           device=self._emb.all_indices.device)  # fmt: skip
        out = self._emb(ids)
        if scalar:
            out = out[0]
        return out[rest] if rest else out


class NPVQEmbedding(nn.Module):
    """VQ-compressed embedding with pre-unpacked indices (see the module docstring)."""

    def __init__(
        self,
        all_indices: torch.Tensor,
        proxy: VQProxy,
        embedding_dim: int,
        vector_len: int,
        scale: float = 1.0,
        inv_perm: torch.Tensor | None = None,
        out_dtype: torch.dtype | None = None,
    ) -> None:
        super().__init__()
        self.register_buffer("all_indices", all_indices.to(torch.int16))
        object.__setattr__(self, "proxy", proxy)  # registered by the owner model, not here
        self.embedding_dim = embedding_dim
        self.vector_len = vector_len
        self.scale = scale
        if inv_perm is not None:
            self.register_buffer("inv_perm", inv_perm)
        else:
            self.inv_perm = None
        self.out_dtype = out_dtype
        self._source_qtensor = None
        self._derived: dict = {}

    def _apply(self, fn, recurse: bool = True):
        result = super()._apply(fn, recurse)
        self._derived = {}
        return result

    def to_qtensor(self):
        """The VQ weight this module was built from (kept at lowering time)."""
        if self._source_qtensor is None:
            raise RuntimeError(
                "NPVQEmbedding._source_qtensor is None - was this module built "
                "via linearize_vq_embeddings()? Cannot unlower for save."
            )
        return self._source_qtensor

    @property
    def weight(self) -> _WeightProxy:
        return _WeightProxy(self)

    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        if input_ids.is_cuda and self.all_indices.is_cuda:
            from .. import kernels

            perm = None
            if self.inv_perm is not None:
                perm = self._derived.get("perm_i32")
                if perm is None or perm.device != input_ids.device:
                    perm = self.inv_perm.to(device=input_ids.device, dtype=torch.int32).contiguous()
                    self._derived["perm_i32"] = perm
            return kernels.vq_embedding(input_ids, self.all_indices, self.proxy.centroids, self.scale, perm,
                                        self.out_dtype)  # fmt: skip
        # torch ops: the specification (reference: np_vq_embedding.py:120-142), indices read as unsigned
        flat = input_ids.flatten()
        idx = self.all_indices[flat].long() & 0xFFFF
        out = self.proxy.centroids[idx].reshape(flat.shape[0], self.embedding_dim)
        if self.inv_perm is not None:
            out = out[:, self.inv_perm]
        if self.scale != 1.0:
            out = out * self.scale
        if self.out_dtype is not None:
            out = out.to(self.out_dtype)
        return out.reshape(*input_ids.shape, self.embedding_dim)

    def extra_repr(self) -> str:
        scale_str = f", scale={self.scale:.4g}" if self.scale != 1.0 else ""
        perm_str = ", perm=True" if self.inv_perm is not None else ""
        dtype_str = f", out_dtype={self.out_dtype}" if self.out_dtype else ""
        return (
            f"vocab={self.all_indices.shape[0]}, dim={self.embedding_dim}, vector_len={self.vector_len}, "
            f"num_centroids={self.proxy.num_centroids}{scale_str}{perm_str}{dtype_str}"
        )


def linearize_vq_embeddings(model: nn.Module) -> int:
    """Replace every non-linear module whose ``weight`` is a VQ weight by an :class:`NPVQEmbedding`.

    Follows neuropress/nn/np_vq_embedding.py:166-289: proxies already registered by
    ``linearize_vq_weights`` are reused (same codebook tensor object), new ones are registered on
    the model root as ``_vq_emb_proxy_<i>``; an ``embed_scale`` attribute of the replaced module
    becomes the lookup's scale; the output dtype is the model's first fp16 / bf16 parameter dtype.
    Returns the number of replacements.
    """
    from ..transforms.vq_entropy_packing import decode_to_flat

    proxy_cache = {id(m.centroids): m for m in model.modules() if isinstance(m, VQProxy)}
    source_cache: dict[int, VQProxy] = {}
    new_proxies: list[VQProxy] = []
    try:
        out_dtype = next(p.dtype for p in model.parameters() if p.dtype in (torch.float16, torch.bfloat16))
    except StopIteration:
        out_dtype = None

    replacements: list[tuple[str, NPVQEmbedding]] = []
    for name, module in model.named_modules():
        if isinstance(module, (NPVQEmbedding, nn.Linear)):
            continue
        weight = module.__dict__.get("weight", None)
        if weight is None:
            weight = getattr(module, "_parameters", {}).get("weight")
        if not is_vq_weight(weight):
            continue
        qs = weight.qscheme
        if qs.original_shape is None or len(tuple(qs.original_shape)) != 2:
            log.warning("linearize_vq_embeddings: skipping %s - qscheme.original_shape is not [vocab, dim].", name)
            continue
        if qs.num_centroids > 65536:
            log.warning("linearize_vq_embeddings: skipping %s - more than 65536 codebook rows.", name)
            continue
        vocab, dim = int(qs.original_shape[0]), int(qs.original_shape[1])
        groups = dim // qs.vector_len
        cid = id(qs.centroids)
        proxy = proxy_cache.get(cid) or source_cache.get(cid)
        if proxy is None:
            proxy = VQProxy(qs.centroids)
            source_cache[cid] = proxy
            new_proxies.append(proxy)
        if getattr(qs, "use_tiered", False) or getattr(qs, "tier_bits", None) or getattr(qs, "zero_escape", False):
            flat = decode_to_flat(weight.u8_blob, use_tiered=qs.use_tiered, tier_bits=qs.tier_bits,
                                  zero_escape=qs.zero_escape)  # fmt: skip
        else:
            flat = IndexPacking.unpack(weight.u8_blob, qs.is_packed_indices, vocab * groups)
        inv_perm = None
        if qs.column_permutation is not None:
            inv_perm = torch.argsort(qs.column_permutation.detach().clone())
        emb = NPVQEmbedding(
            all_indices=flat.reshape(vocab, groups).to(torch.int16),
            proxy=proxy,
            embedding_dim=dim,
            vector_len=qs.vector_len,
            scale=float(getattr(module, "embed_scale", 1.0)),
            inv_perm=inv_perm,
            out_dtype=out_dtype,
        )
        emb._source_qtensor = weight
        replacements.append((name, emb))

    if not replacements:
        log.info("linearize_vq_embeddings: no VQ-weight embedding layers found.")
        return 0
    taken = {n for n, m in model.named_modules() if isinstance(m, VQProxy)}
    i = 0
    for proxy in new_proxies:
        while f"_vq_emb_proxy_{i}" in taken:
            i += 1
        model.add_module(f"_vq_emb_proxy_{i}", proxy)
        taken.add(f"_vq_emb_proxy_{i}")
    for name, emb in replacements:
        parent_name, _, attr = name.rpartition(".")
        setattr(model.get_submodule(parent_name) if parent_name else model, attr, emb)
    log.info("linearize_vq_embeddings: replaced %d layer(s).", len(replacements))
    return len(replacements)
