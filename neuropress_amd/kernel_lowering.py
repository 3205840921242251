"""Kernel lowering: swap quantized ``nn.Linear`` modules for hardware modules.

Same surface as the reference (neuropress/kernel_lowering.py:43-368):
``LoweringConfig`` (four backend keys, YAML / dict loading),
``AutoKernelLowering(linear_backend, vq_backend, embedding_backend,
norm_backend).apply(model)`` / ``.from_config(src)``, ``is_lowered`` and
``unlower_model``.

``apply`` lowers, in the reference's order (kernel_lowering.py:200-219): scalar-quantized
embeddings, scalar-quantized linears, VQ linears, VQ embeddings and - with ``norm_backend``
``"auto"`` or ``"cuda"`` - the RMSNorms that live on a GPU.
"""

from __future__ import annotations

import logging
from abc import ABC, abstractmethod
from dataclasses import asdict, dataclass
from pathlib import Path

import torch
from torch import nn

__all__ = ["AutoKernelLowering", "KernelLowering", "LoweringConfig", "is_lowered", "prepare_decode", "unlower_model"]

LOGGER = logging.getLogger(__name__)

_VALID_FIELDS = frozenset({"vq_backend", "linear_backend", "embedding_backend", "norm_backend"})


@dataclass
class LoweringConfig:
    """Per-path backend selection; every field defaults to ``"auto"``."""

    vq_backend: str = "auto"
    linear_backend: str = "auto"
    embedding_backend: str = "auto"
    norm_backend: str = "auto"

    @classmethod
    def from_dict(cls, d: dict) -> LoweringConfig:
        unknown = set(d) - _VALID_FIELDS
        if unknown:
            raise ValueError(
                f"Unknown lowering config key(s): {sorted(unknown)}. Valid: {sorted(_VALID_FIELDS)}"
            )
        return cls(**{k: str(v) for k, v in d.items()})

    @classmethod
    def from_file(cls, path: Path | str) -> LoweringConfig:
        import yaml

        with open(path) as fh:
            data = yaml.safe_load(fh) or {}
        if not isinstance(data, dict):
            raise ValueError(f"{path}: expected a YAML mapping, got {type(data).__name__}")
        return cls.from_dict(data)

    @classmethod
    def load(cls, src: Path | str | dict | None) -> LoweringConfig:
        if src is None:
            return cls()
        if isinstance(src, dict):
            return cls.from_dict(src)
        return cls.from_file(src)

    def save(self, path: Path | str) -> None:
        import yaml

        p = Path(path)
        p.parent.mkdir(parents=True, exist_ok=True)
        with p.open("w") as fh:
            yaml.safe_dump(asdict(self), fh, default_flow_style=False, sort_keys=True)


class KernelLowering(ABC):
    """Replace quantized-weight modules with hardware modules, in place."""

    @abstractmethod
    def apply(self, model: nn.Module) -> None: ...


class AutoKernelLowering(KernelLowering):
    """Run the linear lowering passes with per-path backends (kernel_lowering.py:136-249)."""

    def __init__(
        self,
        linear_backend: str = "auto",
        vq_backend: str = "auto",
        embedding_backend: str = "auto",
        norm_backend: str = "auto",
    ) -> None:
        self.linear_backend = linear_backend
        self.vq_backend = vq_backend
        self.embedding_backend = embedding_backend
        self.norm_backend = norm_backend

    @classmethod
    def from_config(cls, src: Path | str | dict | LoweringConfig | None = None) -> AutoKernelLowering:
        cfg = src if isinstance(src, LoweringConfig) else LoweringConfig.load(src)
        return cls(
            linear_backend=cfg.linear_backend,
            vq_backend=cfg.vq_backend,
            embedding_backend=cfg.embedding_backend,
            norm_backend=cfg.norm_backend,
        )

    def apply(self, model: nn.Module) -> None:
        from .nn.np_embedding import NPEmbedding, linearize_qtensor_embeddings
        from .nn.np_linear import NPLinear, linearize_qtensor_weights
        from .nn.np_rms_norm import linearize_rms_norms
        from .nn.np_vq_embedding import NPVQEmbedding, linearize_vq_embeddings
        from .nn.np_vq_linear import NPVQLinear, linearize_vq_weights

        linearize_qtensor_embeddings(model, backend=self.embedding_backend)
        linearize_qtensor_weights(model, backend=self.linear_backend)
        linearize_vq_weights(model, backend=self.vq_backend)
        linearize_vq_embeddings(model)
        n_norms = linearize_rms_norms(model) if self.norm_backend in ("auto", "cuda") else 0

        # A lowered lm_head no longer shares storage with the embedding table:
        # keep later tie_weights() calls from trying to re-tie (kernel_lowering.py:221-227).
        if hasattr(model, "config") and hasattr(model.config, "tie_word_embeddings"):
            model.config.tie_word_embeddings = False

        counts: dict[str, int] = {}
        for m in model.modules():
            if isinstance(m, NPLinear):
                key = f"NPLinear({m.backend.value})"
            elif isinstance(m, NPVQLinear):
                key = f"NPVQLinear({m.backend.value})"
            elif isinstance(m, NPEmbedding):
                key = f"NPEmbedding({m.backend.value})"
            elif isinstance(m, NPVQEmbedding):
                key = "NPVQEmbedding"
            else:
                continue
            counts[key] = counts.get(key, 0) + 1
        if n_norms:
            counts["NPRMSNorm"] = n_norms
        if counts:
            summary = ", ".join(f"{v}x {k}" for k, v in sorted(counts.items()))
            LOGGER.warning("Kernel lowering applied: %s", summary)
        else:
            LOGGER.warning("Kernel lowering: no modules were lowered.")


def is_lowered(model: nn.Module) -> bool:
    """True if *model* contains any lowered linear, embedding or norm module (kernel_lowering.py:252-277)."""
    from .nn.np_embedding import NPEmbedding
    from .nn.np_linear import NPLinear
    from .nn.np_rms_norm import NPRMSNorm
    from .nn.np_vq_embedding import NPVQEmbedding
    from .nn.np_vq_linear import NPVQLinear

    lowered = (NPLinear, NPVQLinear, NPEmbedding, NPVQEmbedding, NPRMSNorm)
    return any(isinstance(m, lowered) for m in model.modules())


def unlower_model(model: nn.Module) -> None:
    """Inverse of :meth:`KernelLowering.apply` (kernel_lowering.py:280-368).

    Each lowered module's ``to_qtensor()`` rebuilds its quantized weight, which is
    placed back on a plain ``nn.Linear`` (allocated on the meta device so no dense
    weight is ever materialised).  Codebook proxies registered on the model root
    are removed.
    """
    from .nn.np_embedding import NPEmbedding
    from .nn.np_linear import NPLinear
    from .nn.np_rms_norm import NPRMSNorm
    from .nn.np_vq_embedding import NPVQEmbedding
    from .nn.np_vq_linear import NPVQLinear
    from .qweights import attach_quantized_weight

    replacements: list[tuple[str, nn.Module]] = []
    for name, module in model.named_modules():
        if isinstance(module, NPRMSNorm):
            source = module.to_source_module()
            if source is not None:
                replacements.append((name, source))
            continue
        if isinstance(module, (NPEmbedding, NPVQEmbedding)):
            vocab = module.num_embeddings if isinstance(module, NPEmbedding) else module.all_indices.shape[0]
            with torch.device("meta"):
                emb = nn.Embedding(vocab, module.embedding_dim, padding_idx=getattr(module, "padding_idx", None))
            attach_quantized_weight(emb, module.to_qtensor())
            scale = module.embed_scale if isinstance(module, NPEmbedding) else module.scale
            if scale != 1.0:
                emb.embed_scale = scale  # read back by the next lowering (and by scaled-embedding classes)
            replacements.append((name, emb))
            continue
        if not isinstance(module, (NPLinear, NPVQLinear)):
            continue
        qweight = module.to_qtensor()
        has_bias = module.bias is not None
        with torch.device("meta"):
            linear = nn.Linear(module.in_features, module.out_features, bias=has_bias)
        attach_quantized_weight(linear, qweight)
        if has_bias:
            linear._parameters["bias"] = nn.Parameter(module.bias.detach(), requires_grad=False)
        replacements.append((name, linear))

    for name, new_mod in replacements:
        if "." in name:
            parent_name, attr = name.rsplit(".", 1)
            parent = model.get_submodule(parent_name)
        else:
            parent, attr = model, name
        setattr(parent, attr, new_mod)

    for pname in [n for n, _ in model.named_children()
                  if n.startswith(("_vq_proxy_", "_vq_res_proxy_", "_vq_emb_proxy_"))]:  # fmt: skip
        delattr(model, pname)
    LOGGER.info("unlower_model: restored %d module(s) to quantized-weight form", len(replacements))


def prepare_decode(model: nn.Module) -> int:
    """Build, for every lowered VQ layer that is on a GPU and uses it, the slice-list form its
    1-4 token calls read (``NPVQLinear.prepare_sliced``); returns the number of layers prepared.

    The layers would otherwise do this host work at their first short call.  Call it after
    moving the model to the GPU and before capturing a HIP graph (a capture must not contain
    the host round trip).  No counterpart in the reference.
    """
    from .nn.np_vq_linear import NPVQLinear

    return sum(1 for m in model.modules() if isinstance(m, NPVQLinear) and m.prepare_sliced())
