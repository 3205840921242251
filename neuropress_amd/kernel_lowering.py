"""Kernel lowering: swap quantized ``nn.Linear`` modules for hardware modules.

Same surface as the reference (neuropress/kernel_lowering.py:43-368):
``LoweringConfig`` (four backend keys, YAML / dict loading),
``AutoKernelLowering(linear_backend, vq_backend, embedding_backend,
norm_backend).apply(model)`` / ``.from_config(src)``, ``is_lowered`` and
``unlower_model``.

``apply`` runs the lowering passes in the reference's order (kernel_lowering.py:200-219):
scalar-quantized embeddings, scalar-quantized linears, VQ linears, VQ embeddings and -- with
``norm_backend`` ``"auto"`` or ``"cuda"`` -- the RMSNorms that live on a GPU.  When the lowered
model already sits on a GPU it then makes the tensors the decode kernels derive from the
module buffers (:func:`prepare_decode`), so that no forward call has host work left to do.

The module is organised around one table, ``_kinds()``: a row per lowered module class with
the label the summary line shows for it and the function that turns an instance back into
its quantized-weight module.  ``apply``'s summary, ``is_lowered`` and ``unlower_model`` all
read that table.
"""

from __future__ import annotations

import dataclasses
import logging
from abc import ABC, abstractmethod
from collections import Counter
from pathlib import Path
from typing import Callable, NamedTuple

import torch
from torch import nn

__all__ = ["AutoKernelLowering", "KernelLowering", "LoweringConfig", "is_lowered", "prepare_decode", "unlower_model"]

LOGGER = logging.getLogger(__name__)

# Codebook holders the VQ passes register on the model root.
_PROXY_PREFIXES = ("_vq_proxy_", "_vq_res_proxy_", "_vq_emb_proxy_")


@dataclasses.dataclass
class LoweringConfig:
    """Per-path backend selection; every field defaults to ``"auto"``."""

    vq_backend: str = "auto"
    linear_backend: str = "auto"
    embedding_backend: str = "auto"
    norm_backend: str = "auto"

    @classmethod
    def keys(cls) -> list[str]:
        return sorted(f.name for f in dataclasses.fields(cls))

    @classmethod
    def from_dict(cls, d: dict) -> LoweringConfig:
        strangers = sorted(k for k in d if k not in cls.keys())
        if strangers:
            raise ValueError(f"Unknown lowering config key(s): {strangers}. Valid: {cls.keys()}")
        return cls(**{key: str(value) for key, value in d.items()})

    @classmethod
    def from_file(cls, path: Path | str) -> LoweringConfig:
        import yaml

        content = yaml.safe_load(Path(path).read_text())
        if content is None:
            return cls()
        if not isinstance(content, dict):
            raise ValueError(f"{path}: expected a YAML mapping, got {type(content).__name__}")
        return cls.from_dict(content)

    @classmethod
    def load(cls, src: Path | str | dict | None) -> LoweringConfig:
        """*src*: None (defaults), a mapping, or the path of a YAML file."""
        if isinstance(src, dict):
            return cls.from_dict(src)
        return cls() if src is None else cls.from_file(src)

    def save(self, path: Path | str) -> None:
        import yaml

        target = Path(path)
        target.parent.mkdir(parents=True, exist_ok=True)
        target.write_text(yaml.safe_dump(dataclasses.asdict(self), default_flow_style=False, sort_keys=True))


# --------------------------------------------------------------------------------------
# The lowered module classes
# --------------------------------------------------------------------------------------


class _Kind(NamedTuple):
    cls: type
    label: Callable[[nn.Module], str]  # how an instance is named in the summary line
    restore: Callable[[nn.Module], nn.Module | None]  # the quantized-weight module it came from


def _meta_linear(module: nn.Module) -> nn.Module:
    """A plain ``nn.Linear`` carrying *module*'s quantized weight (and bias).  It is allocated
    on the meta device, so no dense weight is ever materialised."""
    from .qweights import attach_quantized_weight

    with torch.device("meta"):
        linear = nn.Linear(module.in_features, module.out_features, bias=module.bias is not None)
    attach_quantized_weight(linear, module.to_qtensor())
    if module.bias is not None:
        linear._parameters["bias"] = nn.Parameter(module.bias.detach(), requires_grad=False)
    return linear


def _meta_embedding(module: nn.Module, vocab: int, scale: float) -> nn.Module:
    from .qweights import attach_quantized_weight

    with torch.device("meta"):
        table = nn.Embedding(vocab, module.embedding_dim, padding_idx=getattr(module, "padding_idx", None))
    attach_quantized_weight(table, module.to_qtensor())
    if scale != 1.0:
        table.embed_scale = scale  # read back by the next lowering (and by scaled-embedding classes)
    return table


def _kinds() -> tuple[_Kind, ...]:
    from .nn.np_embedding import NPEmbedding
    from .nn.np_linear import NPLinear
    from .nn.np_rms_norm import NPRMSNorm
    from .nn.np_vq_embedding import NPVQEmbedding
    from .nn.np_vq_linear import NPVQLinear

    def with_backend(m: nn.Module) -> str:
        return f"{type(m).__name__}({m.backend.value})"

    return (
        _Kind(NPLinear, with_backend, _meta_linear),
        _Kind(NPVQLinear, with_backend, _meta_linear),
        _Kind(NPEmbedding, with_backend, lambda m: _meta_embedding(m, m.num_embeddings, m.embed_scale)),
        _Kind(NPVQEmbedding, lambda m: "NPVQEmbedding", lambda m: _meta_embedding(m, m.all_indices.shape[0], m.scale)),
        _Kind(NPRMSNorm, lambda m: "NPRMSNorm", lambda m: m.to_source_module()),
    )


def _kind_of(module: nn.Module, kinds: tuple[_Kind, ...]) -> _Kind | None:
    return next((kind for kind in kinds if isinstance(module, kind.cls)), None)


def _replace_child(model: nn.Module, dotted: str, new: nn.Module) -> None:
    parent_path, _, leaf = dotted.rpartition(".")
    setattr(model.get_submodule(parent_path) if parent_path else model, leaf, new)


# --------------------------------------------------------------------------------------
# Lowering
# --------------------------------------------------------------------------------------


class KernelLowering(ABC):
    """Replace quantized-weight modules with hardware modules, in place."""

    @abstractmethod
    def apply(self, model: nn.Module) -> None: ...


class AutoKernelLowering(KernelLowering):
    """Run the lowering passes with per-path backends (kernel_lowering.py:136-249)."""

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
        return cls(**dataclasses.asdict(cfg))

    def _passes(self) -> list[Callable[[nn.Module], object]]:
        from .nn.np_embedding import linearize_qtensor_embeddings
        from .nn.np_linear import linearize_qtensor_weights
        from .nn.np_rms_norm import linearize_rms_norms
        from .nn.np_vq_embedding import linearize_vq_embeddings
        from .nn.np_vq_linear import linearize_vq_weights

        passes: list[Callable[[nn.Module], object]] = [
            lambda model: linearize_qtensor_embeddings(model, backend=self.embedding_backend),
            lambda model: linearize_qtensor_weights(model, backend=self.linear_backend),
            lambda model: linearize_vq_weights(model, backend=self.vq_backend),
            linearize_vq_embeddings,
        ]
        if self.norm_backend in ("auto", "cuda"):
            passes.append(linearize_rms_norms)
        return passes

    def apply(self, model: nn.Module) -> None:
        for lowering_pass in self._passes():
            lowering_pass(model)

        # A lowered lm_head no longer shares storage with the embedding table, so a later
        # tie_weights() must not try to re-tie the two (kernel_lowering.py:221-227).
        model_config = getattr(model, "config", None)
        if hasattr(model_config, "tie_word_embeddings"):
            model_config.tie_word_embeddings = False

        kinds = _kinds()
        tally = Counter(kind.label(m) for m in model.modules() if (kind := _kind_of(m, kinds)) is not None)
        if not tally:
            LOGGER.warning("Kernel lowering: no modules were lowered.")
            return
        LOGGER.warning("Kernel lowering applied: %s", ", ".join(f"{n}x {label}" for label, n in sorted(tally.items())))
        prepare_decode(model)


def is_lowered(model: nn.Module) -> bool:
    """True if *model* contains any lowered linear, embedding or norm module (kernel_lowering.py:252-277)."""
    kinds = _kinds()
    return any(_kind_of(m, kinds) is not None for m in model.modules())


def unlower_model(model: nn.Module) -> None:
    """Inverse of :meth:`KernelLowering.apply` (kernel_lowering.py:280-368).

    Every lowered module is turned back into the module it came from (``to_qtensor()``
    rebuilds the quantized weight, which goes onto a plain ``nn.Linear`` / ``nn.Embedding``
    allocated on the meta device; a norm returns its source module) and the codebook holders
    the VQ passes registered on the model root are removed.
    """
    kinds = _kinds()
    restored: dict[str, nn.Module] = {}
    for path, module in model.named_modules():
        kind = _kind_of(module, kinds)
        original = kind.restore(module) if kind is not None else None
        if original is not None:
            restored[path] = original
    for path, original in restored.items():
        _replace_child(model, path, original)
    for child_name in [name for name, _ in model.named_children() if name.startswith(_PROXY_PREFIXES)]:
        delattr(model, child_name)
    LOGGER.info("unlower_model: restored %d module(s) to quantized-weight form", len(restored))


def prepare_decode(model: nn.Module) -> int:
    """Make, for every lowered linear that sits on a GPU, the tensors its kernels derive from the
    module buffers: the fp32 bias, a widened index stream, the int32 column permutation, the
    codebook in the activation dtypes, and -- for layers with codebooks of more than 4096 rows --
    the slice-list form their 1-7 token calls read (``NPVQLinear.prepare_sliced``, the only
    expensive part: a host round trip per layer).  Returns the number of layers whose slice
    lists exist afterwards.

    ``forward`` never does this work: a layer that was not prepared runs its slower decode
    kernel (and says so once).  A lowered module does it by itself when ``.to()`` / ``.cuda()`` /
    ``load_state_dict()`` leave it on a GPU (``NEUROPRESS_VQ_PREPARE_ON_MOVE=0`` switches that
    off), and ``AutoKernelLowering.apply`` calls this function when the model is already there;
    it remains the explicit form -- for buffers replaced by hand, and in front of a HIP-graph
    capture.  No counterpart in the reference.
    """
    from .nn.np_linear import NPLinear
    from .nn.np_vq_linear import NPVQLinear

    with_lists = 0
    for module in model.modules():
        if isinstance(module, NPVQLinear):
            if module.prepare_sliced():
                with_lists += 1
            else:
                module.prepare()
        elif isinstance(module, NPLinear):
            module._bias_f32()
    return with_lists
