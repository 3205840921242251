"""Checkpoint IO: one safetensors file holding regular tensors and quantized weights.

Same file layout as the reference's ``save_quantized_model`` / ``load_quantized_model``
(neuropress/t2n/model_io.py:55-67, 214-310, 463-596; component names and metadata of each
quantized-weight type: neuropress/t2n/qtensors.py:302-548), so a checkpoint written by either
side names its parts the same way:

* ``{param_path}``                      a regular parameter or buffer
* ``{param_path}::{component}``         one component of a quantized weight
* file metadata ``__neuropress_manifest__`` = JSON ``{"format_version": "2", "transforms":
  [{"type": "qtensor_assignment", "qtensor_params": {param_path: {"type", "tensor_keys",
  "metadata"}}}, ...], "recipe_config": ...}``

Quantized-weight types and their components:

=======================  =======================================  ================================
type                     components                               metadata (all strings)
=======================  =======================================  ================================
``QTensorTractVQ``       u8_blob, centroids (f16),                proxy_selector, original_shape,
                         column_permutation (optional)            bits_per_index, dequant_to_dtype,
                                                                  proxy_content_hash,
                                                                  has_column_perm, use_tiered,
                                                                  zero_escape
``QTensorTractScaleOnly`` u8_blob, scale                           shape, packing, n_bits,
                                                                  group_size, dequant_to_dtype,
                                                                  nnef_name
``QTensorScaleZp``       u8_blob, scale, zero_point               the same + export_as_float
=======================  =======================================  ================================

Additions of this backend, ignored by a reader that does not know them: VQ metadata
``tier_bits`` (JSON list; the reference's file does not record the n-tier widths) and, for
residual VQ layers, components ``residual_blob`` / ``residual_centroids`` / ``row_scale`` /
``row_bias`` with metadata ``residual_bits``.

The weights handled are the containers of :mod:`neuropress_amd.qweights` (and anything with the
same attributes), found as the ``.weight`` of ``nn.Linear`` and ``nn.Embedding`` modules.  A kernel-lowered model is
unlowered for the save and lowered again afterwards, as in the reference.
"""

from __future__ import annotations

import hashlib
import json
import logging
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any

import torch
from torch import nn

from ..qweights import (
    ScalarQScheme,
    ScalarQWeight,
    VQScheme,
    VQWeight,
    attach_quantized_weight,
    is_scalar_qweight,
    is_vq_weight,
)
from .packing import BitPacking

_log = logging.getLogger(__name__)

_MANIFEST_META_KEY = "__neuropress_manifest__"
_QT_SEP = "::"
_FORMAT_VERSION = "2"


@dataclass
class QuantizationManifest:
    """What a checkpoint's metadata records: the ordered transforms and the recipe JSON."""

    transforms: list[dict[str, Any]] = field(default_factory=list)
    recipe_config_json: str | None = None

    def _assignment(self) -> dict[str, dict[str, Any]]:
        for t in self.transforms:
            if t.get("type") == "qtensor_assignment":
                return t.get("qtensor_params", {})
        return {}

    @property
    def qtensor_params(self) -> dict[str, str]:
        """Parameter path -> quantized-weight type name."""
        return {path: entry["type"] for path, entry in self._assignment().items()}


# ---------------------------------------------------------------------------
# Per-type (de)composition
# ---------------------------------------------------------------------------


def _centroid_hash(centroids: torch.Tensor) -> str:
    """SHA-256 of the codebook's fp16 bytes (reference: neuropress/t2n/qtensors.py:68-71)."""
    return hashlib.sha256(centroids.to(torch.float16).cpu().contiguous().numpy().tobytes()).hexdigest()


def _dtype_name(dtype: torch.dtype) -> str:
    return str(dtype).replace("torch.", "")


def _type_name(weight) -> str | None:
    if is_vq_weight(weight):
        return "QTensorTractVQ"
    if is_scalar_qweight(weight):
        return "QTensorScaleZp" if getattr(weight.qscheme, "zero_point", None) is not None else "QTensorTractScaleOnly"
    return None


def _vq_tensors(w) -> dict[str, torch.Tensor]:
    qs = w.qscheme
    out = {"u8_blob": w.u8_blob.cpu(), "centroids": qs.centroids.to(torch.float16).cpu().clone()}
    if getattr(qs, "column_permutation", None) is not None:
        out["column_permutation"] = qs.column_permutation.cpu()
    if getattr(w, "residual_blob", None) is not None:
        out["residual_blob"] = w.residual_blob.cpu()
    for key in ("residual_centroids", "row_scale", "row_bias"):
        t = getattr(qs, key, None)
        if t is not None:
            out[key] = t.to(torch.float16).cpu().clone()
    return out


def _vq_metadata(w) -> dict[str, str]:
    qs = w.qscheme
    shape = tuple(qs.original_shape) if qs.original_shape is not None else ()
    selector = getattr(qs, "proxy_selector", "l2")
    meta = {
        "proxy_selector": getattr(selector, "value", selector),
        "original_shape": ",".join(str(int(d)) for d in shape),
        "bits_per_index": str(qs.is_packed_indices),
        "dequant_to_dtype": _dtype_name(getattr(w, "dequant_to_dtype", torch.float16)),
        "proxy_content_hash": _centroid_hash(qs.centroids),
        "has_column_perm": "1" if getattr(qs, "column_permutation", None) is not None else "0",
        "use_tiered": "1" if getattr(qs, "use_tiered", False) else "0",
        "zero_escape": "1" if getattr(qs, "zero_escape", False) else "0",
    }
    if getattr(qs, "tier_bits", None) is not None:
        meta["tier_bits"] = json.dumps(list(qs.tier_bits))
    if getattr(qs, "residual_bits", 0):
        meta["residual_bits"] = str(qs.residual_bits)
    return meta


def _vq_from_parts(tensors: dict[str, torch.Tensor], meta: dict[str, str], cache: dict[str, torch.Tensor]) -> VQWeight:
    # Layers saved with the same codebook get the same tensor object back, so that lowering
    # shares one proxy between them (reference: neuropress/t2n/qtensors.py:496-509).
    centroids = tensors["centroids"]
    key = meta.get("proxy_content_hash")
    if key is not None:
        centroids = cache.setdefault(key, centroids)
    shape = meta.get("original_shape", "")
    tier_bits = json.loads(meta["tier_bits"]) if "tier_bits" in meta else None
    blob = tensors["u8_blob"]
    use_tiered = meta.get("use_tiered", "0") == "1"
    zero_escape = meta.get("zero_escape", "0") == "1"
    scheme = VQScheme(
        centroids=centroids,
        original_shape=tuple(int(d) for d in shape.split(",")) if shape else (),
        is_packed_indices=int(meta.get("bits_per_index", 0) or 0),
        column_permutation=tensors.get("column_permutation") if meta.get("has_column_perm") == "1" else None,
        use_tiered=use_tiered,
        tier_bits=tier_bits,
        zero_escape=zero_escape,
        residual_centroids=tensors.get("residual_centroids"),
        residual_bits=int(meta.get("residual_bits", 0) or 0),
        row_scale=tensors.get("row_scale"),
        row_bias=tensors.get("row_bias"),
    )
    if tier_bits is None and not zero_escape and not use_tiered:
        _adopt_unlabelled_ntier(scheme, blob)
    return VQWeight(blob, scheme, tensors.get("residual_blob"))


def _adopt_unlabelled_ntier(scheme: VQScheme, blob: torch.Tensor) -> None:
    """An n-tier buffer whose file does not say so (the reference's writer keeps no ``tier_bits``).

    Taken as n-tier only when the magic matches, the header's index count is the layer's and the
    byte count is not the one a fixed-width stream of that many indices would have.
    """
    from ..transforms.vq_packing import IndexPacking, NTieredIndexPacking

    if not NTieredIndexPacking.is_ntier_buffer(blob) or not scheme.original_shape:
        return
    n_vec = 1
    for d in scheme.original_shape:
        n_vec *= d
    n_vec //= scheme.vector_len
    if blob.numel() == IndexPacking.packed_nbytes(n_vec, scheme.is_packed_indices):
        return
    try:
        n, _, _, bits, _ = NTieredIndexPacking._parse_header(blob)
    except ValueError:
        return
    if n == n_vec:
        scheme.tier_bits = list(bits)


def _scalar_tensors(w) -> dict[str, torch.Tensor]:
    out = {"u8_blob": w.u8_blob.cpu(), "scale": w.qscheme.scale.cpu()}
    if getattr(w.qscheme, "zero_point", None) is not None:
        out["zero_point"] = w.qscheme.zero_point.cpu()
    return out


def _scalar_shape(w) -> list[int]:
    shape = getattr(w, "decompressed_shape", None)
    if shape is not None:
        return [int(d) for d in shape]
    blob = w.u8_blob
    per_byte = 1
    for comp in getattr(w, "u8_compressors", []):
        per_byte *= 8 // comp.nbits
    return [int(blob.shape[0]), int(blob.shape[1]) * per_byte]


def _scalar_metadata(w) -> dict[str, str]:
    comps = list(getattr(w, "u8_compressors", []))
    if any(not isinstance(c, BitPacking) and not hasattr(c, "nbits") for c in comps):
        raise ValueError("Scalar tensor persistence requires BitPacking compressors")
    meta = {
        "shape": json.dumps(_scalar_shape(w)),
        "packing": json.dumps([int(c.nbits) for c in comps]),
        "n_bits": str(w.qscheme.n_bits),
        "group_size": str(w.qscheme.group_size),
        "dequant_to_dtype": _dtype_name(getattr(w, "dequant_to_dtype", torch.float16)),
        "nnef_name": getattr(w, "nnef_name", None) or "",
    }
    if getattr(w.qscheme, "zero_point", None) is not None:
        meta["export_as_float"] = "1" if getattr(w, "export_as_float", False) else "0"
    return meta


def _scalar_from_parts(tensors: dict[str, torch.Tensor], meta: dict[str, str]) -> ScalarQWeight:
    n_bits = int(meta["n_bits"])
    if "packing" in meta:
        packing = json.loads(meta["packing"])
    else:  # older files: packed iff the blob is smaller than the code count (qtensors.py:219-227)
        count = tensors["scale"].numel() * int(meta["group_size"])
        packing = [n_bits] if tensors["u8_blob"].numel() < count else []
    scheme = ScalarQScheme(n_bits, int(meta["group_size"]), tensors["scale"], tensors.get("zero_point"))
    w = ScalarQWeight(tensors["u8_blob"], scheme, getattr(torch, meta["dequant_to_dtype"]),
                      u8_compressors=[BitPacking(b) for b in packing])  # fmt: skip
    if "shape" in meta:
        w.decompressed_shape = torch.Size(json.loads(meta["shape"]))
    w.nnef_name = meta.get("nnef_name") or None
    w.export_as_float = meta.get("export_as_float") == "1"
    return w


def _to_tensors(weight) -> dict[str, torch.Tensor]:
    return _vq_tensors(weight) if is_vq_weight(weight) else _scalar_tensors(weight)


def _to_metadata(weight) -> dict[str, str]:
    return _vq_metadata(weight) if is_vq_weight(weight) else _scalar_metadata(weight)


_KNOWN_TYPES = ("QTensorTractVQ", "QTensorTractScaleOnly", "QTensorScaleZp")


# ---------------------------------------------------------------------------
# Manifest
# ---------------------------------------------------------------------------


def _quantized_weights(model: nn.Module) -> dict[str, Any]:
    """``{param_path: weight}`` for every ``nn.Linear`` / ``nn.Embedding`` whose weight is a quantized container."""
    found = {}
    for name, module in model.named_modules():
        if isinstance(module, (nn.Linear, nn.Embedding)):
            w = module.__dict__.get("weight", None)
            if w is None:
                w = module._parameters.get("weight")
            if _type_name(w) is not None:
                found[f"{name}.weight" if name else "weight"] = w
    return found


def attach_manifest(model: nn.Module, recipe_config_json: str | None = None) -> QuantizationManifest:
    """Record the model's quantized weights in ``model.__neuropress_manifest__``.

    Other transform entries already on the manifest are kept; with no quantized weight found
    an existing assignment entry is kept too (reference: neuropress/t2n/model_io.py:146-206).
    """
    manifest = getattr(model, "__neuropress_manifest__", None)
    if not isinstance(manifest, QuantizationManifest):
        manifest = QuantizationManifest()
    entries = {
        path: {"type": _type_name(w), "tensor_keys": list(_to_tensors(w)), "metadata": _to_metadata(w)}
        for path, w in _quantized_weights(model).items()
    }
    if entries:
        manifest.transforms = [t for t in manifest.transforms if t.get("type") != "qtensor_assignment"]
        manifest.transforms.append({"type": "qtensor_assignment", "qtensor_params": entries})
    if recipe_config_json is not None:
        manifest.recipe_config_json = recipe_config_json
    model.__neuropress_manifest__ = manifest
    return manifest


# ---------------------------------------------------------------------------
# Save / load
# ---------------------------------------------------------------------------


def save_quantized_model(model: nn.Module, path: str | Path, recipe_config_json: str | None = None) -> None:
    """Write *model* (regular tensors + quantized weights + manifest) to *path*."""
    from safetensors.torch import save_file

    from ..kernel_lowering import is_lowered, unlower_model

    lowering = getattr(model, "__neuropress_kernel_lowering__", None)
    was_lowered = is_lowered(model)
    if was_lowered:
        if torch.cuda.is_available():
            torch.cuda.synchronize()
        unlower_model(model)
    try:
        manifest = attach_manifest(model, recipe_config_json=recipe_config_json)
        tensors: dict[str, torch.Tensor] = {}
        for param_path, w in _quantized_weights(model).items():
            for key, t in _to_tensors(w).items():
                tensors[f"{param_path}{_QT_SEP}{key}"] = t
        for name, p in model.named_parameters():
            if p.device.type != "meta":
                tensors.setdefault(name, p.data)
        for name, b in model.named_buffers():
            if b is not None and b.device.type != "meta":
                tensors.setdefault(name, b)
        rc = json.loads(manifest.recipe_config_json) if manifest.recipe_config_json else None
        meta = {"format_version": _FORMAT_VERSION, "transforms": manifest.transforms, "recipe_config": rc}
        # safetensors refuses entries that share storage (two layers with one codebook or one
        # scale tensor): every storage is written once as it is, later users of it as copies.
        out: dict[str, torch.Tensor] = {}
        seen: set[int] = set()
        for k, v in tensors.items():
            v = v.detach().cpu().contiguous()
            ptr = v.untyped_storage().data_ptr() if v.numel() else 0
            if ptr and ptr in seen:
                v = v.clone()
            seen.add(v.untyped_storage().data_ptr() if v.numel() else 0)
            out[k] = v
        save_file(out, str(path), metadata={_MANIFEST_META_KEY: json.dumps(meta)})
    finally:
        if was_lowered and lowering is not None:
            lowering.apply(model)


def load_quantized_model(model: nn.Module, path: str | Path, kernel_lowering: str | None = "auto") -> QuantizationManifest:
    """Load a checkpoint written by :func:`save_quantized_model` (or by the reference) into *model*.

    Regular tensors go through ``load_state_dict(strict=False)``; every quantized weight is rebuilt
    from its components and attached to its ``nn.Linear``; with ``kernel_lowering="auto"`` the
    model is then lowered (``AutoKernelLowering``).  Raises ``ValueError`` for a file without a
    manifest, with a quantized-weight type this backend has no container for, or with a
    ``mixed_precision_split`` transform (it changes the module tree; not replayed here).
    """
    from safetensors import safe_open

    if kernel_lowering not in ("auto", None):
        raise ValueError(f"kernel_lowering must be 'auto' or None, got {kernel_lowering!r}")
    with safe_open(str(path), framework="pt") as f:
        raw_meta = f.metadata() or {}
        all_tensors = {k: f.get_tensor(k) for k in f.keys()}
    manifest_str = raw_meta.get(_MANIFEST_META_KEY)
    if manifest_str is None:
        raise ValueError(
            f"File {str(path)!r} is missing the {_MANIFEST_META_KEY!r} metadata key.  "
            "Was it written by save_quantized_model()?"
        )
    manifest_dict = json.loads(manifest_str)
    manifest = QuantizationManifest(transforms=list(manifest_dict.get("transforms", [])))
    for t in manifest.transforms:
        kind = t.get("type")
        if kind == "mixed_precision_split":
            # The reference replays this one before load_state_dict (t2n/model_io.py:367-420): it
            # swaps nn.Linear modules for MixedPrecisionLinear ones whose sub-linears own the saved
            # tensors.  Loading without it would drop those tensors silently (strict=False).
            raise ValueError(
                f"File {str(path)!r} records a 'mixed_precision_split' transform, which replaces the "
                f"modules at {sorted(t.get('modules', {}))[:4]} ... by split mixed-precision linears; this "
                "backend has no such module, so the checkpoint cannot be loaded here."
            )
        if kind != "qtensor_assignment":
            _log.warning("load_quantized_model: transform %r is not replayed by this backend", kind)
    entries = manifest._assignment()

    regular = {k: v for k, v in all_tensors.items() if _QT_SEP not in k and k not in entries}
    model.load_state_dict(regular, strict=False)

    cache: dict[str, torch.Tensor] = {}
    for param_path, entry in entries.items():
        if entry["type"] not in _KNOWN_TYPES:
            raise ValueError(
                f"No QTensorSerde registered for type {entry['type']!r} (needed for parameter "
                f"{param_path!r}).  Available: {sorted(_KNOWN_TYPES)}"
            )
        module_path, _, attr = param_path.rpartition(".")
        module = model.get_submodule(module_path) if module_path else model
        if attr != "weight" or not isinstance(module, (nn.Linear, nn.Embedding)):
            raise ValueError(f"quantized parameter {param_path!r} is not the weight of an nn.Linear / nn.Embedding")
        device = next((t.device for t in list(module.parameters()) + list(module.buffers())
                       if t.device.type != "meta"), torch.device("cpu"))  # fmt: skip
        parts = {k: all_tensors[f"{param_path}{_QT_SEP}{k}"].to(device) for k in entry["tensor_keys"]}
        meta = {k: str(v) for k, v in entry["metadata"].items()}
        weight = _vq_from_parts(parts, meta, cache) if entry["type"] == "QTensorTractVQ" else _scalar_from_parts(parts, meta)
        attach_quantized_weight(module, weight)

    rc = manifest_dict.get("recipe_config")
    manifest.recipe_config_json = json.dumps(rc) if rc is not None else None
    model.__neuropress_manifest__ = manifest
    if kernel_lowering is not None:
        from ..kernel_lowering import AutoKernelLowering

        lowering = AutoKernelLowering()
        model.__neuropress_kernel_lowering__ = lowering
        lowering.apply(model)
    return manifest
