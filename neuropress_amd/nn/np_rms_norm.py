"""NPRMSNorm: RMSNorm as one HIP kernel, and the pass that installs it.

Same module surface and detection rules as the reference
(neuropress/nn/np_rms_norm.py:42-208): any module whose class name contains
"RMSNorm", with exactly one 1-D parameter ``weight`` and an ``eps`` attribute,
on a GPU, is replaced.  Models differ in how the weight enters
(``x_normed * weight`` or ``x_normed * (1 + weight)``); which one a module uses
is found by running it once with a zeroed weight, and the "+1" is folded into
the weight handed to the kernel.
"""

from __future__ import annotations

import logging

import torch
from torch import nn

__all__ = ["NPRMSNorm", "linearize_rms_norms"]

log = logging.getLogger(__name__)


class NPRMSNorm(nn.Module):
    """``x * rsqrt(mean(x^2, -1) + eps) * weight`` in f32 arithmetic, rounded once."""

    def __init__(self, weight: torch.Tensor, eps: float = 1e-6, source: nn.Module | None = None) -> None:
        super().__init__()
        self.register_buffer("weight", weight.clone())
        self.eps = eps
        self.__dict__["_source"] = source  # outside the module tree: no state_dict entries

    def to_source_module(self) -> nn.Module | None:
        """The module this one replaced (its own weight untouched), on this module's device."""
        source = self.__dict__.get("_source")
        return None if source is None else source.to(self.weight.device)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        *leading, h = x.shape
        w = self.weight if self.weight.dtype == x.dtype else self.weight.to(x.dtype)
        if x.is_cuda:
            from .. import kernels

            return kernels.rms_norm(x.reshape(-1, h), w, self.eps).reshape(*leading, h)
        xf = x.float()  # specification of the kernel, for tensors that are not on a GPU
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps) * w.float()).to(x.dtype)

    def extra_repr(self) -> str:
        return f"H={self.weight.shape[0]}, eps={self.eps}"


def _is_unfused_rms_norm(module: nn.Module) -> bool:
    if isinstance(module, NPRMSNorm) or "RMSNorm" not in type(module).__name__:
        return False
    params = dict(module.named_parameters(recurse=False))
    return set(params) == {"weight"} and params["weight"].dim() == 1 and hasattr(module, "eps")


def _uses_plus_one_convention(module: nn.Module, weight: torch.Tensor) -> bool:
    """True when *module* computes ``x_normed * (1 + weight)``: with the weight zeroed such a module
    still returns the normalized probe, a plain-weight module returns zeros."""
    probe = torch.randn(1, weight.shape[0], device=weight.device, dtype=weight.dtype)
    saved = weight.clone()
    try:
        weight.zero_()
        with torch.no_grad():
            out = module(probe)
    finally:
        weight.copy_(saved)
    return bool(out.float().abs().max().item() > 1e-3)


def linearize_rms_norms(model: nn.Module) -> int:
    """Replace every unfused RMSNorm of *model* that lives on a GPU; returns how many."""
    from .backends import is_hip_backend_available

    if not is_hip_backend_available():
        log.debug("linearize_rms_norms: HIP kernel library unavailable - skipping")
        return 0
    targets = [
        (name, mod)
        for name, mod in model.named_modules()
        if _is_unfused_rms_norm(mod) and next(mod.parameters()).device.type == "cuda"
    ]
    plus_one = 0
    for name, mod in targets:
        weight = next(mod.parameters()).data
        if _uses_plus_one_convention(mod, weight):
            effective = 1.0 + weight
            plus_one += 1
        else:
            effective = weight.clone()
        fused = NPRMSNorm(effective, eps=float(mod.eps), source=mod).to(weight.device, weight.dtype)
        parent_name, _, attr = name.rpartition(".")
        setattr(model.get_submodule(parent_name) if parent_name else model, attr, fused)
    if targets:
        log.debug("linearize_rms_norms: replaced %d module(s) (%d used the '+1' convention)", len(targets), plus_one)
    return len(targets)
