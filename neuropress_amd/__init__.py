"""neuropress_amd: MI355X (gfx950) backend for neuropress's quantized-linear forward path.

Drop-in for the reference's kernel-lowering API on that path:

    from neuropress_amd import AutoKernelLowering
    AutoKernelLowering().apply(model)        # swaps quantized nn.Linear for NPVQLinear / NPLinear

The modules call hand-written HIP kernels through the C ABI of
``libnpamd.so`` (``include/npamd.h``); build it with
``python -m neuropress_amd.build``.
"""

from .kernel_lowering import (  # noqa: F401
    AutoKernelLowering,
    KernelLowering,
    LoweringConfig,
    is_lowered,
    prepare_decode,
    unlower_model,
)
from .nn import (  # noqa: F401
    LinearBackend,
    NPLinear,
    NPVQLinear,
    VQBackend,
    VQProxy,
    linearize_qtensor_weights,
    linearize_vq_weights,
)



def save_quantized_model(model, path, recipe_config_json=None):
    """Write a (lowered or unlowered) quantized model to one safetensors file (``t2n.model_io``)."""
    from .t2n.model_io import save_quantized_model as _save

    return _save(model, path, recipe_config_json)


def load_quantized_model(model, path, kernel_lowering="auto"):
    """Load such a file into *model* and, by default, lower it (``t2n.model_io``)."""
    from .t2n.model_io import load_quantized_model as _load

    return _load(model, path, kernel_lowering)


__version__ = "0.1.0"
