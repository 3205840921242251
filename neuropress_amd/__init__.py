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

__version__ = "0.1.0"
