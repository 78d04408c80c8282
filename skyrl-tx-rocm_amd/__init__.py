"""MI355X-native W8A8 LoRA linear forward path (gfx950 HIP kernels behind a C ABI).

The directory name carries a hyphen, so the package is imported through
``__graft_entry__.load_package()`` (or any ``importlib`` spec loader) under the
module name ``skyrl_tx_rocm_amd``.
"""

from . import _native  # noqa: F401
from .kernels import quantized_lora  # noqa: F401
from .kernels import bounded_lora  # noqa: F401
from .kernels.rocm import w8a8_lora  # noqa: F401
from .kernels.rocm import bf16_lora_residual, bf16_rms_gate_up_lora_swiglu_contiguous  # noqa: F401
from .kernels.rocm import gq_linear  # noqa: F401
from .layers import lora  # noqa: F401

__all__ = ["_native", "quantized_lora", "bounded_lora", "w8a8_lora", "gq_linear", "lora"]
