"""triton_kernels: the Flux transformer-block operator set, backed by hand-written HIP kernels for
MI355X (gfx950) in libfluxhip.so. The public names are those of the reference package
(triton_kernels/__init__.py:1-10); nothing here uses Triton."""
from triton_kernels.functional import (
    apply_rope_torch,
    apply_rope_torch_compile,
    layer_norm_modulation_torch,
    layer_norm_modulation_torch_compile,
    rms_norm_torch,
    rms_norm_torch_compile,
)
from triton_kernels.kernels import (
    apply_rope,
    attention_into,
    layer_norm_modulation,
    linear,
    linear_into,
    qkv_prep,
    rms_norm,
    scaled_dot_product_attention,
)
from triton_kernels.modules import DoubleStreamBlock, QKNorm, RMSNorm, SingleStreamBlock

__all__ = [
    "apply_rope_torch", "apply_rope_torch_compile", "layer_norm_modulation_torch",
    "layer_norm_modulation_torch_compile", "rms_norm_torch", "rms_norm_torch_compile",
    "apply_rope", "layer_norm_modulation", "linear", "rms_norm", "scaled_dot_product_attention",
    "attention_into", "linear_into", "qkv_prep",
    "DoubleStreamBlock", "QKNorm", "RMSNorm", "SingleStreamBlock",
]
