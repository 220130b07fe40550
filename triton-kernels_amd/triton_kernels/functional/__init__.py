from triton_kernels.functional.normalization import (
    layer_norm_modulation_torch,
    layer_norm_modulation_torch_compile,
    modulate,
    rms_norm_torch,
    rms_norm_torch_compile,
)
from triton_kernels.functional.positional_embedding import apply_rope_torch, apply_rope_torch_compile

__all__ = [
    "apply_rope_torch", "apply_rope_torch_compile", "layer_norm_modulation_torch",
    "layer_norm_modulation_torch_compile", "modulate", "rms_norm_torch", "rms_norm_torch_compile",
]
