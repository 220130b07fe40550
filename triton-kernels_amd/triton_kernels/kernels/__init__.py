"""Operator entry points: thin Python launchers over the C ABI of libfluxhip.so."""
from triton_kernels.kernels.normalization import layer_norm_modulation, rms_norm
from triton_kernels.kernels.positional_embedding import apply_rope, qkv_prep
from triton_kernels.kernels.linear import linear, linear_into, qk_fusable
from triton_kernels.kernels.attention import attention_into, scaled_dot_product_attention

__all__ = [
    "apply_rope", "layer_norm_modulation", "linear", "rms_norm", "scaled_dot_product_attention",
    "qkv_prep", "linear_into", "attention_into",
]
