"""Raw operator kernels under their reference names (triton_kernels/ops/*.py of the reference)."""
from triton_kernels.ops.linear import triton_linear
from triton_kernels.ops.modulation import triton_modulation_gate_proj, triton_modulation_scale_shift
from triton_kernels.ops.qkv_concat import triton_qkv_concat
from triton_kernels.ops.silu import triton_silu

__all__ = [
    "triton_linear", "triton_modulation_gate_proj", "triton_modulation_scale_shift", "triton_qkv_concat", "triton_silu",
]
