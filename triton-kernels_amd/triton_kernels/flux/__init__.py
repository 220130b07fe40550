from triton_kernels.flux.layers import DoubleStreamBlock, EmbedND, SingleStreamBlock, apply_rope, rope

__all__ = ["DoubleStreamBlock", "EmbedND", "SingleStreamBlock", "apply_rope", "rope"]
