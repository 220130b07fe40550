from triton_kernels.modules.blocks import (
    MLP,
    DoubleStreamBlock,
    Linear,
    LinearGELU,
    Modulation,
    ModulationOut,
    SelfAttention,
    SingleStreamBlock,
    attention,
)
from triton_kernels.modules.normalization import QKNorm, RMSNorm

__all__ = [
    "MLP", "DoubleStreamBlock", "Linear", "LinearGELU", "Modulation", "ModulationOut", "SelfAttention",
    "SingleStreamBlock", "attention", "QKNorm", "RMSNorm",
]
