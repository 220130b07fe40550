"""Plain-PyTorch statements of the two norm ops, in the rounding order PyTorch itself produces on
bf16 tensors. These are the functions the reference's tests compare its kernels with
(functional/normalization.py:6-25); the *_compile names are kept as aliases and never invoke a
compiler, since nothing on this path may generate GPU code at run time."""
import torch
import torch.nn.functional as F
from torch import Tensor


def modulate(x: Tensor, scale: Tensor, shift: Tensor) -> Tensor:
    return shift + (scale + 1) * x


def layer_norm_modulation_torch(x: Tensor, scale: Tensor, shift: Tensor) -> Tensor:
    normed = F.layer_norm(x, (x.shape[-1],))
    return modulate(normed, scale=scale, shift=shift)


def rms_norm_torch(x: Tensor, scale: Tensor) -> Tensor:
    xf = x.float()
    inv_rms = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + 1e-6)
    return (xf * inv_rms).to(x.dtype) * scale


layer_norm_modulation_torch_compile = layer_norm_modulation_torch
rms_norm_torch_compile = rms_norm_torch
