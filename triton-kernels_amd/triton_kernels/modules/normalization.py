"""RMSNorm / QKNorm modules on the HIP rms_norm (modules/normalization.py:8-26 of the reference).
Parameter names (`scale`, `query_norm`, `key_norm`) are part of the state-dict contract."""
import torch
from torch import Tensor, nn

from triton_kernels.kernels.normalization import rms_norm


class RMSNorm(nn.Module):
    def __init__(self, dim: int) -> None:
        super().__init__()
        self.scale = nn.Parameter(torch.ones(dim))

    def forward(self, x: Tensor) -> Tensor:
        return rms_norm(x, self.scale)


class QKNorm(nn.Module):
    def __init__(self, dim: int) -> None:
        super().__init__()
        self.query_norm = RMSNorm(dim)
        self.key_norm = RMSNorm(dim)

    def forward(self, q: Tensor, k: Tensor, v: Tensor) -> tuple[Tensor, Tensor]:
        return self.query_norm(q).to(v), self.key_norm(k).to(v)
