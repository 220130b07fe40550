"""Plain-PyTorch Flux transformer blocks: the un-accelerated statement of what the HIP-backed
modules compute. Structure follows black-forest-labs/flux as carried in flux/layers.py of the
reference (attention :11-17, rope :20-27, apply_rope :30-35, EmbedND :38-52, RMSNorm/QKNorm :88-109,
Modulation :138-151, DoubleStreamBlock :154-216, SingleStreamBlock :219-264). Only what the two
blocks need is here. Parameter names are the state-dict contract shared with triton_kernels.modules.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F
from torch import Tensor, nn


# ------------------------------------------------------------------------------------------------
# rotary position tables
# ------------------------------------------------------------------------------------------------
def rope(pos: Tensor, dim: int, theta: int) -> Tensor:
    """pos [..., n] -> [..., n, dim/2, 2, 2] rotation matrices [[cos, -sin], [sin, cos]] of the angle
    pos * theta^(-2j/dim), evaluated in float64 and returned as float32."""
    assert dim % 2 == 0
    exponent = torch.arange(0, dim, 2, dtype=torch.float64, device=pos.device) / dim
    freq = theta ** (-exponent)
    angle = pos.to(torch.float64).unsqueeze(-1) * freq
    c, s = torch.cos(angle), torch.sin(angle)
    mat = torch.stack((c, -s, s, c), dim=-1)
    return mat.unflatten(-1, (2, 2)).float()


class EmbedND(nn.Module):
    """Concatenate the rope tables of the id axes along the pair dimension: ids [B, L, n_axes] ->
    [B, 1, L, sum(axes_dim)/2, 2, 2]."""

    def __init__(self, dim: int, theta: int, axes_dim: list[int]):
        super().__init__()
        self.dim, self.theta, self.axes_dim = dim, theta, list(axes_dim)

    def forward(self, ids: Tensor) -> Tensor:
        tables = [rope(ids[..., axis], self.axes_dim[axis], self.theta) for axis in range(ids.shape[-1])]
        return torch.cat(tables, dim=-3).unsqueeze(1)


def apply_rope(xq: Tensor, xk: Tensor, freqs_cis: Tensor) -> tuple[Tensor, Tensor]:
    def rotate(x: Tensor) -> Tensor:
        pairs = x.float().unflatten(-1, (-1, 1, 2))
        return (freqs_cis[..., 0] * pairs[..., 0] + freqs_cis[..., 1] * pairs[..., 1]).flatten(-2).type_as(x)

    return rotate(xq), rotate(xk)


def attention(q: Tensor, k: Tensor, v: Tensor, pe: Tensor) -> Tensor:
    q, k = apply_rope(q, k, pe)
    o = F.scaled_dot_product_attention(q, k, v)          # [B, H, L, D]
    return o.transpose(1, 2).flatten(2)                    # [B, L, H*D]


def split_heads(qkv: Tensor, num_heads: int) -> tuple[Tensor, Tensor, Tensor]:
    """[B, L, 3*H*D] -> q, k, v each [B, H, L, D]."""
    B, L, _ = qkv.shape
    t = qkv.view(B, L, 3, num_heads, -1).permute(2, 0, 3, 1, 4)
    return t[0], t[1], t[2]


# ------------------------------------------------------------------------------------------------
# small modules
# ------------------------------------------------------------------------------------------------
class RMSNorm(nn.Module):
    def __init__(self, dim: int):
        super().__init__()
        self.scale = nn.Parameter(torch.ones(dim))

    def forward(self, x: Tensor) -> Tensor:
        xf = x.float()
        inv_rms = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + 1e-6)
        return (xf * inv_rms).to(x.dtype) * self.scale


class QKNorm(nn.Module):
    def __init__(self, dim: int):
        super().__init__()
        self.query_norm = RMSNorm(dim)
        self.key_norm = RMSNorm(dim)

    def forward(self, q: Tensor, k: Tensor, v: Tensor) -> tuple[Tensor, Tensor]:
        return self.query_norm(q).to(v), self.key_norm(k).to(v)


class SelfAttention(nn.Module):
    def __init__(self, dim: int, num_heads: int = 8, qkv_bias: bool = False):
        super().__init__()
        self.num_heads = num_heads
        self.qkv = nn.Linear(dim, dim * 3, bias=qkv_bias)
        self.norm = QKNorm(dim // num_heads)
        self.proj = nn.Linear(dim, dim)

    def forward(self, x: Tensor, pe: Tensor) -> Tensor:
        q, k, v = split_heads(self.qkv(x), self.num_heads)
        q, k = self.norm(q, k, v)
        return self.proj(attention(q, k, v, pe=pe))


@dataclass
class ModulationOut:
    shift: Tensor
    scale: Tensor
    gate: Tensor


class Modulation(nn.Module):
    def __init__(self, dim: int, double: bool):
        super().__init__()
        self.is_double = double
        self.multiplier = 6 if double else 3
        self.lin = nn.Linear(dim, self.multiplier * dim, bias=True)

    def forward(self, vec: Tensor) -> tuple[ModulationOut, ModulationOut | None]:
        chunks = self.lin(F.silu(vec))[:, None, :].chunk(self.multiplier, dim=-1)
        return ModulationOut(*chunks[:3]), (ModulationOut(*chunks[3:]) if self.is_double else None)


def _mlp(hidden_size: int, mlp_hidden_dim: int) -> nn.Sequential:
    return nn.Sequential(
        nn.Linear(hidden_size, mlp_hidden_dim, bias=True),
        nn.GELU(approximate="tanh"),
        nn.Linear(mlp_hidden_dim, hidden_size, bias=True),
    )


def _adaln(norm: nn.LayerNorm, x: Tensor, mod: ModulationOut) -> Tensor:
    return (1 + mod.scale) * norm(x) + mod.shift


# ------------------------------------------------------------------------------------------------
# blocks
# ------------------------------------------------------------------------------------------------
class DoubleStreamBlock(nn.Module):
    def __init__(self, hidden_size: int, num_heads: int, mlp_ratio: float, qkv_bias: bool = False):
        super().__init__()
        mlp_hidden_dim = int(hidden_size * mlp_ratio)
        self.num_heads = num_heads
        self.hidden_size = hidden_size
        for s in ("img", "txt"):
            setattr(self, f"{s}_mod", Modulation(hidden_size, double=True))
            setattr(self, f"{s}_norm1", nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6))
            setattr(self, f"{s}_attn", SelfAttention(dim=hidden_size, num_heads=num_heads, qkv_bias=qkv_bias))
            setattr(self, f"{s}_norm2", nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6))
            setattr(self, f"{s}_mlp", _mlp(hidden_size, mlp_hidden_dim))

    def _qkv(self, s: str, x: Tensor, mod1: ModulationOut):
        attn: SelfAttention = getattr(self, f"{s}_attn")
        q, k, v = split_heads(attn.qkv(_adaln(getattr(self, f"{s}_norm1"), x, mod1)), self.num_heads)
        q, k = attn.norm(q, k, v)
        return q, k, v

    def _tail(self, s: str, x: Tensor, attn_out: Tensor, mod1: ModulationOut, mod2: ModulationOut) -> Tensor:
        x = x + mod1.gate * getattr(self, f"{s}_attn").proj(attn_out)
        return x + mod2.gate * getattr(self, f"{s}_mlp")(_adaln(getattr(self, f"{s}_norm2"), x, mod2))

    def forward(self, img: Tensor, txt: Tensor, vec: Tensor, pe: Tensor) -> tuple[Tensor, Tensor]:
        img_mod1, img_mod2 = self.img_mod(vec)
        txt_mod1, txt_mod2 = self.txt_mod(vec)
        iq, ik, iv = self._qkv("img", img, img_mod1)
        tq, tk, tv = self._qkv("txt", txt, txt_mod1)
        joint = attention(torch.cat((tq, iq), dim=2), torch.cat((tk, ik), dim=2), torch.cat((tv, iv), dim=2), pe=pe)
        n_txt = txt.shape[1]
        img = self._tail("img", img, joint[:, n_txt:], img_mod1, img_mod2)
        txt = self._tail("txt", txt, joint[:, :n_txt], txt_mod1, txt_mod2)
        return img, txt


class SingleStreamBlock(nn.Module):
    """DiT block with parallel attention and MLP branches (https://arxiv.org/abs/2302.05442)."""

    def __init__(self, hidden_size: int, num_heads: int, mlp_ratio: float = 4.0, qk_scale: float | None = None):
        super().__init__()
        self.hidden_dim = hidden_size
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        head_dim = hidden_size // num_heads
        self.scale = qk_scale or head_dim**-0.5
        self.mlp_hidden_dim = int(hidden_size * mlp_ratio)
        self.linear1 = nn.Linear(hidden_size, hidden_size * 3 + self.mlp_hidden_dim)
        self.linear2 = nn.Linear(hidden_size + self.mlp_hidden_dim, hidden_size)
        self.norm = QKNorm(head_dim)
        self.pre_norm = nn.LayerNorm(hidden_size, elementwise_affine=False, eps=1e-6)
        self.mlp_act = nn.GELU(approximate="tanh")
        self.modulation = Modulation(hidden_size, double=False)

    def forward(self, x: Tensor, vec: Tensor, pe: Tensor) -> Tensor:
        mod, _ = self.modulation(vec)
        qkv, mlp = self.linear1(_adaln(self.pre_norm, x, mod)).split([3 * self.hidden_size, self.mlp_hidden_dim], dim=-1)
        q, k, v = split_heads(qkv, self.num_heads)
        q, k = self.norm(q, k, v)
        attn = attention(q, k, v, pe=pe)
        out = self.linear2(torch.cat((attn, self.mlp_act(mlp)), dim=2))
        return x + mod.gate * out
