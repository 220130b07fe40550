"""Seeded synthetic inputs for the five Flux-shaped workloads the kernels are measured on.

Everything is drawn on the CPU in float32 from torch.Generator().manual_seed(1000 + config), cast to
bfloat16 and only then moved to `device`, so a CPU reference and the GPU kernels see the same bits.
"""
from __future__ import annotations

import math

import torch

from triton_kernels.flux.layers import EmbedND

H, D, HID, MLP = 24, 128, 3072, 12288
L_TXT, GRID = 512, 64
L_IMG = GRID * GRID
L = L_TXT + L_IMG


def _gen(config: int) -> torch.Generator:
    return torch.Generator().manual_seed(1000 + config)


def _normal(g, shape, std=1.0, dtype=torch.bfloat16):
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)


def flux_position_ids(n_txt: int = L_TXT, grid: int = GRID) -> torch.Tensor:
    """zeros for the text tokens, (0, h, w) on a grid x grid raster for the image tokens."""
    ids = torch.zeros(1, n_txt + grid * grid, 3)
    r = torch.arange(grid, dtype=torch.float32)
    ids[0, n_txt:, 1] = r.repeat_interleave(grid)
    ids[0, n_txt:, 2] = r.repeat(grid)
    return ids


def flux_pe(n_txt: int = L_TXT, grid: int = GRID, head_dim: int = D) -> torch.Tensor:
    """fp32 [1, 1, n_txt + grid^2, head_dim/2, 2, 2], EmbedND with axes (16, 56, 56) scaled to head_dim = 128."""
    assert head_dim == 128
    return EmbedND(dim=head_dim, theta=10000, axes_dim=[16, 56, 56])(flux_position_ids(n_txt, grid))


def config1(device="cpu", scale: float = 1.0):
    """QK RMSNorm: x [1,24,L,128] ~ N(0,1), scale [128] ~ U(0.5,1.5)."""
    g = _gen(1)
    x = _normal(g, (1, H, int(L * scale), D))
    w = (torch.rand((D,), generator=g, dtype=torch.float32) + 0.5).to(torch.bfloat16)
    return x.to(device), w.to(device)


def config2(device="cpu", scale: float = 1.0):
    """LayerNorm + modulation: x [1,L,3072] ~ N(0,1); shift, scale [1,1,3072] ~ N(0,0.1)."""
    g = _gen(2)
    x = _normal(g, (1, int(L * scale), HID))
    shift = _normal(g, (1, 1, HID), 0.1)
    sc = _normal(g, (1, 1, HID), 0.1)
    return x.to(device), sc.to(device), shift.to(device)


def config3(device="cpu", n_txt: int = L_TXT, grid: int = GRID):
    """RoPE + concat: txt q,k,v [1,24,n_txt,128], img q,k,v [1,24,grid^2,128] ~ N(0,1); pe from EmbedND."""
    g = _gen(3)
    txt = [_normal(g, (1, H, n_txt, D)).to(device) for _ in range(3)]
    img = [_normal(g, (1, H, grid * grid, D)).to(device) for _ in range(3)]
    return txt, img, flux_pe(n_txt, grid).to(device)


def config4(device="cpu", which: str = "mlp_in", m: int = L):
    """Linear: mlp_in A [m,3072] W [12288,3072] b [12288] (GELU); proj_out A [m,15360] W [3072,15360] b [3072]."""
    g = _gen(4)
    if which == "mlp_in":
        k, n = HID, MLP
    elif which == "proj_out":
        k, n = HID + MLP, HID
        g = torch.Generator().manual_seed(1004 + 100)
    elif which == "linear1":
        k, n = HID, 3 * HID + MLP
        g = torch.Generator().manual_seed(1004 + 200)
    else:
        raise ValueError(which)
    a = _normal(g, (m, k))
    w = _normal(g, (n, k), 1.0 / math.sqrt(k))
    b = _normal(g, (n,), 0.02)
    return a.to(device), w.to(device), b.to(device)


def config5_attention(device="cpu", seq: int = L):
    g = _gen(5)
    return tuple(_normal(g, (1, H, seq, D)).to(device) for _ in range(3))


def config5_block(device="cpu", n_txt: int = L_TXT, grid: int = GRID, hidden: int = HID, heads: int = H):
    """Single-stream block inputs and a state dict: x ~ N(0,1), vec ~ N(0,1), weights ~ N(0, 1/fan_in),
    biases ~ N(0, 0.02), RMSNorm scales = 1."""
    g = torch.Generator().manual_seed(1005 + 100)
    seq = n_txt + grid * grid
    mlp = 4 * hidden
    x = _normal(g, (1, seq, hidden))
    vec = _normal(g, (1, hidden))
    sd = {
        "modulation.lin.weight": _normal(g, (3 * hidden, hidden), hidden ** -0.5),
        "modulation.lin.bias": _normal(g, (3 * hidden,), 0.02),
        "linear1.weight": _normal(g, (3 * hidden + mlp, hidden), hidden ** -0.5),
        "linear1.bias": _normal(g, (3 * hidden + mlp,), 0.02),
        "linear2.weight": _normal(g, (hidden, hidden + mlp), (hidden + mlp) ** -0.5),
        "linear2.bias": _normal(g, (hidden,), 0.02),
        "norm.query_norm.scale": torch.ones(hidden // heads, dtype=torch.bfloat16),
        "norm.key_norm.scale": torch.ones(hidden // heads, dtype=torch.bfloat16),
    }
    pe = flux_pe(n_txt, grid, hidden // heads)
    return x.to(device), vec.to(device), pe.to(device), {k: v.to(device) for k, v in sd.items()}
