"""Helpers shared by the GPU parity tests."""
import torch

DEV = "cuda"


def seeded(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def randn(g, *shape, dtype=torch.float32, std=1.0):
    return (torch.randn(*shape, generator=g, dtype=torch.float32) * std).to(dtype)


def report(name: str, got: torch.Tensor, want: torch.Tensor) -> str:
    d = (got.float() - want.float()).abs()
    return f"{name}: max_abs={d.max().item():.3e} mean_abs={d.mean().item():.3e}"


def load_golden(name: str = "flux_small.npz") -> dict:
    """tests/golden/<name> as a dict of tensors: "<key>.bf16" entries (uint16 bit patterns) come back
    as bfloat16 tensors, "<key>.f32" entries as float32."""
    import os

    import numpy as np

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name)
    out = {}
    with np.load(path, allow_pickle=False) as z:
        for k in z.files:
            a = z[k]
            if k.endswith(".bf16"):
                out[k[:-5]] = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
            else:
                out[k[:-4]] = torch.from_numpy(a.copy())
    return out
