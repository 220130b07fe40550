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
