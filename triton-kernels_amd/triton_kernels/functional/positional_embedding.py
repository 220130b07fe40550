"""Plain-PyTorch RoPE application (functional/positional_embedding.py:5-10 of the reference): every
adjacent pair (x[2i], x[2i+1]) is multiplied by the 2x2 matrix freqs_cis[..., i, :, :]."""
from torch import Tensor


def _rotate(x: Tensor, freqs_cis: Tensor) -> Tensor:
    pairs = x.float().unflatten(-1, (-1, 1, 2))          # [..., D/2, 1, 2]
    out = freqs_cis[..., 0] * pairs[..., 0] + freqs_cis[..., 1] * pairs[..., 1]
    return out.flatten(-2).type_as(x)


def apply_rope_torch(xq: Tensor, xk: Tensor, freqs_cis: Tensor) -> tuple[Tensor, Tensor]:
    return _rotate(xq, freqs_cis), _rotate(xk, freqs_cis)


apply_rope_torch_compile = apply_rope_torch
