"""scaled_dot_product_attention: non-causal flash-attention forward (kernels/attention.py:173-221 of
the reference) on the HIP kernel flux_attention_fwd_bf16."""
from __future__ import annotations

import math

import torch
from torch import Tensor

from triton_kernels import _native as nv


def _bhld_view(t: Tensor) -> Tensor:
    if t.stride(-1) != 1 or any(s % 8 for s in t.stride()[:-1]) or t.data_ptr() % 16:
        t = t.contiguous()
    return t


def attention_into(q: Tensor, k: Tensor, v: Tensor, out: Tensor, sm_scale: float | None = None,
                   lse: Tensor | None = None) -> Tensor:
    """q,k,v,out are [B,H,L,D] views (bf16, last dim contiguous, any other strides)."""
    D = q.shape[-1]
    assert D == k.shape[-1] == v.shape[-1]
    assert D in {16, 32, 64, 128, 256}
    assert q.dim() == 4 and q.shape == k.shape == v.shape == out.shape
    if q.dtype != torch.bfloat16 or k.dtype != q.dtype or v.dtype != q.dtype or out.dtype != q.dtype:
        raise TypeError("scaled_dot_product_attention: the HIP kernel takes bfloat16 q, k, v")
    dev = nv.require_gpu(q, k, v, out, lse)
    if sm_scale is None:
        sm_scale = 1 / math.sqrt(D)
    q, k, v = _bhld_view(q), _bhld_view(k), _bhld_view(v)
    B, H, L, _ = q.shape
    a = nv.AttnArgs()
    a.q, a.k, a.v = nv.src4(q), nv.src4(k), nv.src4(v)
    a.o, a.o_sb, a.o_sh, a.o_sl = out.data_ptr(), out.stride(0), out.stride(1), out.stride(2)
    assert out.stride(3) == 1
    a.lse = nv.ptr(lse)
    a.B, a.H, a.L, a.D, a.sm_scale = B, H, L, D, float(sm_scale)
    with nv.on_device(dev):
        rc = nv.lib().flux_attention_fwd_bf16(nv.byref(a), nv.stream_ptr(dev))
    nv.check(rc, "flux_attention_fwd_bf16")
    return out


def scaled_dot_product_attention(q: Tensor, k: Tensor, v: Tensor, sm_scale: float = None) -> Tensor:
    o = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    return attention_into(q, k, v, o, sm_scale)
