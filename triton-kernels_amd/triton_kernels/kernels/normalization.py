"""rms_norm and layer_norm_modulation: Python launchers over the HIP row-wise kernels.

Same call signatures, defaults and assertion behaviour as kernels/normalization.py:47-77 and
:142-193 of the reference; the device work is flux_rms_norm / flux_rms_norm_bwd /
flux_layer_norm_modulation in libfluxhip.so.
"""
from __future__ import annotations

import torch

from triton_kernels import _native as nv
from triton_kernels.kernels.utils import calculate_settings


def _as_4d_view(x: torch.Tensor):
    """Sizes (d0,d1,d2) and strides (s0,s1,s2) of x seen as [d0,d1,d2,n] rows, without copying when x
    has at most four dims and a contiguous last dim; otherwise a contiguous copy is described."""
    if x.dim() == 0:
        raise AssertionError("rms_norm needs at least one dimension")
    if x.dim() > 4 or x.stride(-1) != 1:
        x = x.contiguous()
        if x.dim() > 4:
            x = x.reshape(-1, x.shape[-1])
    lead = list(x.shape[:-1])
    strides = list(x.stride()[:-1])
    while len(lead) < 3:
        lead.insert(0, 1)
        strides.insert(0, 0)
    return x, lead, strides


def rms_norm_forward(x: torch.Tensor, scale: torch.Tensor, eps: float = 1e-6, want_rstd: bool = False):
    assert x.shape[-1] == scale.shape[-1]
    dev = nv.require_gpu(x, scale)
    n = x.shape[-1]
    calculate_settings(n)  # raises for rows wider than 65536, like the reference
    scale = scale.contiguous()
    if scale.dtype != x.dtype and not (x.dtype == torch.bfloat16 and scale.dtype == torch.float32):
        scale = scale.to(x.dtype)
    xv, lead, strides = _as_4d_view(x)
    y = torch.empty(x.shape, dtype=x.dtype, device=dev)
    rows = lead[0] * lead[1] * lead[2]
    rstd = torch.empty((rows,), dtype=torch.float32, device=dev) if want_rstd else None
    with nv.on_device(dev):
        rc = nv.lib().flux_rms_norm(
            xv.data_ptr(), scale.data_ptr(), y.data_ptr(), nv.ptr(rstd),
            lead[0], lead[1], lead[2], n, strides[0], strides[1], strides[2],
            nv.dtype_code(x), nv.dtype_code(scale), float(eps), nv.stream_ptr(dev))
    nv.check(rc, "flux_rms_norm")
    return y, rstd, xv


class _rms_norm(torch.autograd.Function):
    """y = x * rsqrt(mean(x^2, -1) + eps) * scale with a HIP forward and backward."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, scale: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
        need_grad = x.requires_grad or scale.requires_grad
        if need_grad:
            x = x.contiguous()
        y, rstd, _ = rms_norm_forward(x, scale, eps, want_rstd=need_grad)
        if need_grad:
            ctx.save_for_backward(x.reshape(-1, x.shape[-1]), scale.contiguous(), rstd)
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        x2, scale, rstd = ctx.saved_tensors
        dev = nv.require_gpu(dy, x2)
        rows, n = x2.shape
        dy2 = dy.contiguous().reshape(rows, n)
        if dy2.dtype != x2.dtype:
            dy2 = dy2.to(x2.dtype)
        sc = scale
        if sc.dtype != x2.dtype and not (x2.dtype == torch.bfloat16 and sc.dtype == torch.float32):
            sc = sc.to(x2.dtype)
        dx = torch.empty_like(x2)
        dscale = torch.zeros((n,), dtype=torch.float32, device=dev)
        with nv.on_device(dev):
            rc = nv.lib().flux_rms_norm_bwd(
                dy2.data_ptr(), x2.data_ptr(), sc.data_ptr(), rstd.data_ptr(), dx.data_ptr(), dscale.data_ptr(),
                rows, n, nv.dtype_code(x2), nv.dtype_code(sc), nv.stream_ptr(dev))
        nv.check(rc, "flux_rms_norm_bwd")
        return dx.reshape(dy.shape), dscale.to(scale.dtype).reshape(scale.shape), None


rms_norm = _rms_norm.apply


def layer_norm_modulation(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps=1e-5) -> torch.Tensor:
    """(1 + weight) * layer_norm(x) + bias, where weight is the adaLN *scale* and bias the *shift*,
    each [B, 1, N] (or [B, N]); chunks of a wider modulation tensor are read in place."""
    assert x.shape[0] == weight.shape[0] == bias.shape[0]
    assert x.shape[-1] == weight.shape[-1] == bias.shape[-1]
    dev = nv.require_gpu(x, weight, bias)
    batch, n = x.shape[0], x.shape[-1]
    calculate_settings(n)
    x = x.contiguous()
    if weight.dtype != x.dtype:
        weight = weight.to(x.dtype)
    if bias.dtype != x.dtype:
        bias = bias.to(x.dtype)
    assert weight.numel() == batch * n and bias.numel() == batch * n, "scale/shift must be [B, 1, N]"
    in_place = weight.stride(-1) == 1 and bias.stride(-1) == 1 and (batch == 1 or weight.stride(0) == bias.stride(0))
    if not in_place:
        weight, bias = weight.contiguous(), bias.contiguous()
    mod_stride = weight.stride(0) if batch > 1 else n
    if batch > 1 and mod_stride < n:
        weight, bias = weight.contiguous(), bias.contiguous()
        mod_stride = weight.stride(0)
    y = torch.empty_like(x)
    rows = x.numel() // n
    with nv.on_device(dev):
        rc = nv.lib().flux_layer_norm_modulation(
            x.data_ptr(), weight.data_ptr(), bias.data_ptr(), y.data_ptr(),
            batch, rows // batch if batch else 0, n, mod_stride, nv.dtype_code(x), float(eps), nv.stream_ptr(dev))
    nv.check(rc, "flux_layer_norm_modulation")
    return y
