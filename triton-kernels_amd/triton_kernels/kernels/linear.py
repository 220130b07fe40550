"""linear: y = act(x @ w.T + b) on the bf16 matrix cores (kernels/linear.py:104-151 of the reference),
with the extra epilogues the fused Flux blocks use."""
from __future__ import annotations

import ctypes

import torch
from torch import Tensor

from triton_kernels import _native as nv

_ACTIVATIONS = {"": nv.ACT_NONE, "GELU": nv.ACT_GELU_TANH}
# Tile plan per dtype; like the reference's table it has a single entry, so any other dtype is a KeyError.
_PLANS = {torch.bfloat16: {"tile": (256, 256, 64), "waves": 4, "mfma": "16x16x32"}}


# Optional callable(dict) invoked with the metadata of every launch of the linear kernel, on the launching
# thread, right before the launch. Profilers and benchmarks set it (e.g. to open a named range); None
# costs nothing. The dictionary is what the reference attaches to its launches for its profiler
# (kernels/linear.py:9-19): "name" with the problem size, "flops16" = 2 M N K and "bytes" = the three
# matrices once.
launch_hook = None


def linear_launch_metadata(M: int, N: int, K: int, elem_bytes: int = 2, epilogue: str = "") -> dict:
    name = f"flux_linear_bf16 [M={M}, N={N}, K={K}]" + (f" {epilogue}" if epilogue else "")
    return {"name": name, f"flops{elem_bytes * 8}": 2.0 * M * N * K, "bytes": elem_bytes * (M * K + N * K + M * N)}


def _rows_2d(x: Tensor, K: int) -> Tensor:
    x2 = x.reshape(-1, K)
    if x2.shape[0] > 1 and (x2.stride(1) != 1 or x2.stride(0) < K):
        x2 = x2.contiguous()
    elif x2.shape[0] <= 1 and x2.stride(1) != 1:
        x2 = x2.contiguous()
    return x2


def linear_into(x: Tensor, w: Tensor, b: Tensor | None, *, activation: str = "", act_begin: int = 0,
                out: Tensor | None = None, out2: Tensor | None = None, split: int | None = None,
                resid: Tensor | None = None, gate: Tensor | None = None, qk: dict | None = None,
                in_activation: str = "", shared_gpu: bool = False) -> Tensor:
    """General form of the fused linear.

    out   : [M, >=split] destination (row stride free) for columns [0, split)
    out2  : destination for columns [split, N), written starting at its column 0
    act_begin : GELU applies to columns >= act_begin only
    resid, gate : y = resid + gate * y with resid [..., N] and gate [B, 1, N] (or [B, N])
    in_activation : "SiLU" applies x * sigmoid(x) (rounded to bf16) to x on the way in; at most 8 rows
    qk    : QK RMSNorm + RoPE on the way out for the leading 2 * heads * 128 columns (q heads, then k
            heads), which then go to q_out / k_out [B, heads, out_len, 128] instead of `out`:
            dict(q_out, k_out, q_scale, k_scale, pe, heads, seq_len, pos0=0, eps=1e-6); see
            qk_fusable() for the shapes this form takes
    shared_gpu : the launch runs beside another stream's work; the library then keeps a tile shape
            that leaves CUs free in its last round instead of one that fills the GPU exactly (same
            result, only the schedule differs)
    """
    assert x.shape[-1] == w.shape[-1], "Incompatible dimensions"
    assert x.dtype == w.dtype, "Incompatible dtypes"
    _PLANS[x.dtype]  # KeyError for anything but bfloat16, as in the reference
    act = _ACTIVATIONS[activation]
    dev = nv.require_gpu(x, w, b, out, out2, resid, gate)
    N, K = w.shape
    x2 = _rows_2d(x, K)
    M = x2.shape[0]
    if w.stride(1) != 1 or (N > 1 and w.stride(0) < K):
        w = w.contiguous()
    if b is not None:
        assert b.shape[-1] == N
        b = b.to(x.dtype).contiguous()
    a = nv.LinearArgs()
    a.A, a.W, a.bias = x2.data_ptr(), w.data_ptr(), nv.ptr(b)
    a.M, a.N, a.K = M, N, K
    a.lda = x2.stride(0) if M > 1 else K
    a.ldw = w.stride(0) if N > 1 else K
    if out is None:
        out = torch.empty((M, N if split is None else split), device=dev, dtype=x.dtype)
    assert out.dim() == 2 and out.shape[0] == M and out.stride(1) == 1 and out.dtype == x.dtype
    a.Y, a.ldy = out.data_ptr(), out.stride(0)
    if split is not None and split < N:
        assert out2 is not None and out2.dim() == 2 and out2.shape[0] == M and out2.stride(1) == 1
        assert out.shape[1] >= split and out2.shape[1] >= N - split and out2.dtype == x.dtype
        a.Y2, a.ldy2, a.split_n, a.y2_col0 = out2.data_ptr(), out2.stride(0), split, 0
    else:
        assert out.shape[1] >= N
        a.Y2, a.split_n = None, N
    if gate is not None:
        assert resid is not None
        r2 = resid.reshape(-1, N)
        assert r2.shape[0] == M and r2.stride(1) == 1 and r2.dtype == x.dtype
        g2 = gate.reshape(-1, N) if gate.is_contiguous() else gate.reshape(gate.shape[0], N)
        if g2.dtype != x.dtype:
            g2 = g2.to(x.dtype)
        if g2.stride(1) != 1:
            g2 = g2.contiguous()
        nb = g2.shape[0]
        assert M % nb == 0
        a.resid, a.ldresid = r2.data_ptr(), r2.stride(0)
        a.gate, a.gate_batch_stride, a.rows_per_batch = g2.data_ptr(), (g2.stride(0) if nb > 1 else N), M // nb
    a.act, a.act_begin = act, act_begin
    a.flags = nv.LINEAR_SHARED_GPU if shared_gpu else 0
    a.in_act = {"": nv.ACT_NONE, "SiLU": nv.ACT_SILU}[in_activation]
    assert a.in_act == nv.ACT_NONE or M <= 8, "the input activation is fused for at most 8 rows"
    keep = None
    if qk is not None:
        f = nv.LinearQKFusion()
        q_out, k_out, pe = qk["q_out"], qk["k_out"], qk["pe"]
        heads, seq_len = int(qk["heads"]), int(qk["seq_len"])
        assert q_out.is_contiguous() and k_out.is_contiguous() and q_out.shape == k_out.shape and q_out.dtype == x.dtype
        assert q_out.dim() == 4 and q_out.shape[1] == heads and q_out.shape[3] == 128 and M % seq_len == 0 and q_out.shape[0] == M // seq_len
        out_len = q_out.shape[2]
        pe2 = pe.reshape(-1, out_len, 64, 2, 2)
        assert pe2.dtype == torch.float32 and pe2.is_contiguous()
        qs, ks = qk["q_scale"].to(x.dtype).contiguous(), qk["k_scale"].to(x.dtype).contiguous()
        f.q_out, f.k_out, f.q_scale, f.k_scale = q_out.data_ptr(), k_out.data_ptr(), qs.data_ptr(), ks.data_ptr()
        f.pe, f.pe_batch_stride = pe2.data_ptr(), (pe2.stride(0) if pe2.shape[0] > 1 else 0)
        f.heads, f.seq_len, f.out_len, f.pos0 = heads, seq_len, out_len, int(qk.get("pos0", 0))
        f.eps = float(qk.get("eps", 1e-6))
        a.qk = ctypes.pointer(f)
        keep = (f, qs, ks, pe2)
    if launch_hook is not None:
        parts = [activation and f"{activation}>={act_begin}", split is not None and f"split@{split}", gate is not None and "gated-residual",
                 qk is not None and "qk-norm-rope", in_activation and f"in:{in_activation}"]
        launch_hook(linear_launch_metadata(M, N, K, x.element_size(), "+".join(p for p in parts if p)))
    with nv.on_device(dev):
        rc = nv.lib().flux_linear_bf16(nv.byref(a), nv.stream_ptr(dev))
    nv.check(rc, "flux_linear_bf16")
    del keep
    return out


def qk_fusable(x: Tensor, w: Tensor, seq_len: int, head_dim: int) -> bool:
    """Whether linear_into(..., qk=...) takes this projection and is worth it: bf16, heads of 128,
    columns in multiples of the 256-wide tile, sequences of at least one tile (a tile then holds rows
    of at most two batch elements; ragged row counts and sequence lengths are fine), and enough
    tiles that the library would pick the 256-wide ones anyway (the fused epilogue exists for them only)."""
    M = x.numel() // x.shape[-1]
    N = w.shape[0]
    return (x.dtype == torch.bfloat16 and head_dim == 128 and seq_len >= 256 and M % seq_len == 0
            and N % 256 == 0 and w.shape[1] % 8 == 0 and -(-M // 256) * (N // 256) >= 160)


def linear(x: Tensor, w: Tensor, b: Tensor | None, activation: str = "", shared_gpu: bool = False) -> Tensor:
    N = w.shape[0]
    y = linear_into(x, w, b, activation=activation, shared_gpu=shared_gpu)
    return y.reshape(*x.shape[:-1], N)
