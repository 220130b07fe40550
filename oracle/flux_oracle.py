"""CPU oracle for the Flux block kernel path.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain PyTorch (CPU or whatever device the inputs live on), the functions the
reference's own tests use as ground truth, plus fp32/fp64 textbook forms for the two contractions.
Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import it; the
product package (triton-kernels_amd/triton_kernels) never does and has no CPU path.

Each function cites the reference lines it follows (paths relative to the reference repository).
How each one is pinned (tests/test_oracle_pins.py): closed forms evaluated in float64 with numpy,
invariants of the mathematics, special cases that reduce to a torch library routine, and brute
force on tiny inputs. The reference holds no golden vectors or seeds for this path, so there is
nothing stored to compare with; every function below has at least one such pin, none is
"parity unpinned".
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F
from torch import Tensor


# --------------------------------------------------------------------------------------------------
# row-wise ops
# --------------------------------------------------------------------------------------------------
def rms_norm_ref(x: Tensor, scale: Tensor, eps: float = 1e-6) -> Tensor:
    """functional/normalization.py:21-25 (== flux/layers.py:88-97): statistics in fp32, the normalised
    value cast back to x.dtype BEFORE the multiply by scale."""
    xf = x.float()
    rrms = torch.rsqrt(torch.mean(xf * xf, dim=-1, keepdim=True) + eps)
    return (xf * rrms).to(x.dtype) * scale


def rms_norm_bwd_ref(x: Tensor, scale: Tensor, dy: Tensor, eps: float = 1e-6) -> tuple[Tensor, Tensor]:
    """Gradients of rms_norm_ref by autograd, what tests/test_rms_norm.py:25-36 compares with."""
    x = x.detach().clone().requires_grad_(True)
    scale = scale.detach().clone().requires_grad_(True)
    rms_norm_ref(x, scale, eps).backward(dy)
    return x.grad, scale.grad


def layer_norm_modulation_ref(x: Tensor, scale: Tensor, shift: Tensor, eps: float = 1e-5) -> Tensor:
    """functional/normalization.py:6-12: F.layer_norm without affine, then x * (1 + scale) + shift.
    The reference oracle uses F.layer_norm's default eps (1e-5); flux/layers.py:247 uses 1e-6."""
    normed = F.layer_norm(x, (x.shape[-1],), eps=eps)
    return normed * (1 + scale) + shift


def apply_rope_ref(xq: Tensor, xk: Tensor, freqs_cis: Tensor) -> tuple[Tensor, Tensor]:
    """functional/positional_embedding.py:5-10 (== flux/layers.py:30-35)."""
    def one(x: Tensor) -> Tensor:
        x_ = x.float().reshape(*x.shape[:-1], -1, 1, 2)
        out = freqs_cis[..., 0] * x_[..., 0] + freqs_cis[..., 1] * x_[..., 1]
        return out.reshape(*x.shape).type_as(x)
    return one(xq), one(xk)


def rope_table_ref(pos: Tensor, dim: int, theta: int) -> Tensor:
    """flux/layers.py:20-27: [..., n] positions -> [..., n, dim/2, 2, 2] fp32, angles in fp64."""
    assert dim % 2 == 0
    scale = torch.arange(0, dim, 2, dtype=torch.float64) / dim
    omega = 1.0 / (theta ** scale)
    ang = torch.einsum("...n,d->...nd", pos.to(torch.float64), omega)
    out = torch.stack([torch.cos(ang), -torch.sin(ang), torch.sin(ang), torch.cos(ang)], dim=-1)
    return out.reshape(*out.shape[:-1], 2, 2).float()


def embed_nd_ref(ids: Tensor, axes_dim=(16, 56, 56), theta: int = 10000) -> Tensor:
    """flux/layers.py:38-52: ids [B, L, n_axes] -> pe [B, 1, L, sum(axes_dim)/2, 2, 2]."""
    emb = torch.cat([rope_table_ref(ids[..., i], axes_dim[i], theta) for i in range(ids.shape[-1])], dim=-3)
    return emb.unsqueeze(1)


def flux_ids(n_txt: int, grid_h: int, grid_w: int) -> Tensor:
    """Position ids of a Flux sequence: zeros for the text tokens, (0, h, w) row-major for the image."""
    ids = torch.zeros(1, n_txt + grid_h * grid_w, 3)
    hh, ww = torch.meshgrid(torch.arange(grid_h), torch.arange(grid_w), indexing="ij")
    ids[0, n_txt:, 1] = hh.reshape(-1).float()
    ids[0, n_txt:, 2] = ww.reshape(-1).float()
    return ids


# --------------------------------------------------------------------------------------------------
# data movement
# --------------------------------------------------------------------------------------------------
def split_heads_ref(qkv: Tensor, num_heads: int) -> tuple[Tensor, Tensor, Tensor]:
    """rearrange(qkv, "B L (K H D) -> K B H L D", K=3) of modules/blocks.py:115,148,154."""
    B, L, W = qkv.shape
    D = W // (3 * num_heads)
    t = qkv.reshape(B, L, 3, num_heads, D).permute(2, 0, 3, 1, 4)
    return t[0], t[1], t[2]


def qkv_concat_ref(txt_qkv: Tensor, img_qkv: Tensor, num_heads: int) -> tuple[Tensor, Tensor, Tensor]:
    """ops/qkv_concat.py:5-60 == split heads of both streams, torch.cat along the sequence, txt first
    (modules/blocks.py:158-160)."""
    tq, tk, tv = split_heads_ref(txt_qkv, num_heads)
    iq, ik, iv = split_heads_ref(img_qkv, num_heads)
    return (torch.cat((tq, iq), 2).contiguous(), torch.cat((tk, ik), 2).contiguous(), torch.cat((tv, iv), 2).contiguous())


# --------------------------------------------------------------------------------------------------
# element-wise
# --------------------------------------------------------------------------------------------------
def gelu_tanh_ref(x: Tensor) -> Tensor:
    """kernels/linear.py:22-28 == F.gelu(approximate="tanh")."""
    return F.gelu(x, approximate="tanh")


def silu_ref(x: Tensor) -> Tensor:
    """ops/silu.py:5-13: x * sigmoid(x) in fp32, stored in x.dtype."""
    xf = x.float()
    return (xf * torch.sigmoid(xf)).to(x.dtype)


def modulation_scale_shift_ref(x: Tensor, mod: Tensor, is_mod1: bool) -> Tensor:
    """ops/modulation.py:5-27: x [B,L,hid], mod [B, >=6*hid] (or 3*hid for mod1); (1 + scale) * x + shift
    with shift/scale = chunks 0/1 (mod1) or 3/4 (mod2); arithmetic in the promoted type of the loads
    (the stored dtype), i.e. fp32 here, rounded once."""
    hid = x.shape[-1]
    c = 0 if is_mod1 else 3
    shift = mod[:, None, c * hid:(c + 1) * hid].float()
    scale = mod[:, None, (c + 1) * hid:(c + 2) * hid].float()
    return ((scale + 1.0) * x.float() + shift).to(x.dtype)


def modulation_gate_proj_ref(img: Tensor, mod: Tensor, proj: Tensor) -> Tensor:
    """ops/modulation.py:29-44: img + gate * proj in fp32 with gate = chunk 2 of mod, rounded once."""
    hid = img.shape[-1]
    gate = mod[:, None, 2 * hid:3 * hid].float()
    return (img.float() + gate * proj.float()).to(img.dtype)


def gated_residual_ref(x: Tensor, gate: Tensor, y: Tensor) -> Tensor:
    """x + mod.gate * output as two PyTorch ops (modules/blocks.py:123,166-171)."""
    return x + gate * y


# --------------------------------------------------------------------------------------------------
# contractions
# --------------------------------------------------------------------------------------------------
def linear_ref(x: Tensor, w: Tensor, b: Tensor | None, activation: str = "") -> Tensor:
    """tests/test_linear.py:21-23: F.linear in the storage dtype, then F.gelu(tanh) on that result."""
    y = F.linear(x, w, b)
    return gelu_tanh_ref(y) if activation == "GELU" else y


def linear_ref_fp32(x: Tensor, w: Tensor, b: Tensor | None, activation: str = "") -> Tensor:
    """The same function with every step in fp32 (no intermediate rounding)."""
    y = x.float() @ w.float().t()
    if b is not None:
        y = y + b.float()
    return gelu_tanh_ref(y) if activation == "GELU" else y


def attention_ref_fp32(q: Tensor, k: Tensor, v: Tensor, sm_scale: float | None = None, chunk: int = 1024) -> Tensor:
    """softmax(q k^T * scale) v in fp32, row-chunked to bound memory (textbook form of what
    kernels/attention.py:10-46 computes online). Returns fp32 [B,H,L,D]."""
    D = q.shape[-1]
    s = (1.0 / math.sqrt(D)) if sm_scale is None else sm_scale
    kf, vf = k.float(), v.float()
    out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    for i in range(0, q.shape[-2], chunk):
        p = torch.softmax((q[..., i:i + chunk, :].float() @ kf.transpose(-1, -2)) * s, dim=-1)
        out[..., i:i + chunk, :] = p @ vf
    return out


def attention_ref(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
    """tests/test_attention.py:19 / flux/layers.py:14: the library routine in the storage dtype."""
    return F.scaled_dot_product_attention(q, k, v)


def attention_lse_ref(q: Tensor, k: Tensor, sm_scale: float | None = None) -> Tensor:
    """kernels/attention.py:166-169: M = m + log2(l) in the base-2 domain == log2 sum_j 2^(s_ij * log2 e)."""
    D = q.shape[-1]
    s = (1.0 / math.sqrt(D)) if sm_scale is None else sm_scale
    logits = (q.float() @ k.float().transpose(-1, -2)) * s
    return torch.logsumexp(logits, dim=-1) / math.log(2.0)


# --------------------------------------------------------------------------------------------------
# composed blocks (state-dict driven, no nn.Module): flux/layers.py:219-264 and :154-216
# --------------------------------------------------------------------------------------------------
def _modulation(sd: dict, prefix: str, vec: Tensor, n: int):
    out = F.linear(F.silu(vec), sd[f"{prefix}.lin.weight"], sd[f"{prefix}.lin.bias"])[:, None, :]
    return out.chunk(n, dim=-1)


def _qk_norm(sd: dict, prefix: str, q: Tensor, k: Tensor, v: Tensor):
    return (rms_norm_ref(q, sd[f"{prefix}.query_norm.scale"]).to(v), rms_norm_ref(k, sd[f"{prefix}.key_norm.scale"]).to(v))


def _attention(q: Tensor, k: Tensor, v: Tensor, pe: Tensor) -> Tensor:
    q, k = apply_rope_ref(q, k, pe)
    o = F.scaled_dot_product_attention(q, k, v)
    B, H, L, D = o.shape
    return o.permute(0, 2, 1, 3).reshape(B, L, H * D)


def single_stream_block_ref(sd: dict, x: Tensor, vec: Tensor, pe: Tensor, num_heads: int) -> Tensor:
    hid = x.shape[-1]
    shift, scale, gate = _modulation(sd, "modulation", vec, 3)
    x_mod = (1 + scale) * F.layer_norm(x, (hid,), eps=1e-6) + shift
    y1 = F.linear(x_mod, sd["linear1.weight"], sd["linear1.bias"])
    qkv, mlp = y1[..., :3 * hid], y1[..., 3 * hid:]
    q, k, v = split_heads_ref(qkv, num_heads)
    q, k = _qk_norm(sd, "norm", q, k, v)
    attn = _attention(q, k, v, pe)
    out = F.linear(torch.cat((attn, gelu_tanh_ref(mlp)), 2), sd["linear2.weight"], sd["linear2.bias"])
    return x + gate * out


def double_stream_block_ref(sd: dict, img: Tensor, txt: Tensor, vec: Tensor, pe: Tensor, num_heads: int):
    hid = img.shape[-1]
    mods = {s: _modulation(sd, f"{s}_mod", vec, 6) for s in ("img", "txt")}
    xs = {"img": img, "txt": txt}
    qkvs = {}
    for s in ("img", "txt"):
        shift, scale = mods[s][0], mods[s][1]
        xm = (1 + scale) * F.layer_norm(xs[s], (hid,), eps=1e-6) + shift
        q, k, v = split_heads_ref(F.linear(xm, sd[f"{s}_attn.qkv.weight"], sd.get(f"{s}_attn.qkv.bias")), num_heads)
        q, k = _qk_norm(sd, f"{s}_attn.norm", q, k, v)
        qkvs[s] = (q, k, v)
    q, k, v = (torch.cat((qkvs["txt"][i], qkvs["img"][i]), dim=2) for i in range(3))
    attn = _attention(q, k, v, pe)
    n_txt = txt.shape[1]
    parts = {"txt": attn[:, :n_txt], "img": attn[:, n_txt:]}
    outs = {}
    for s in ("img", "txt"):
        shift1, scale1, gate1, shift2, scale2, gate2 = mods[s]
        x = xs[s] + gate1 * F.linear(parts[s], sd[f"{s}_attn.proj.weight"], sd[f"{s}_attn.proj.bias"])
        xm = (1 + scale2) * F.layer_norm(x, (hid,), eps=1e-6) + shift2
        h = gelu_tanh_ref(F.linear(xm, sd[f"{s}_mlp.0.weight"], sd[f"{s}_mlp.0.bias"]))
        outs[s] = x + gate2 * F.linear(h, sd[f"{s}_mlp.2.weight"], sd[f"{s}_mlp.2.bias"])
    return outs["img"], outs["txt"]
