"""Flux single- and double-stream blocks on the HIP kernel set.

Module and parameter names match modules/blocks.py:18-172 of the reference (and therefore the
plain-PyTorch blocks in triton_kernels.flux), so state dicts are interchangeable. The forward
passes compute the same function with fewer trips through HBM:

  * linear1 of the single block writes its qkv columns and its GELU'd mlp columns straight into the
    two buffers the rest of the block reads (no split / nn.GELU / torch.cat passes),
  * QK RMSNorm + RoPE (+ the txt/img concat of the double block) is one gather kernel reading the
    strided qkv projection in place; v is never copied in the single block,
  * attention writes its output in "B L (H D)" order into the buffer linear2 / proj consumes,
  * the gated residual x + gate * y is the epilogue of the last linear.

Every intermediate is rounded to bf16 exactly where the un-fused sequence of PyTorch ops rounds it.
Inputs that are not bf16 CUDA tensors take the un-fused operator sequence (same operators, one at a
time), which is also what `fused = False` selects.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn as nn
from torch import Tensor

from triton_kernels import _native as nv
from triton_kernels.kernels.attention import attention_into, scaled_dot_product_attention
from triton_kernels.kernels.linear import linear, linear_into, qk_fusable
from triton_kernels.kernels.normalization import layer_norm_modulation
from triton_kernels.kernels.positional_embedding import apply_rope, qkv_prep
from triton_kernels.modules.normalization import QKNorm


def _heads(qkv: Tensor, num_heads: int) -> tuple[Tensor, Tensor, Tensor]:
    """[B, L, 3*H*D] -> three [B, H, L, D] views (no copy)."""
    B, L, width = qkv.shape
    D = width // (3 * num_heads)
    t = qkv.view(B, L, 3, num_heads, D).permute(2, 0, 3, 1, 4)
    return t[0], t[1], t[2]


def _merge_heads(x: Tensor) -> Tensor:
    """[B, H, L, D] -> [B, L, H*D]."""
    B, H, L, D = x.shape
    return x.permute(0, 2, 1, 3).reshape(B, L, H * D)


def _silu(x: Tensor) -> Tensor:
    dev = nv.require_gpu(x)
    x = x.contiguous()
    y = torch.empty_like(x)
    with nv.on_device(dev):
        rc = nv.lib().flux_silu(x.data_ptr(), y.data_ptr(), x.numel(), nv.dtype_code(x), nv.stream_ptr(dev))
    nv.check(rc, "flux_silu")
    return y


def _gelu_tanh(x: Tensor) -> Tensor:
    """tanh-GELU of a [.., n] tensor whose rows may be strided; result is contiguous."""
    dev = nv.require_gpu(x)
    n = x.shape[-1]
    x2 = x.reshape(-1, n) if x.is_contiguous() else x.flatten(0, -2)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    y = torch.empty((x2.shape[0], n), dtype=x.dtype, device=dev)
    with nv.on_device(dev):
        rc = nv.lib().flux_gelu_tanh(x2.data_ptr(), y.data_ptr(), x2.shape[0], n, x2.stride(0) if x2.shape[0] > 1 else n,
                                     n, nv.dtype_code(x), nv.stream_ptr(dev))
    nv.check(rc, "flux_gelu_tanh")
    return y.reshape(*x.shape)


def _gated_residual(x: Tensor, gate: Tensor, y: Tensor) -> Tensor:
    """x + gate * y with gate [B, 1, hid]; the product is rounded like the two PyTorch ops it replaces."""
    dev = nv.require_gpu(x, gate, y)
    B, hid = x.shape[0], x.shape[-1]
    x, y = x.contiguous(), y.contiguous()
    g = gate.reshape(B, hid)
    if g.stride(1) != 1:
        g = g.contiguous()
    out = torch.empty_like(x)
    with nv.on_device(dev):
        rc = nv.lib().flux_gate_residual(x.data_ptr(), g.data_ptr(), y.data_ptr(), out.data_ptr(), B, x.numel() // (B * hid),
                                         hid, g.stride(0) if B > 1 else hid, 1, nv.dtype_code(x), nv.stream_ptr(dev))
    nv.check(rc, "flux_gate_residual")
    return out


def attention(q: Tensor, k: Tensor, v: Tensor, pe: Tensor) -> Tensor:
    q, k = apply_rope(q, k, pe)
    return _merge_heads(scaled_dot_product_attention(q, k, v))


class Linear(nn.Linear):
    def forward(self, input: Tensor) -> Tensor:
        return linear(input, self.weight, self.bias)


class LinearGELU(nn.Linear):
    def forward(self, input: Tensor) -> Tensor:
        return linear(input, self.weight, self.bias, activation="GELU")


class SelfAttention(nn.Module):
    def __init__(self, dim: int, num_heads: int = 8, qkv_bias: bool = False):
        super().__init__()
        self.num_heads = num_heads
        self.qkv = Linear(dim, dim * 3, bias=qkv_bias)
        self.norm = QKNorm(dim // num_heads)
        self.proj = Linear(dim, dim)

    def forward(self, x: Tensor, pe: Tensor) -> Tensor:
        q, k, v = _heads(self.qkv(x), self.num_heads)
        q, k = self.norm(q, k, v)
        return self.proj(attention(q, k, v, pe=pe))


@dataclass
class ModulationOut:
    shift: Tensor
    scale: Tensor
    gate: Tensor


class Modulation(nn.Module):
    fused_silu = True

    def __init__(self, dim: int, double: bool):
        super().__init__()
        self.is_double = double
        self.multiplier = 6 if double else 3
        self.lin = Linear(dim, self.multiplier * dim, bias=True)

    def forward(self, vec: Tensor) -> tuple[ModulationOut, ModulationOut | None]:
        rows = vec.numel() // vec.shape[-1]
        if self.fused_silu and vec.is_cuda and vec.dtype == torch.bfloat16 and rows <= 8:
            # one launch: the row-vector kernel applies SiLU to vec as it reads it
            out = linear_into(vec, self.lin.weight, self.lin.bias, in_activation="SiLU").reshape(*vec.shape[:-1], -1)
        else:
            out = self.lin(_silu(vec))
        chunks = out[:, None, :].chunk(self.multiplier, dim=-1)
        first = ModulationOut(*chunks[:3])
        return first, (ModulationOut(*chunks[3:]) if self.is_double else None)


def MLP(hidden_size: int, mlp_hidden_dim: int, bias: bool = True):
    # index 1 is a placeholder so that the Linear layers keep state-dict indices 0 and 2
    return nn.Sequential(
        LinearGELU(hidden_size, mlp_hidden_dim, bias=bias),
        nn.Identity(),
        Linear(mlp_hidden_dim, hidden_size, bias=bias),
    )


def _fusable(*tensors: Tensor) -> bool:
    return all(t.is_cuda and t.dtype == torch.bfloat16 for t in tensors)


class SingleStreamBlock(nn.Module):
    """DiT block with parallel attention and MLP branches (https://arxiv.org/abs/2302.05442)."""

    fused = True
    # QKNorm + RoPE inside linear1's epilogue when the shapes allow (heads of 128, sequences of at least
    # 256 tokens); otherwise, or with this switched off, one preparation kernel behind linear1
    fuse_qk_epilogue = True
    # Optional callable(stage, edge), invoked on the launching thread right before (edge "begin") and
    # right after ("end") the launch of a stage of the forward: "modulation", "layer_norm" and, in the
    # fused forward, "linear1", "attention", "linear2". Benchmarks set it to record stream events
    # around a kernel inside real block passes.
    stage_hook = None

    def __init__(self, hidden_size: int, num_heads: int, mlp_ratio: float = 4.0, qk_scale: float | None = None):
        super().__init__()
        self.hidden_dim = hidden_size
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        head_dim = hidden_size // num_heads
        self.scale = qk_scale or head_dim**-0.5
        self.mlp_hidden_dim = int(hidden_size * mlp_ratio)
        self.linear1 = Linear(hidden_size, hidden_size * 3 + self.mlp_hidden_dim)   # qkv and mlp_in
        self.linear2 = Linear(hidden_size + self.mlp_hidden_dim, hidden_size)       # proj and mlp_out
        self.norm = QKNorm(head_dim)
        self.mlp_act = nn.GELU(approximate="tanh")
        self.modulation = Modulation(hidden_size, double=False)

    def forward(self, x: Tensor, vec: Tensor, pe: Tensor) -> Tensor:
        hook = self.stage_hook or (lambda stage, edge: None)
        hook("modulation", "begin")
        mod, _ = self.modulation(vec)
        hook("modulation", "end")
        hook("layer_norm", "begin")
        x_mod = layer_norm_modulation(x, mod.scale, mod.shift)
        hook("layer_norm", "end")
        if self.fused and _fusable(x, self.linear1.weight, self.linear2.weight, self.norm.query_norm.scale):
            return self._forward_fused(x, x_mod, mod, pe)
        hid = self.hidden_size
        y1 = self.linear1(x_mod)
        q, k, v = _heads(y1[..., : 3 * hid], self.num_heads)
        q, k = self.norm(q, k, v)
        attn = attention(q, k, v, pe=pe)
        both = torch.cat((attn, _gelu_tanh(y1[..., 3 * hid:])), 2)
        return _gated_residual(x, mod.gate, self.linear2(both))

    def _forward_fused(self, x: Tensor, x_mod: Tensor, mod: ModulationOut, pe: Tensor) -> Tensor:
        B, L, hid = x.shape
        H, D = self.num_heads, hid // self.num_heads
        M = B * L
        qkv = torch.empty((B, L, 3 * hid), dtype=x.dtype, device=x.device)
        both = torch.empty((B, L, hid + self.mlp_hidden_dim), dtype=x.dtype, device=x.device)
        both2 = both.view(M, -1)
        _, _, v_src = _heads(qkv, H)
        hook = self.stage_hook or (lambda stage, edge: None)
        hook("linear1", "begin")
        pe_ok = pe.dtype == torch.float32 and pe.is_contiguous() and pe.numel() in (L * D * 2, B * L * D * 2)
        if self.fuse_qk_epilogue and pe_ok and qk_fusable(x_mod, self.linear1.weight, L, D):
            # linear1: q and k columns -> bias, RMSNorm, RoPE -> q, k [B,H,L,D]; v columns -> qkv;
            # mlp columns -> GELU -> both[:, hid:]
            q = torch.empty((B, H, L, D), dtype=x.dtype, device=x.device)
            k = torch.empty_like(q)
            linear_into(x_mod, self.linear1.weight, self.linear1.bias, activation="GELU", act_begin=3 * hid,
                        out=qkv.view(M, -1), out2=both2[:, hid:], split=3 * hid,
                        qk=dict(q_out=q, k_out=k, q_scale=self.norm.query_norm.scale, k_scale=self.norm.key_norm.scale,
                                pe=pe, heads=H, seq_len=L, eps=1e-6))
        else:
            # linear1: qkv columns -> qkv, mlp columns -> GELU -> both[:, hid:]
            linear_into(x_mod, self.linear1.weight, self.linear1.bias, activation="GELU", act_begin=3 * hid,
                        out=qkv.view(M, -1), out2=both2[:, hid:], split=3 * hid)
            q_src, k_src, _ = _heads(qkv, H)
            q, k, _ = qkv_prep(q_src, k_src, None, pe=pe,
                               q_scale_img=self.norm.query_norm.scale, k_scale_img=self.norm.key_norm.scale)
        hook("linear1", "end")
        # attention output lands in both[:, :hid] in "B L (H D)" order
        attn_out = both[..., :hid].view(B, L, H, D).permute(0, 2, 1, 3)
        hook("attention", "begin")
        attention_into(q, k, v_src, attn_out)
        hook("attention", "end")
        out = torch.empty_like(x)
        hook("linear2", "begin")
        linear_into(both2, self.linear2.weight, self.linear2.bias, out=out.view(M, hid),
                    resid=x.contiguous().view(M, hid), gate=mod.gate)
        hook("linear2", "end")
        return out


class DoubleStreamBlock(nn.Module):
    fused = True

    def __init__(self, hidden_size: int, num_heads: int, mlp_ratio: float, qkv_bias: bool = False):
        super().__init__()
        mlp_hidden_dim = int(hidden_size * mlp_ratio)
        self.num_heads = num_heads
        self.hidden_size = hidden_size
        self.img_mod = Modulation(hidden_size, double=True)
        self.img_attn = SelfAttention(dim=hidden_size, num_heads=num_heads, qkv_bias=qkv_bias)
        self.img_mlp = MLP(hidden_size, mlp_hidden_dim)
        self.txt_mod = Modulation(hidden_size, double=True)
        self.txt_attn = SelfAttention(dim=hidden_size, num_heads=num_heads, qkv_bias=qkv_bias)
        self.txt_mlp = MLP(hidden_size, mlp_hidden_dim)

    # The txt stream is a ninth of the img stream's work: its small GEMMs (96 tiles of 128 x 128)
    # leave most CUs idle when they run alone, so the fused path runs the txt chain on a second HIP
    # stream of default priority, next to the img chain, and joins the two around the joint attention.
    two_streams = True

    def _side_stream(self, dev: torch.device) -> "torch.cuda.Stream":
        """This block's second stream on `dev`. Each instance keeps its own (per device), so two blocks
        driven from different host threads or streams never order their txt chains behind each
        other; setdefault makes the lazy creation safe when one instance is called from two threads."""
        streams = self.__dict__.setdefault("_side_streams", {})
        st = streams.get(dev.index)
        if st is None:
            st = streams.setdefault(dev.index, torch.cuda.Stream(device=dev))
        return st

    def __getstate__(self):
        state = self.__dict__.copy()
        state.pop("_side_streams", None)   # streams are neither copied nor pickled with the block
        return state

    def forward(self, img: Tensor, txt: Tensor, vec: Tensor, pe: Tensor) -> tuple[Tensor, Tensor]:
        H = self.num_heads
        Lt = txt.shape[1]
        fused = self.fused and _fusable(img, txt, self.img_attn.qkv.weight, self.img_attn.norm.query_norm.scale)
        if fused and self.two_streams and not torch.is_grad_enabled():
            return self._forward_two_streams(img, txt, vec, pe)

        img_mod1, img_mod2 = self.img_mod(vec)
        txt_mod1, txt_mod2 = self.txt_mod(vec)
        img_qkv = self.img_attn.qkv(layer_norm_modulation(img, img_mod1.scale, img_mod1.shift))
        txt_qkv = self.txt_attn.qkv(layer_norm_modulation(txt, txt_mod1.scale, txt_mod1.shift))
        img_q, img_k, img_v = _heads(img_qkv, H)
        txt_q, txt_k, txt_v = _heads(txt_qkv, H)

        if fused:
            B, Li, hid = img.shape
            q, k, v = qkv_prep(img_q, img_k, img_v, txt_q, txt_k, txt_v, pe=pe,
                               q_scale_img=self.img_attn.norm.query_norm.scale, k_scale_img=self.img_attn.norm.key_norm.scale,
                               q_scale_txt=self.txt_attn.norm.query_norm.scale, k_scale_txt=self.txt_attn.norm.key_norm.scale)
            attn = torch.empty((B, Lt + Li, hid), dtype=img.dtype, device=img.device)
            attention_into(q, k, v, attn.view(B, Lt + Li, H, hid // H).permute(0, 2, 1, 3))
        else:
            img_q, img_k = self.img_attn.norm(img_q, img_k, img_v)
            txt_q, txt_k = self.txt_attn.norm(txt_q, txt_k, txt_v)
            q, k, v = qkv_prep(img_q, img_k, img_v, txt_q, txt_k, txt_v)   # torch.cat(dim=2) of the three pairs
            attn = attention(q, k, v, pe=pe)
        txt_attn, img_attn = attn[:, :Lt], attn[:, Lt:]

        img = self._stream_tail(img, img_attn, img_mod1, img_mod2, self.img_attn.proj, self.img_mlp, fused)
        txt = self._stream_tail(txt, txt_attn, txt_mod1, txt_mod2, self.txt_attn.proj, self.txt_mlp, fused)
        return img, txt

    def _forward_two_streams(self, img: Tensor, txt: Tensor, vec: Tensor, pe: Tensor) -> tuple[Tensor, Tensor]:
        """Same arithmetic as the fused path of forward(), txt chain on a side stream. Everything the
        main stream reads later is allocated on the main stream (the caching allocator ties a block
        to the stream it was allocated on); temporaries of the side chain live and die on the side
        stream."""
        H = self.num_heads
        B, Li, hid = img.shape
        Lt = txt.shape[1]
        dev = img.device
        main = torch.cuda.current_stream(dev)
        side = self._side_stream(dev)
        txt_qkv = torch.empty((B * Lt, 3 * hid), dtype=txt.dtype, device=dev)
        txt_out = torch.empty((B, Lt, hid), dtype=txt.dtype, device=dev)
        attn = torch.empty((B, Lt + Li, hid), dtype=img.dtype, device=dev)

        side.wait_stream(main)            # inputs are ready on the main stream
        with torch.cuda.stream(side):
            txt_mod1, txt_mod2 = self.txt_mod(vec)
            qkv_lin = self.txt_attn.qkv
            linear_into(layer_norm_modulation(txt, txt_mod1.scale, txt_mod1.shift), qkv_lin.weight, qkv_lin.bias, out=txt_qkv,
                        shared_gpu=True)
        img_mod1, img_mod2 = self.img_mod(vec)
        img_qkv = self.img_attn.qkv(layer_norm_modulation(img, img_mod1.scale, img_mod1.shift))
        main.wait_stream(side)            # txt_qkv is complete

        img_q, img_k, img_v = _heads(img_qkv, H)
        txt_q, txt_k, txt_v = _heads(txt_qkv.view(B, Lt, 3 * hid), H)
        q, k, v = qkv_prep(img_q, img_k, img_v, txt_q, txt_k, txt_v, pe=pe,
                           q_scale_img=self.img_attn.norm.query_norm.scale, k_scale_img=self.img_attn.norm.key_norm.scale,
                           q_scale_txt=self.txt_attn.norm.query_norm.scale, k_scale_txt=self.txt_attn.norm.key_norm.scale)
        attention_into(q, k, v, attn.view(B, Lt + Li, H, hid // H).permute(0, 2, 1, 3))
        txt_attn, img_attn = attn[:, :Lt], attn[:, Lt:]

        side.wait_stream(main)            # attention output is complete
        with torch.cuda.stream(side):
            self._stream_tail(txt, txt_attn, txt_mod1, txt_mod2, self.txt_attn.proj, self.txt_mlp, True, out=txt_out, side_chain=True)
        img = self._stream_tail(img, img_attn, img_mod1, img_mod2, self.img_attn.proj, self.img_mlp, True, beside_txt=True)
        main.wait_stream(side)
        # tensors made on the side stream that the caller's stream may still be reading when they die
        for t in (txt_mod1.shift, txt_mod1.scale, txt_mod1.gate, txt_mod2.shift, txt_mod2.scale, txt_mod2.gate):
            t.record_stream(main)
        return img, txt_out

    @staticmethod
    def _stream_tail(x: Tensor, attn: Tensor, mod1: ModulationOut, mod2: ModulationOut, proj: Linear, mlp: nn.Sequential,
                     fused: bool, out: Tensor | None = None, beside_txt: bool = False, side_chain: bool = False) -> Tensor:
        if not fused:
            x = _gated_residual(x, mod1.gate, proj(attn))
            return _gated_residual(x, mod2.gate, mlp(layer_norm_modulation(x, mod2.scale, mod2.shift)))
        B, L, hid = x.shape
        M = B * L
        x = x.contiguous()
        x1 = torch.empty_like(x)
        # attn is a slice of the [B, Lt+Li, hid] buffer: rows of one batch element are evenly strided,
        # batches are not, so flatten per call only when there is a single batch element.
        a2 = attn.reshape(M, hid) if B > 1 else attn[0]
        # beside_txt: the txt chain's projection runs on the other stream at the same time and lives on the
        # CUs this launch leaves free (192 tiles at 4096 rows); a tile shape that fills all 256 CUs would
        # push it behind. By the time of the last projection the txt chain has finished: measured at
        # 4096 + 512 tokens, 1.18 ms like this, 1.23 ms with the flag on every launch or on none.
        # side_chain: this is the txt chain on the side stream; its small launches keep few, larger workgroups
        # instead of spreading over every CU the img chain is using (1.25 against 1.30 ms).
        linear_into(a2, proj.weight, proj.bias, out=x1.view(M, hid), resid=x.view(M, hid), gate=mod1.gate, shared_gpu=beside_txt or side_chain)
        h = linear(layer_norm_modulation(x1, mod2.scale, mod2.shift), mlp[0].weight, mlp[0].bias, activation="GELU", shared_gpu=side_chain)
        x2 = torch.empty_like(x) if out is None else out
        linear_into(h, mlp[2].weight, mlp[2].bias, out=x2.view(M, hid), resid=x1.view(M, hid), gate=mod2.gate, shared_gpu=side_chain)
        return x2
