"""apply_rope: rotate q and k by per-position 2x2 matrices (kernels/positional_embedding.py:55-82 of
the reference), plus the fused gather flux_qkv_prep it is a special case of."""
from __future__ import annotations

import torch
from torch import Tensor

from triton_kernels import _native as nv


def _row_view(t: Tensor) -> Tensor:
    """[B,H,L,D] tensor whose last dim is contiguous and whose strides keep 16-byte addressing."""
    vec = 16 // t.element_size()
    if t.stride(-1) != 1 or any(s % vec for s in t.stride()[:-1]) or t.data_ptr() % 16:
        t = t.contiguous()
    return t


def _pe_table(pe: Tensor, B: int, L: int, D: int) -> tuple[Tensor, int]:
    """fp32 [.., L, D/2, 2, 2] -> contiguous table and its batch stride (0 = shared by all batches).
    The reference kernel reads the first [L, D/2, 2, 2] table whatever the leading extents are
    (kernels/positional_embedding.py:31-32). A head extent is treated the same way here (the first
    head's table serves all heads); a batch extent equal to B is honoured, as broadcasting in the
    plain-PyTorch apply_rope would."""
    assert pe.shape[-4:] == (L, D // 2, 2, 2), f"freqs_cis must end in [{L}, {D // 2}, 2, 2], got {tuple(pe.shape)}"
    if pe.dim() >= 6 and pe.shape[-5] > 1:
        pe = pe.narrow(-5, 0, 1)
    lead = pe.shape[:-4]
    if pe.dtype != torch.float32:
        pe = pe.float()
    pe = pe.contiguous()
    n_lead = 1
    for s in lead:
        n_lead *= s
    if n_lead == 1:
        return pe, 0
    if len(lead) == 2 and lead[0] == B and lead[1] == 1:
        return pe, L * D * 2
    raise NotImplementedError(f"freqs_cis with leading shape {tuple(lead)}: only [1,1,...] or [B,1,...] are supported")


def qkv_prep(q_img: Tensor | None, k_img: Tensor | None, v_img: Tensor | None,
             q_txt: Tensor | None = None, k_txt: Tensor | None = None, v_txt: Tensor | None = None, *,
             pe: Tensor | None = None,
             q_scale_img: Tensor | None = None, k_scale_img: Tensor | None = None,
             q_scale_txt: Tensor | None = None, k_scale_txt: Tensor | None = None,
             eps: float = 1e-6):
    """One streaming pass: concat(txt, img) along the sequence, optional per-head RMS norm of q/k,
    optional RoPE of q/k, v copied. Returns (q, k, v) contiguous [B,H,Lt+Li,D]; entries whose inputs
    were None come back as None. All sources are [B,H,L*,D] views (any batch/head/row strides)."""
    ref = next(t for t in (q_img, k_img, v_img) if t is not None)
    B, H, Li, D = ref.shape
    txt_ref = next((t for t in (q_txt, k_txt, v_txt) if t is not None), None)
    Lt = 0 if txt_ref is None else txt_ref.shape[2]
    dev = nv.require_gpu(q_img, k_img, v_img, q_txt, k_txt, v_txt, pe)
    L = Lt + Li
    a = nv.QkvPrepArgs()
    keep = []
    outs = []
    for name, img, txt in (("q", q_img, q_txt), ("k", k_img, k_txt), ("v", v_img, v_txt)):
        if img is None:
            outs.append(None)
            continue
        assert img.shape == (B, H, Li, D) and img.dtype == ref.dtype
        img = _row_view(img)
        keep.append(img)
        setattr(a, f"{name}_img", nv.src4(img))
        if Lt:
            assert txt is not None and txt.shape == (B, H, Lt, D) and txt.dtype == ref.dtype
            txt = _row_view(txt)
            keep.append(txt)
            setattr(a, f"{name}_txt", nv.src4(txt))
        out = torch.empty((B, H, L, D), dtype=ref.dtype, device=dev)
        setattr(a, f"{name}_out", out.data_ptr())
        outs.append(out)
    scales = [q_scale_img, k_scale_img, q_scale_txt, k_scale_txt]
    if any(s is not None for s in scales):
        sdt = next(s for s in scales if s is not None).dtype
        if not (sdt == ref.dtype or (ref.dtype == torch.bfloat16 and sdt == torch.float32)):
            sdt = ref.dtype
        fixed = []
        for s in scales:
            if s is not None:
                assert s.shape[-1] == D
                s = s.to(sdt).contiguous()
                keep.append(s)
            fixed.append(s)
        a.q_scale_img, a.k_scale_img, a.q_scale_txt, a.k_scale_txt = [nv.ptr(s) for s in fixed]
        a.scale_dtype = nv._DTYPE_CODE[sdt]
    else:
        a.scale_dtype = nv.dtype_code(ref)
    if pe is not None:
        table, stride = _pe_table(pe, B, L, D)
        keep.append(table)
        a.pe = table.data_ptr()
        a.pe_batch_stride = stride
    a.B, a.H, a.Lt, a.Li, a.D = B, H, Lt, Li, D
    a.dtype = nv.dtype_code(ref)
    a.eps = float(eps)
    with nv.on_device(dev):
        rc = nv.lib().flux_qkv_prep(nv.byref(a), nv.stream_ptr(dev))
    nv.check(rc, "flux_qkv_prep")
    return tuple(outs)


def apply_rope(xq: Tensor, xk: Tensor, freqs_cis: Tensor) -> tuple[Tensor, Tensor]:
    assert xq.dim() == 4 and xq.shape == xk.shape and xq.dtype == xk.dtype
    q, k, _ = qkv_prep(xq, xk, None, pe=freqs_cis)
    return q, k
