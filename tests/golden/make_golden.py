#!/usr/bin/env python3
"""Writes tests/golden/flux_small.npz: seeded small inputs and the CPU oracle's outputs for every
op of the path. bf16 tensors are stored as their uint16 bit patterns under the key "<name>.bf16",
fp32 tensors as float32 under "<name>.f32" (tests/util.py: load_golden turns them back).

The reference repository holds no golden vectors for this path and none of its code is imported
here: the expected outputs come from oracle/flux_oracle.py, which tests/test_oracle_pins.py pins
against closed forms, invariants and library routines. The fixture is a regression anchor: it
fixes today's pinned oracle outputs so that a later change to the oracle or to a kernel shows up
against data, not against a moving reference.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
for p in (ROOT, os.path.join(ROOT, "triton-kernels_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

from oracle import flux_oracle as oracle  # noqa: E402

BF = torch.bfloat16


def build():
    g = torch.Generator().manual_seed(20240607)

    def rn(*shape, std=1.0, dtype=BF):
        return (torch.randn(*shape, generator=g, dtype=torch.float32) * std).to(dtype)

    out = {}
    # RMSNorm over head_dim 128: x [1,2,12,128]
    x = rn(1, 2, 12, 128)
    w = (torch.rand(128, generator=g) + 0.5).to(BF)
    out["rms_x"], out["rms_w"], out["rms_y"] = x, w, oracle.rms_norm_ref(x, w, 1e-6)
    # LayerNorm + modulation: x [2,8,256], scale/shift [2,1,256]
    x = rn(2, 8, 256)
    sc, sh = rn(2, 1, 256, std=0.5), rn(2, 1, 256, std=0.5)
    out["ln_x"], out["ln_scale"], out["ln_shift"] = x, sc, sh
    out["ln_y"] = oracle.layer_norm_modulation_ref(x, sc, sh, 1e-6)
    # RoPE: q,k [1,2,12,128], pe from the Flux table (3 txt + 3x3 img positions)
    q, k = rn(1, 2, 12, 128), rn(1, 2, 12, 128)
    pe = oracle.embed_nd_ref(oracle.flux_ids(3, 3, 3), (16, 56, 56), 10000)
    oq, ok = oracle.apply_rope_ref(q, k, pe)
    out["rope_q"], out["rope_k"], out["rope_pe"], out["rope_oq"], out["rope_ok"] = q, k, pe.float(), oq, ok
    # Linear + bias + tanh-GELU: A [40,64], W [48,64]
    a, wt, b = rn(40, 64), rn(48, 64, std=0.125), rn(48, std=0.02)
    out["lin_a"], out["lin_w"], out["lin_b"] = a, wt, b
    out["lin_y"] = oracle.linear_ref_fp32(a, wt, b, "")
    out["lin_y_gelu"] = oracle.linear_ref_fp32(a, wt, b, "GELU")
    # Attention: q,k,v [1,2,80,64] (ragged against the 64-key tile)
    q, k, v = rn(1, 2, 80, 64), rn(1, 2, 80, 64), rn(1, 2, 80, 64)
    out["att_q"], out["att_k"], out["att_v"] = q, k, v
    out["att_o"] = oracle.attention_ref_fp32(q, k, v)
    # QKV concat: txt [1,8,3*2*64], img [1,16,3*2*64], 2 heads
    t, i = rn(1, 8, 384), rn(1, 16, 384)
    cq, ck, cv = oracle.qkv_concat_ref(t, i, 2)
    out["cat_txt"], out["cat_img"], out["cat_q"], out["cat_k"], out["cat_v"] = t, i, cq, ck, cv
    packed = {}
    for k_, v_ in out.items():
        if v_.dtype == BF:
            packed[k_ + ".bf16"] = v_.contiguous().view(torch.int16).numpy().view(np.uint16)
        else:
            packed[k_ + ".f32"] = v_.float().numpy()
    return packed


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "flux_small.npz")
    np.savez_compressed(path, **build())
    print("wrote", path, os.path.getsize(path), "bytes")
