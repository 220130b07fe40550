"""Pins of the oracle (oracle/flux_oracle.py) that do not involve the code under test: float64
closed forms in numpy, invariants of the mathematics, special cases that reduce to a torch library
routine, and brute force on tiny inputs. The reference ships no golden vectors or seeds for this
path, so these are what anchor the oracle; a dropped term, a wrong sign or index or a transposed
operand fails at least one of them. Runs on the CPU."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import flux_oracle as oracle


def rng(seed):
    return torch.Generator().manual_seed(seed)


# ---------------------------------------------------------------- RMSNorm
def test_rms_norm_float64_closed_form_and_invariants():
    g = rng(1)
    x = torch.randn(3, 5, 7, 64, generator=g)
    w = torch.rand(64, generator=g) + 0.5
    y = oracle.rms_norm_ref(x, w)
    xn = x.double().numpy()
    want = xn / np.sqrt((xn ** 2).mean(-1, keepdims=True) + 1e-6) * w.double().numpy()
    np.testing.assert_allclose(y.numpy(), want, rtol=2e-6, atol=2e-6)
    # mean((y / scale)^2) == 1 up to eps
    np.testing.assert_allclose(((y / w) ** 2).mean(-1).numpy(), 1.0, rtol=1e-4)
    # invariant under positive rescaling of x (eps aside), equivariant in scale
    torch.testing.assert_close(oracle.rms_norm_ref(7.5 * x, w), y, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(oracle.rms_norm_ref(x, 2 * w), 2 * y)
    # library cross-check
    torch.testing.assert_close(y, F.rms_norm(x, (64,), weight=w, eps=1e-6), rtol=1e-5, atol=1e-6)


def test_rms_norm_bf16_rounding_order():
    """The normalised value is rounded to bf16 BEFORE the multiply by scale."""
    g = rng(2)
    x = torch.randn(64, 128, generator=g).to(torch.bfloat16)
    w = (torch.rand(128, generator=g) + 0.5).to(torch.bfloat16)
    y = oracle.rms_norm_ref(x, w)
    xf = x.float()
    normed = (xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + 1e-6)).to(torch.bfloat16)
    assert torch.equal(y, (normed.float() * w.float()).to(torch.bfloat16))
    assert y.dtype == torch.bfloat16


def test_rms_norm_backward_closed_form():
    g = rng(3)
    x = torch.randn(4, 6, 32, generator=g, dtype=torch.float64)
    w = torch.rand(32, generator=g, dtype=torch.float64) + 0.5
    dy = torch.randn(4, 6, 32, generator=g, dtype=torch.float64)
    dx, dw = oracle.rms_norm_bwd_ref(x, w, dy, eps=1e-6)
    r = torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6)
    m = dy * w
    dx_want = r * m - r ** 3 * (m * x).sum(-1, keepdim=True) * x / 32
    # the oracle evaluates in float32 whatever the input type
    torch.testing.assert_close(dx, dx_want, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dw, (dy * x * r).sum((0, 1)), rtol=1e-4, atol=1e-5)


# ---------------------------------------------------------------- LayerNorm + modulation
def test_layer_norm_modulation_special_cases():
    g = rng(4)
    x = torch.randn(2, 9, 48, generator=g)
    zero = torch.zeros(2, 1, 48)
    torch.testing.assert_close(oracle.layer_norm_modulation_ref(x, zero, zero), F.layer_norm(x, (48,)))
    scale = torch.randn(2, 1, 48, generator=g)
    shift = torch.randn(2, 1, 48, generator=g)
    y = oracle.layer_norm_modulation_ref(x, scale, shift)
    # affine in shift, and in (1 + scale)
    torch.testing.assert_close(oracle.layer_norm_modulation_ref(x, scale, shift + 2.0), y + 2.0)
    torch.testing.assert_close(oracle.layer_norm_modulation_ref(x, scale, zero) , y - shift)
    xn = x.double().numpy()
    ln = (xn - xn.mean(-1, keepdims=True)) / np.sqrt(xn.var(-1, keepdims=True) + 1e-5)
    want = ln * (1 + scale.double().numpy()) + shift.double().numpy()
    np.testing.assert_allclose(y.numpy(), want, rtol=1e-5, atol=1e-5)
    # swapping the two arguments is a different function (guards the (x, scale, shift) order)
    assert not torch.allclose(oracle.layer_norm_modulation_ref(x, shift, scale), y)


# ---------------------------------------------------------------- RoPE
def test_apply_rope_identity_norm_and_complex_form():
    g = rng(5)
    B, H, L, D = 2, 3, 11, 16
    q = torch.randn(B, H, L, D, generator=g)
    k = torch.randn(B, H, L, D, generator=g)
    eye = torch.eye(2).expand(1, 1, L, D // 2, 2, 2)
    oq, ok = oracle.apply_rope_ref(q, k, eye)
    assert torch.equal(oq, q) and torch.equal(ok, k)
    phi = torch.rand(1, 1, L, D // 2, generator=g, dtype=torch.float64) * 6.28
    rot = torch.stack((torch.cos(phi), -torch.sin(phi), torch.sin(phi), torch.cos(phi)), -1).reshape(1, 1, L, D // 2, 2, 2).float()
    oq, ok = oracle.apply_rope_ref(q, k, rot)
    # rotations preserve the norm of every pair
    torch.testing.assert_close(oq.reshape(B, H, L, -1, 2).norm(dim=-1), q.reshape(B, H, L, -1, 2).norm(dim=-1), rtol=1e-5, atol=1e-5)
    # equals multiplication by e^{i phi} of the complex number (x[2i] + i x[2i+1])
    zc = torch.view_as_complex(q.double().reshape(B, H, L, -1, 2)) * torch.polar(torch.ones_like(phi), phi)
    torch.testing.assert_close(oq.double(), torch.view_as_real(zc).reshape(B, H, L, D), rtol=1e-5, atol=1e-5)
    # general 2x2 (not a rotation): brute force over every pair
    f = torch.randn(1, 1, L, D // 2, 2, 2, generator=g)
    oq, _ = oracle.apply_rope_ref(q, k, f)
    for i in range(D // 2):
        for a in range(2):
            want = f[0, 0, :, i, a, 0] * q[..., 2 * i] + f[0, 0, :, i, a, 1] * q[..., 2 * i + 1]
            torch.testing.assert_close(oq[..., 2 * i + a], want)


def test_rope_table_and_embed_nd_known_answers():
    pos = torch.tensor([[0.0, 1.0, 2.0, 10.0]])
    t = oracle.rope_table_ref(pos, 8, 10000)
    assert t.shape == (1, 4, 4, 2, 2) and t.dtype == torch.float32
    assert torch.equal(t[0, 0], torch.eye(2).expand(4, 2, 2))            # position 0: identity
    for p_i, p in enumerate(pos[0].tolist()):                            # pair 0: angle == position
        np.testing.assert_allclose(t[0, p_i, 0].numpy(), [[math.cos(p), -math.sin(p)], [math.sin(p), math.cos(p)]], atol=1e-6)
    # pair j: angle = pos * theta^(-2j/dim)
    np.testing.assert_allclose(t[0, 3, 2, 1, 0].item(), math.sin(10.0 * 10000 ** (-4 / 8)), atol=1e-6)
    ids = oracle.flux_ids(5, 3, 4)
    assert ids.shape == (1, 17, 3) and (ids[0, :5] == 0).all()
    assert ids[0, 5 + 1 * 4 + 2].tolist() == [0.0, 1.0, 2.0]              # token = h * W + w
    pe = oracle.embed_nd_ref(ids)
    assert pe.shape == (1, 1, 17, 64, 2, 2)
    assert torch.equal(pe[0, 0, :5], torch.eye(2).expand(5, 64, 2, 2))   # text tokens are not rotated
    # axis split 8 / 28 / 28 pairs: axis 0 is all zeros here, so its 8 pairs are identities everywhere
    assert torch.equal(pe[0, 0, :, :8], torch.eye(2).expand(17, 8, 2, 2))
    tok = 5 + 2 * 4 + 3                                                   # h = 2, w = 3
    np.testing.assert_allclose(pe[0, 0, tok, 8, 0, 0].item(), math.cos(2.0), atol=1e-6)    # first pair of the h axis
    np.testing.assert_allclose(pe[0, 0, tok, 36, 1, 0].item(), math.sin(3.0), atol=1e-6)   # first pair of the w axis


# ---------------------------------------------------------------- data movement
def test_split_heads_and_qkv_concat_match_einops():
    from einops import rearrange

    g = rng(6)
    B, H, D, Lt, Li = 2, 3, 8, 4, 6
    txt = torch.randn(B, Lt, 3 * H * D, generator=g)
    img = torch.randn(B, Li, 3 * H * D, generator=g)
    q, k, v = oracle.split_heads_ref(img, H)
    rq, rk, rv = rearrange(img, "B L (K H D) -> K B H L D", K=3, H=H)
    assert torch.equal(q, rq) and torch.equal(k, rk) and torch.equal(v, rv)
    cq, ck, cv = oracle.qkv_concat_ref(txt, img, H)
    tq, tk, tv = rearrange(txt, "B L (K H D) -> K B H L D", K=3, H=H)
    assert torch.equal(cq, torch.cat((tq, rq), 2)) and torch.equal(cv, torch.cat((tv, rv), 2)) and torch.equal(ck, torch.cat((tk, rk), 2))
    # index emulation of the flat kernel: out[b,h,s,d] = src[b, s', k*hid + h*D + d]
    hid = H * D
    b, h, s, d = 1, 2, Lt + 3, 5
    assert cq[b, h, s, d] == img[b, s - Lt, 0 * hid + h * D + d] and ck[b, h, 1, d] == txt[b, 1, 1 * hid + h * D + d]


# ---------------------------------------------------------------- element-wise
def test_elementwise_closed_forms():
    x = torch.linspace(-6, 6, 101)
    want = 0.5 * x.double() * (1 + torch.tanh(math.sqrt(2 / math.pi) * (x.double() + 0.044715 * x.double() ** 3)))
    torch.testing.assert_close(oracle.gelu_tanh_ref(x).double(), want, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(oracle.silu_ref(x), x / (1 + torch.exp(-x)), rtol=1e-5, atol=1e-6)
    g = rng(7)
    B, L, hid = 2, 3, 8
    xx = torch.randn(B, L, hid, generator=g)
    mod = torch.randn(B, 6 * hid, generator=g)
    for is_mod1, c in ((True, 0), (False, 3)):
        want = (1 + mod[:, None, (c + 1) * hid:(c + 2) * hid]) * xx + mod[:, None, c * hid:(c + 1) * hid]
        torch.testing.assert_close(oracle.modulation_scale_shift_ref(xx, mod, is_mod1), want)
    proj = torch.randn(B, L, hid, generator=g)
    torch.testing.assert_close(oracle.modulation_gate_proj_ref(xx, mod, proj), xx + mod[:, None, 2 * hid:3 * hid] * proj)


# ---------------------------------------------------------------- contractions
def test_linear_identity_and_brute_force():
    g = rng(8)
    x = torch.randn(5, 6, generator=g)
    b = torch.randn(6, generator=g)
    torch.testing.assert_close(oracle.linear_ref(x, torch.eye(6), b), x + b)
    w = torch.randn(4, 6, generator=g)
    b4 = torch.randn(4, generator=g)
    y = oracle.linear_ref_fp32(x, w, b4)
    for m in range(5):
        for n in range(4):
            assert abs(y[m, n].item() - (sum(x[m, k_].item() * w[n, k_].item() for k_ in range(6)) + b4[n].item())) < 1e-5
    torch.testing.assert_close(oracle.linear_ref(x, w, b4, "GELU"), F.gelu(F.linear(x, w, b4), approximate="tanh"))
    torch.testing.assert_close(oracle.linear_ref_fp32(x, w, b4, "GELU"), F.gelu(y, approximate="tanh"))
    torch.testing.assert_close(oracle.linear_ref_fp32(x, w, None), x @ w.t())


def test_attention_invariants_and_library():
    g = rng(9)
    B, H, L, D = 2, 2, 37, 16
    q, k, v = (torch.randn(B, H, L, D, generator=g) for _ in range(3))
    o = oracle.attention_ref_fp32(q, k, v, chunk=8)
    torch.testing.assert_close(o, F.scaled_dot_product_attention(q, k, v), rtol=1e-5, atol=1e-5)
    # brute force in float64
    s = (q.double() @ k.double().transpose(-1, -2)) / math.sqrt(D)
    p = torch.exp(s - s.max(-1, keepdim=True).values)
    want = (p / p.sum(-1, keepdim=True)) @ v.double()
    torch.testing.assert_close(o.double(), want, rtol=1e-5, atol=1e-6)
    # rows of P sum to one; a single distinct key returns its value; key order does not matter
    torch.testing.assert_close(oracle.attention_ref_fp32(q, k, torch.full_like(v, 0.25)), torch.full_like(v, 0.25))
    k1, v1 = k[:, :, :1].expand(B, H, L, D), v[:, :, :1].expand(B, H, L, D)
    torch.testing.assert_close(oracle.attention_ref_fp32(q, k1, v1), v1.contiguous(), rtol=1e-6, atol=1e-6)
    perm = torch.randperm(L, generator=g)
    torch.testing.assert_close(oracle.attention_ref_fp32(q, k[:, :, perm], v[:, :, perm]), o, rtol=1e-5, atol=1e-5)
    # log-sum-exp in base 2, as the reference kernel stores it
    lse = oracle.attention_lse_ref(q, k)
    torch.testing.assert_close(lse, torch.log2(torch.exp(s).sum(-1)).float(), rtol=1e-5, atol=1e-5)
    # explicit scale
    torch.testing.assert_close(oracle.attention_ref_fp32(q, k, v, sm_scale=0.3),
                               F.scaled_dot_product_attention(q, k, v, scale=0.3), rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- blocks
@pytest.mark.parametrize("kind", ["single", "double"])
def test_block_oracles_agree_with_the_module_restatement(kind):
    """Two independent restatements of the Flux blocks (state-dict driven functions in the oracle,
    nn.Modules in triton_kernels.flux) must agree exactly on the CPU in fp32."""
    from triton_kernels import flux

    torch.manual_seed(0)
    hid, heads, L, Lt = 64, 4, 10, 3
    g = rng(10)
    vec = torch.randn(2, hid, generator=g)
    pe = torch.randn(1, 1, L + (Lt if kind == "double" else 0), hid // heads // 2, 2, 2, generator=g)
    if kind == "single":
        blk = flux.SingleStreamBlock(hid, heads)
        x = torch.randn(2, L, hid, generator=g)
        with torch.no_grad():
            want = blk(x, vec, pe)
            got = oracle.single_stream_block_ref(blk.state_dict(), x, vec, pe, heads)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
    else:
        blk = flux.DoubleStreamBlock(hid, heads, 4.0, qkv_bias=True)
        img = torch.randn(2, L, hid, generator=g)
        txt = torch.randn(2, Lt, hid, generator=g)
        with torch.no_grad():
            w_img, w_txt = blk(img, txt, vec, pe)
            g_img, g_txt = oracle.double_stream_block_ref(blk.state_dict(), img, txt, vec, pe, heads)
        torch.testing.assert_close(g_img, w_img, rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(g_txt, w_txt, rtol=1e-5, atol=1e-5)


def test_single_block_oracle_equals_unfused_composition():
    """The block oracle is nothing but the pinned per-op oracles chained in the reference's order."""
    g = rng(11)
    hid, heads, L = 32, 2, 6
    mlp = 4 * hid
    sd = {
        "modulation.lin.weight": torch.randn(3 * hid, hid, generator=g) * 0.2, "modulation.lin.bias": torch.randn(3 * hid, generator=g) * 0.1,
        "linear1.weight": torch.randn(3 * hid + mlp, hid, generator=g) * 0.2, "linear1.bias": torch.randn(3 * hid + mlp, generator=g) * 0.1,
        "linear2.weight": torch.randn(hid, hid + mlp, generator=g) * 0.1, "linear2.bias": torch.randn(hid, generator=g) * 0.1,
        "norm.query_norm.scale": torch.rand(hid // heads, generator=g) + 0.5, "norm.key_norm.scale": torch.rand(hid // heads, generator=g) + 0.5,
    }
    x = torch.randn(1, L, hid, generator=g)
    vec = torch.randn(1, hid, generator=g)
    pe = torch.randn(1, 1, L, hid // heads // 2, 2, 2, generator=g)
    got = oracle.single_stream_block_ref(sd, x, vec, pe, heads)
    shift, scale, gate = oracle.linear_ref(oracle.silu_ref(vec), sd["modulation.lin.weight"], sd["modulation.lin.bias"])[:, None].chunk(3, -1)
    xm = oracle.layer_norm_modulation_ref(x, scale, shift, eps=1e-6)
    y1 = oracle.linear_ref(xm, sd["linear1.weight"], sd["linear1.bias"])
    q, k, v = oracle.split_heads_ref(y1[..., :3 * hid], heads)
    q = oracle.rms_norm_ref(q, sd["norm.query_norm.scale"])
    k = oracle.rms_norm_ref(k, sd["norm.key_norm.scale"])
    q, k = oracle.apply_rope_ref(q, k, pe)
    a = oracle.attention_ref_fp32(q, k, v).permute(0, 2, 1, 3).reshape(1, L, hid)
    out = oracle.linear_ref(torch.cat((a, oracle.gelu_tanh_ref(y1[..., 3 * hid:])), 2), sd["linear2.weight"], sd["linear2.bias"])
    torch.testing.assert_close(got, oracle.gated_residual_ref(x, gate, out), rtol=1e-5, atol=1e-5)


def test_double_block_oracle_equals_unfused_composition():
    """The double-stream oracle (modules/blocks.py:126-171) is the pinned per-op oracles chained in the
    reference's order: per stream mod1 -> qkv -> QKNorm, txt-first concat, RoPE, attention, then per
    stream proj + gated residual, mod2 -> mlp (GELU) -> gated residual."""
    g = rng(12)
    hid, heads, Li, Lt = 32, 2, 7, 3
    mlp = 4 * hid
    D = hid // heads
    sd = {}
    for s_ in ("img", "txt"):
        sd[f"{s_}_mod.lin.weight"] = torch.randn(6 * hid, hid, generator=g) * 0.2
        sd[f"{s_}_mod.lin.bias"] = torch.randn(6 * hid, generator=g) * 0.1
        sd[f"{s_}_attn.qkv.weight"] = torch.randn(3 * hid, hid, generator=g) * 0.2
        sd[f"{s_}_attn.qkv.bias"] = torch.randn(3 * hid, generator=g) * 0.1
        sd[f"{s_}_attn.norm.query_norm.scale"] = torch.rand(D, generator=g) + 0.5
        sd[f"{s_}_attn.norm.key_norm.scale"] = torch.rand(D, generator=g) + 0.5
        sd[f"{s_}_attn.proj.weight"] = torch.randn(hid, hid, generator=g) * 0.2
        sd[f"{s_}_attn.proj.bias"] = torch.randn(hid, generator=g) * 0.1
        sd[f"{s_}_mlp.0.weight"] = torch.randn(mlp, hid, generator=g) * 0.2
        sd[f"{s_}_mlp.0.bias"] = torch.randn(mlp, generator=g) * 0.1
        sd[f"{s_}_mlp.2.weight"] = torch.randn(hid, mlp, generator=g) * 0.1
        sd[f"{s_}_mlp.2.bias"] = torch.randn(hid, generator=g) * 0.1
    B = 2
    xs = {"img": torch.randn(B, Li, hid, generator=g), "txt": torch.randn(B, Lt, hid, generator=g)}
    vec = torch.randn(B, hid, generator=g)
    pe = torch.randn(1, 1, Lt + Li, D // 2, 2, 2, generator=g)
    g_img, g_txt = oracle.double_stream_block_ref(sd, xs["img"], xs["txt"], vec, pe, heads)

    mods, qkv = {}, {}
    for s_ in ("img", "txt"):
        mods[s_] = oracle.linear_ref(oracle.silu_ref(vec), sd[f"{s_}_mod.lin.weight"], sd[f"{s_}_mod.lin.bias"])[:, None].chunk(6, -1)
        xm = oracle.layer_norm_modulation_ref(xs[s_], mods[s_][1], mods[s_][0], eps=1e-6)
        # the same through the reference's inductor-derived op (ops/modulation.py:5-27, mod1) on the normalised rows
        ln = F.layer_norm(xs[s_], (hid,), eps=1e-6)
        torch.testing.assert_close(oracle.modulation_scale_shift_ref(ln, torch.cat(mods[s_], -1)[:, 0], True), xm, rtol=1e-5, atol=1e-5)
        q, k, v = oracle.split_heads_ref(oracle.linear_ref(xm, sd[f"{s_}_attn.qkv.weight"], sd[f"{s_}_attn.qkv.bias"]), heads)
        qkv[s_] = (oracle.rms_norm_ref(q, sd[f"{s_}_attn.norm.query_norm.scale"]), oracle.rms_norm_ref(k, sd[f"{s_}_attn.norm.key_norm.scale"]), v)
    q, k, v = (torch.cat((qkv["txt"][i], qkv["img"][i]), dim=2) for i in range(3))
    q, k = oracle.apply_rope_ref(q, k, pe)
    attn = oracle.attention_ref_fp32(q, k, v).permute(0, 2, 1, 3).reshape(B, Lt + Li, hid)
    parts = {"txt": attn[:, :Lt], "img": attn[:, Lt:]}
    for s_, got in (("img", g_img), ("txt", g_txt)):
        shift1, scale1, gate1, shift2, scale2, gate2 = mods[s_]
        x = oracle.gated_residual_ref(xs[s_], gate1, oracle.linear_ref(parts[s_], sd[f"{s_}_attn.proj.weight"], sd[f"{s_}_attn.proj.bias"]))
        xm = oracle.layer_norm_modulation_ref(x, scale2, shift2, eps=1e-6)
        h = oracle.linear_ref(xm, sd[f"{s_}_mlp.0.weight"], sd[f"{s_}_mlp.0.bias"], "GELU")
        want = oracle.gated_residual_ref(x, gate2, oracle.linear_ref(h, sd[f"{s_}_mlp.2.weight"], sd[f"{s_}_mlp.2.bias"]))
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
