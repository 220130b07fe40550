"""HIP row-wise kernels vs the oracle: RMSNorm (fwd/bwd), LayerNorm+modulation, RoPE, concat.

The fp32 grids mirror the reference's own unit tests (tests/test_rms_norm.py, test_layer_norm.py,
test_rope.py: fp32, atol 1e-5 forward, 1e-3 backward); the bf16 cases use the tolerance stated for
this path (atol 1e-2, rtol 1e-2) at the Flux shapes, plus ragged and strided edge cases.
"""
import math

import pytest
import torch

import triton_kernels as tk
from oracle import flux_oracle as oracle
from triton_kernels import testing as cfg
from util import DEV, randn, seeded

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("batch_size", [1, 4])
@pytest.mark.parametrize("num_heads", [2, 24])
@pytest.mark.parametrize("seq_len", [256, 1024])
@pytest.mark.parametrize("head_dim", [128, 256, 512])
def test_rms_norm_fp32_fwd_bwd(batch_size, num_heads, seq_len, head_dim):
    g = seeded(batch_size * 7 + num_heads * 3 + seq_len + head_dim)
    x = randn(g, batch_size, num_heads, seq_len, head_dim).to(DEV).requires_grad_(True)
    w = randn(g, head_dim).to(DEV).requires_grad_(True)
    dy = randn(g, batch_size, num_heads, seq_len, head_dim).to(DEV)
    y = tk.rms_norm(x, w)
    y.backward(dy)
    y_ref = oracle.rms_norm_ref(x.detach(), w.detach())
    dx_ref, dw_ref = oracle.rms_norm_bwd_ref(x.detach(), w.detach(), dy)
    torch.testing.assert_close(y, y_ref, atol=1e-5, rtol=0)
    torch.testing.assert_close(x.grad, dx_ref, atol=1e-3, rtol=0)
    torch.testing.assert_close(w.grad, dw_ref, atol=1e-3, rtol=1e-4)


@pytest.mark.parametrize("shape", [(1, 24, 4608, 128), (2, 3, 77, 128), (5, 64), (3, 1000, 96), (2, 7, 4104), (1, 3, 10000),
                                   (2, 2, 50), (1, 24, 13, 128)])
def test_rms_norm_bf16_shapes(shape):
    g = seeded(sum(shape))
    x = randn(g, *shape, dtype=torch.bfloat16).to(DEV)
    w = (torch.rand(shape[-1], generator=g) + 0.5).to(torch.bfloat16).to(DEV)
    y = tk.rms_norm(x, w)
    assert y.shape == x.shape and y.dtype == x.dtype
    torch.testing.assert_close(y, oracle.rms_norm_ref(x, w), atol=1e-2, rtol=1e-2)
    # scale kept in fp32 (a module that was not cast): output stays bf16 as in the reference launcher
    y2 = tk.rms_norm(x, w.float())
    torch.testing.assert_close(y2, oracle.rms_norm_ref(x, w.float()).to(torch.bfloat16), atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("scale_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(1, 24, 4608, 128),   # the Flux q/k shape: one vector per lane
                                   (3, 700, 512),         # two vectors per lane
                                   (2, 333, 1536),        # three
                                   (2, 100, 2048),        # four
                                   (2, 37, 4104),         # more than four: one block per row
                                   (1, 19, 10000),
                                   (5, 9, 100),           # not a multiple of the vector width: one block per row
                                   (4, 64)])
def test_rms_norm_bf16_backward(shape, scale_dtype):
    """_rms_norm.backward (kernels/normalization.py:110-139) for bf16 activations, with the scale in bf16
    or kept in fp32, over every register plan of the backward kernel and its one-block-per-row
    fallback. dx against autograd of the oracle at bf16 tolerance; dscale, an fp32 sum over all rows,
    against the same sum formed in fp64 from the oracle's per-row terms."""
    g = seeded(sum(shape) + (scale_dtype == torch.float32))
    x = randn(g, *shape, dtype=torch.bfloat16).to(DEV).requires_grad_(True)
    w = (torch.rand(shape[-1], generator=g) + 0.5).to(scale_dtype).to(DEV).requires_grad_(True)
    dy = randn(g, *shape, dtype=torch.bfloat16).to(DEV)
    y = tk.rms_norm(x, w)
    y.backward(dy)
    assert x.grad.dtype == torch.bfloat16 and w.grad.dtype == scale_dtype and w.grad.shape == w.shape
    # fp32 oracle of the same function (bf16 values, fp32 arithmetic, no intermediate rounding)
    dx_ref, dw_ref = oracle.rms_norm_bwd_ref(x.detach().float(), w.detach().float(), dy.float())
    torch.testing.assert_close(x.grad.float(), dx_ref, atol=1e-2 * max(1.0, dx_ref.abs().max().item()), rtol=1e-2)
    assert (x.grad.float() - dx_ref).abs().mean().item() < 4e-3
    # dscale[c] = sum_rows dy * x * rstd: a sum of rows terms of size ~1, so its error scales with sqrt(rows)
    xf = x.detach().double()
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)
    dw64 = (dy.double() * xf * rstd).reshape(-1, shape[-1]).sum(0)
    torch.testing.assert_close(dw_ref.double(), dw64, atol=1e-3 * math.sqrt(xf.numel() / shape[-1]), rtol=1e-3)  # the oracle agrees with the closed form
    tol = (2.0 ** -8 if scale_dtype == torch.bfloat16 else 1e-5) * dw64.abs() + 2e-4 * math.sqrt(xf.numel() / shape[-1])
    assert ((w.grad.double() - dw64).abs() <= tol).all()


def test_rms_norm_config1_cpu_oracle_and_strided_view():
    x, w = cfg.config1("cpu", scale=0.25)
    want = oracle.rms_norm_ref(x, w)                       # CPU oracle, same bits
    got = tk.rms_norm(x.to(DEV), w.to(DEV))
    torch.testing.assert_close(got.cpu(), want, atol=1e-2, rtol=1e-2)
    # bit-for-bit against the same formula evaluated by torch on the GPU
    assert (got != oracle.rms_norm_ref(x.to(DEV), w.to(DEV))).float().mean().item() < 1e-3
    # q as the block sees it: a strided [B,H,L,D] view into a [B,L,3*H*D] projection
    B, Hh, L, D = 1, 24, 300, 128
    g = seeded(5)
    qkv = randn(g, B, L, 3 * Hh * D, dtype=torch.bfloat16).to(DEV)
    q = qkv.view(B, L, 3, Hh, D).permute(2, 0, 3, 1, 4)[1]
    assert not q.is_contiguous()
    torch.testing.assert_close(tk.rms_norm(q, w.to(DEV)), oracle.rms_norm_ref(q, w.to(DEV)), atol=1e-2, rtol=1e-2)


def test_rms_norm_too_wide_raises():
    x = torch.zeros(2, 65537, device=DEV)
    with pytest.raises(RuntimeError):
        tk.rms_norm(x, torch.ones(65537, device=DEV))


@pytest.mark.parametrize("batch_size", [1, 2, 16])
@pytest.mark.parametrize("seq_len", [256, 1024])
@pytest.mark.parametrize("embed_dim", [1024, 2048, 3072])
def test_layer_norm_modulation_fp32(batch_size, seq_len, embed_dim):
    g = seeded(batch_size + seq_len + embed_dim)
    x = randn(g, batch_size, seq_len, embed_dim).to(DEV)
    scale = randn(g, batch_size, 1, embed_dim).to(DEV)
    shift = randn(g, batch_size, 1, embed_dim).to(DEV)
    y = tk.layer_norm_modulation(x, scale, shift)
    torch.testing.assert_close(y, oracle.layer_norm_modulation_ref(x, scale, shift), atol=1e-5, rtol=0)


@pytest.mark.parametrize("shape", [(1, 4608, 3072), (2, 333, 3072), (3, 17, 1000), (2, 5, 4104), (1, 9, 20000), (2, 4, 66)])
def test_layer_norm_modulation_bf16(shape):
    g = seeded(sum(shape))
    B, L, N = shape
    x = randn(g, B, L, N, dtype=torch.bfloat16).to(DEV)
    mod = randn(g, B, 3 * N, dtype=torch.bfloat16, std=0.1).to(DEV)
    shift, scale, _ = mod[:, None, :].chunk(3, dim=-1)      # strided chunks, as Modulation produces them
    y = tk.layer_norm_modulation(x, scale, shift, eps=1e-6)
    torch.testing.assert_close(y, oracle.layer_norm_modulation_ref(x, scale, shift, eps=1e-6), atol=1e-2, rtol=1e-2)


def test_layer_norm_modulation_config2_cpu_oracle():
    x, scale, shift = cfg.config2("cpu", scale=0.25)
    want = oracle.layer_norm_modulation_ref(x, scale, shift, eps=1e-6)
    got = tk.layer_norm_modulation(x.to(DEV), scale.to(DEV), shift.to(DEV), eps=1e-6)
    torch.testing.assert_close(got.cpu(), want, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("batch_size", [1, 4])
@pytest.mark.parametrize("num_heads", [2, 24])
@pytest.mark.parametrize("seq_len", [256, 1024])
@pytest.mark.parametrize("head_dim", [128, 256, 512])
def test_rope_fp32(batch_size, num_heads, seq_len, head_dim):
    g = seeded(batch_size + num_heads + seq_len + head_dim)
    q = randn(g, batch_size, num_heads, seq_len, head_dim).to(DEV)
    k = randn(g, batch_size, num_heads, seq_len, head_dim).to(DEV)
    pe = randn(g, 1, 1, seq_len, head_dim // 2, 2, 2).to(DEV)   # general 2x2 matrices, not rotations
    oq, ok = tk.apply_rope(q, k, pe)
    rq, rk = oracle.apply_rope_ref(q, k, pe)
    torch.testing.assert_close(oq, rq, atol=1e-5, rtol=0)
    torch.testing.assert_close(ok, rk, atol=1e-5, rtol=0)


def test_rope_bf16_flux_table_and_per_batch_pe():
    g = seeded(11)
    B, Hh, n_txt, grid = 2, 24, 40, 12
    L = n_txt + grid * grid
    q = randn(g, B, Hh, L, 128, dtype=torch.bfloat16).to(DEV)
    k = randn(g, B, Hh, L, 128, dtype=torch.bfloat16).to(DEV)
    pe = oracle.embed_nd_ref(oracle.flux_ids(n_txt, grid, grid)).to(DEV)
    oq, ok = tk.apply_rope(q, k, pe)
    rq, rk = oracle.apply_rope_ref(q, k, pe)
    torch.testing.assert_close(oq, rq, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(ok, rk, atol=1e-2, rtol=1e-2)
    assert torch.equal(oq[:, :, :n_txt], q[:, :, :n_txt])    # position 0 is the identity rotation
    pe_b = torch.cat((pe, pe.flip(2)), dim=0)                  # a different table per batch element
    oq, ok = tk.apply_rope(q, k, pe_b)
    rq, rk = oracle.apply_rope_ref(q, k, pe_b)
    torch.testing.assert_close(oq, rq, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(ok, rk, atol=1e-2, rtol=1e-2)


def test_rope_table_with_a_head_extent_uses_the_first_head():
    """kernels/positional_embedding.py:31-32 indexes the table by position only, so a [1, H, L, D/2, 2, 2]
    table behaves like its first head's."""
    g = seeded(33)
    B, H, L, D = 2, 3, 40, 64
    q = randn(g, B, H, L, D, dtype=torch.bfloat16).to(DEV)
    k = randn(g, B, H, L, D, dtype=torch.bfloat16).to(DEV)
    pe = randn(g, 1, H, L, D // 2, 2, 2).to(DEV)
    q1, k1 = tk.apply_rope(q, k, pe)
    q0, k0 = tk.apply_rope(q, k, pe[:, :1])
    assert torch.equal(q1, q0) and torch.equal(k1, k0)
    rq, rk = oracle.apply_rope_ref(q, k, pe[:, :1])
    torch.testing.assert_close(q1, rq, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(k1, rk, atol=1e-2, rtol=1e-2)


def test_config3_rope_concat_bit_exact_parts():
    """txt/img concat along the sequence is bit-exact; q,k are rotated on the way, v is copied."""
    txt, img, pe = cfg.config3(DEV, n_txt=64, grid=16)
    q, k, v = tk.qkv_prep(img[0], img[1], img[2], txt[0], txt[1], txt[2])
    for got, t, i in zip((q, k, v), txt, img):
        assert torch.equal(got, torch.cat((t, i), dim=2))
    q2, k2, v2 = tk.qkv_prep(img[0], img[1], img[2], txt[0], txt[1], txt[2], pe=pe)
    rq, rk = oracle.apply_rope_ref(torch.cat((txt[0], img[0]), 2), torch.cat((txt[1], img[1]), 2), pe)
    torch.testing.assert_close(q2, rq, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(k2, rk, atol=1e-2, rtol=1e-2)
    assert torch.equal(v2, torch.cat((txt[2], img[2]), 2))


def test_config3_whole_at_full_size():
    """RoPE with the EmbedND table plus the txt/img concat at the full 512 + 64 x 64 positions, 24 heads:
    one fused launch against the oracle chain (torch.cat along the sequence, then apply_rope), v
    bit-exact, q and k at the bf16 tolerance and at one rounding of the fp32 value; the same through
    the two separate operators (concat, then apply_rope)."""
    txt, img, pe = cfg.config3(DEV)
    assert txt[0].shape == (1, 24, 512, 128) and img[0].shape == (1, 24, 4096, 128) and pe.shape == (1, 1, 4608, 64, 2, 2)
    cat = [torch.cat((t, i), dim=2) for t, i in zip(txt, img)]
    rq, rk = oracle.apply_rope_ref(cat[0], cat[1], pe)
    q, k, v = tk.qkv_prep(img[0], img[1], img[2], txt[0], txt[1], txt[2], pe=pe)
    assert torch.equal(v, cat[2])
    for got, want, src in ((q, rq, cat[0]), (k, rk, cat[1])):
        torch.testing.assert_close(got, want, atol=1e-2, rtol=1e-2)
        # the rotation in fp32 from the bf16 inputs, rounded once
        x_ = src.float().reshape(*src.shape[:-1], -1, 1, 2)
        w32 = (pe[..., 0] * x_[..., 0] + pe[..., 1] * x_[..., 1]).reshape(src.shape)
        assert ((got.float() - w32).abs() <= w32.abs() * 2.0 ** -8 * 1.01 + 1e-6).all()
    # rotations preserve the norm of every (even, odd) pair: |q_rot| == |q| row by row up to rounding
    torch.testing.assert_close(q.float().pow(2).sum(-1), cat[0].float().pow(2).sum(-1), rtol=5e-3, atol=0)
    q0, k0, v0 = tk.qkv_prep(img[0], img[1], img[2], txt[0], txt[1], txt[2])
    assert all(torch.equal(a, b) for a, b in zip((q0, k0, v0), cat))
    q1, k1 = tk.apply_rope(q0, k0, pe)
    assert torch.equal(q1, q) and torch.equal(k1, k)


def test_qkv_prep_norm_rope_matches_unfused_sequence():
    g = seeded(21)
    B, Hh, Lt, Li, D = 2, 6, 37, 91, 128
    txt_qkv = randn(g, B, Lt, 3 * Hh * D, dtype=torch.bfloat16).to(DEV)
    img_qkv = randn(g, B, Li, 3 * Hh * D, dtype=torch.bfloat16).to(DEV)
    scales = [(torch.rand(D, generator=g) + 0.5).to(torch.bfloat16).to(DEV) for _ in range(4)]
    pe = randn(g, 1, 1, Lt + Li, D // 2, 2, 2).to(DEV)
    tq, tk_, tv = oracle.split_heads_ref(txt_qkv, Hh)
    iq, ik, iv = oracle.split_heads_ref(img_qkv, Hh)
    q, k, v = tk.qkv_prep(iq, ik, iv, tq, tk_, tv, pe=pe, q_scale_img=scales[0], k_scale_img=scales[1],
                          q_scale_txt=scales[2], k_scale_txt=scales[3])
    rq = torch.cat((oracle.rms_norm_ref(tq, scales[2]), oracle.rms_norm_ref(iq, scales[0])), 2)
    rk = torch.cat((oracle.rms_norm_ref(tk_, scales[3]), oracle.rms_norm_ref(ik, scales[1])), 2)
    rq, rk = oracle.apply_rope_ref(rq, rk, pe)
    torch.testing.assert_close(q, rq, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(k, rk, atol=1e-2, rtol=1e-2)
    assert torch.equal(v, torch.cat((tv, iv), 2))
