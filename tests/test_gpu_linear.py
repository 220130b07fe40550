"""HIP linear (bf16 MFMA GEMM with fused epilogues) vs the oracle.

Grid and tolerances of the reference's tests/test_linear.py (bf16; atol 1e-5 without activation is
not attainable against a *different* bf16 GEMM on inputs ~N(0,1) with K up to 1024, where one bf16
ulp of the output is 0.25, so the no-activation cases compare against the fp32 result with the
half-ulp bound instead), plus the Flux shapes at atol 2e-2 vs fp32, ragged shapes, and every
epilogue the fused blocks use.
"""
import math

import pytest
import torch

import triton_kernels as tk
from oracle import flux_oracle as oracle
from triton_kernels import testing as cfg
from triton_kernels.kernels import qk_fusable
from util import DEV, randn, seeded

pytestmark = pytest.mark.gpu


def half_ulp_bound(ref_fp32: torch.Tensor) -> torch.Tensor:
    """One correct rounding to bf16 is off by at most half an ulp <= 2^-8 |x|. On top of that the
    fp32 sum itself depends on the order of accumulation: an absolute term for results that cancel
    to nearly zero and 1% slack for results that sit on a rounding boundary."""
    return ref_fp32.abs() * (2.0 ** -8 * 1.01) + 2e-3


@pytest.mark.parametrize("batch_size", [1, 4])
@pytest.mark.parametrize("seq_len", [256, 1024])
@pytest.mark.parametrize("in_channel", [256, 1024])
@pytest.mark.parametrize("out_channel", [1024, 3072])
@pytest.mark.parametrize("activation", ["", "GELU"])
def test_linear_reference_grid(batch_size, seq_len, in_channel, out_channel, activation):
    g = seeded(batch_size + seq_len + in_channel + out_channel)
    x = randn(g, batch_size, seq_len, in_channel, dtype=torch.bfloat16).to(DEV)
    w = randn(g, out_channel, in_channel, dtype=torch.bfloat16).to(DEV)
    b = randn(g, out_channel, dtype=torch.bfloat16).to(DEV)
    y = tk.linear(x, w, b, activation=activation)
    assert y.shape == (batch_size, seq_len, out_channel) and y.dtype == torch.bfloat16
    ref32 = oracle.linear_ref_fp32(x, w, b, activation)
    assert ((y.float() - ref32).abs() <= half_ulp_bound(ref32)).all()
    if activation == "GELU":
        # the reference's own comparison (tests/test_linear.py:21-27: bf16 F.linear then F.gelu, atol 0.02);
        # that oracle rounds twice, so where |y| is large it may sit one bf16 ulp away
        ref = oracle.linear_ref(x, w, b, activation).float()
        assert ((y.float() - ref).abs() <= 0.02 + ref.abs() * 2.0 ** -7).all()


@pytest.mark.parametrize("which,act", [("mlp_in", "GELU"), ("proj_out", ""), ("linear1", "")])
def test_linear_flux_shapes_vs_fp32(which, act):
    """All three Flux GEMMs through the public operator at the full 4608 rows, plain epilogue (bias,
    optional GELU), against the fp32 product at the stated 2e-2 and at the half-ulp bound."""
    a, w, b = cfg.config4(DEV, which, m=4608)
    y = tk.linear(a, w, b, activation=act)
    ref32 = oracle.linear_ref_fp32(a, w, b, act)
    torch.testing.assert_close(y.float(), ref32, atol=2e-2, rtol=0)
    assert ((y.float() - ref32).abs() <= half_ulp_bound(ref32)).all()


@pytest.mark.parametrize("M,N,K", [(1, 9216, 3072), (2, 1000, 512), (7, 33, 64), (8, 18432, 3072), (9, 40, 72),
                                   (130, 70, 200), (257, 513, 136), (300, 256, 8), (64, 64, 1000), (513, 1025, 264)])
@pytest.mark.parametrize("bias", [True, False])
def test_linear_ragged_shapes(M, N, K, bias):
    g = seeded(M * 3 + N * 5 + K)
    x = randn(g, M, K, dtype=torch.bfloat16).to(DEV)
    w = randn(g, N, K, dtype=torch.bfloat16, std=K ** -0.5).to(DEV)
    b = randn(g, N, dtype=torch.bfloat16).to(DEV) if bias else None
    y = tk.linear(x, w, b)
    ref32 = oracle.linear_ref_fp32(x, w, b)
    assert ((y.float() - ref32).abs() <= half_ulp_bound(ref32)).all()


@pytest.mark.parametrize("B,L,N,K,act,bias,gated", [
    (1, 4608, 3072, 512, "", True, True),       # linear2's output shape: 256 tiles of 288 x 192, gated residual
    (2, 1152, 6144, 200, "", False, True),      # K tail, two batch elements of four tile rows each, no bias
    (1, 2304, 6144, 136, "GELU", True, False),  # GELU on every column
    (1, 2304, 6144, 64, "", True, False),       # a single slab
    (1, 4608, 3072, 8, "", True, False),        # less than a slab
    (1, 4096, 3072, 512, "", True, True),       # the double block's img tails: 256 tiles of 256 x 192, gated residual
    (2, 2048, 3072, 200, "", False, True),      # K tail, two batch elements of eight tile rows each, no bias
    (1, 2048, 6144, 136, "GELU", True, False),  # GELU on every column, 256 x 192
    (1, 4096, 9216, 64, "", True, False),       # the double block's img qkv shape: three exact rounds, a single slab
    (1, 4096, 3072, 8, "", True, False),        # less than a slab
    (1, 2816, 3072, 320, "GELU", True, False),  # too few square tiles, two rounds of 128-wide ones: 176 tiles of 256 x 192
])
def test_linear_rectangular_tiles(B, L, N, K, act, bias, gated):
    """Shapes that 288 x 192 or 256 x 192 tiles divide and that fill the 256 CUs better on them than on
    square ones take the rectangular-tile kernel: every epilogue it has, with and without a K tail."""
    g = seeded(B * L + N + K)
    M = B * L
    a = randn(g, M, K, dtype=torch.bfloat16).to(DEV)
    w = randn(g, N, K, dtype=torch.bfloat16, std=K ** -0.5).to(DEV)
    b = randn(g, N, dtype=torch.bfloat16, std=0.5).to(DEV) if bias else None
    ref32 = oracle.linear_ref_fp32(a, w, b, act)
    if not gated:
        y = tk.linear(a, w, b, activation=act)
        assert ((y.float() - ref32).abs() <= half_ulp_bound(ref32)).all()
        return
    x = randn(g, B, L, N, dtype=torch.bfloat16).to(DEV)
    gate = randn(g, B, 1, N, dtype=torch.bfloat16).to(DEV)
    out = torch.empty_like(x)
    tk.linear_into(a, w, b, out=out.view(M, N), resid=x.view(M, N), gate=gate)
    gy = gate.float() * ref32.view(B, L, N)
    want32 = x.float() + gy
    bound = 2.0 ** -8 * 1.01 * (2 * gy.abs() + want32.abs()) + 2e-3
    assert ((out.float() - want32).abs() <= bound).all()
    # and exactly the two PyTorch ops on the kernel's own (once rounded) product
    y = tk.linear(a, w, b)
    assert torch.equal(out, oracle.gated_residual_ref(x, gate, y.view(B, L, N)))


@pytest.mark.parametrize("M,N,K", [(4096, 3072, 192), (4608, 3072, 200), (512, 3072, 256)])
def test_linear_shared_gpu_flag_changes_the_schedule_only(M, N, K):
    """FLUX_LINEAR_SHARED_GPU keeps the square tiles where the library would otherwise fill the CUs
    exactly with rectangular ones; both orders of accumulation are the same, so are the bits."""
    g = seeded(M + K)
    a = randn(g, M, K, dtype=torch.bfloat16).to(DEV)
    w = randn(g, N, K, dtype=torch.bfloat16, std=K ** -0.5).to(DEV)
    b = randn(g, N, dtype=torch.bfloat16, std=0.5).to(DEV)
    y0 = tk.linear_into(a, w, b, activation="GELU")
    y1 = tk.linear_into(a, w, b, activation="GELU", shared_gpu=True)
    assert torch.equal(y0, y1)
    assert ((y1.float() - oracle.linear_ref_fp32(a, w, b, "GELU")).abs() <= half_ulp_bound(oracle.linear_ref_fp32(a, w, b, "GELU"))).all()


def test_linear_unaligned_k_and_strided_input():
    g = seeded(3)
    x = randn(g, 50, 77, dtype=torch.bfloat16).to(DEV)       # K = 77: no 16-byte rows
    w = randn(g, 30, 77, dtype=torch.bfloat16, std=0.1).to(DEV)
    y = tk.linear(x, w, None)
    torch.testing.assert_close(y.float(), oracle.linear_ref_fp32(x, w, None), atol=2e-2, rtol=1e-2)
    big = randn(g, 300, 1024, dtype=torch.bfloat16).to(DEV)
    xs = big[:, 256:768]                                      # row stride 1024, K = 512
    w = randn(g, 384, 512, dtype=torch.bfloat16, std=512 ** -0.5).to(DEV)
    torch.testing.assert_close(tk.linear(xs, w, None).float(), oracle.linear_ref_fp32(xs, w, None), atol=2e-2, rtol=0)


def test_linear_rejects_fp32_like_the_reference():
    x = torch.zeros(4, 8, device=DEV)
    with pytest.raises(KeyError):
        tk.linear(x, torch.zeros(16, 8, device=DEV), None)


@pytest.mark.parametrize("M,hid,mlp", [(512, 256, 1024), (300, 128, 512), (4608, 3072, 12288)])
def test_linear_split_gelu_epilogue(M, hid, mlp):
    """linear1 of the single block: columns [0, 3*hid) plain -> out, columns [3*hid, ..) GELU -> out2."""
    g = seeded(M + hid)
    x = randn(g, M, hid, dtype=torch.bfloat16).to(DEV)
    w = randn(g, 3 * hid + mlp, hid, dtype=torch.bfloat16, std=hid ** -0.5).to(DEV)
    b = randn(g, 3 * hid + mlp, dtype=torch.bfloat16, std=0.02).to(DEV)
    qkv = torch.empty(M, 3 * hid, dtype=torch.bfloat16, device=DEV)
    both = torch.zeros(M, hid + mlp, dtype=torch.bfloat16, device=DEV)
    tk.linear_into(x, w, b, activation="GELU", act_begin=3 * hid, out=qkv, out2=both[:, hid:], split=3 * hid)
    ref32 = oracle.linear_ref_fp32(x, w, b)
    torch.testing.assert_close(qkv.float(), ref32[:, :3 * hid], atol=2e-2, rtol=0)
    want_mlp = oracle.gelu_tanh_ref(ref32[:, 3 * hid:])
    torch.testing.assert_close(both[:, hid:].float(), want_mlp, atol=2e-2, rtol=0)
    assert (both[:, :hid] == 0).all()                        # the attention half is left alone


@pytest.mark.parametrize("B,L,hid,K", [(1, 512, 256, 1280), (2, 300, 128, 640), (1, 4608, 3072, 15360)])
def test_linear_gated_residual_epilogue(B, L, hid, K):
    g = seeded(B + L + hid)
    a = randn(g, B * L, K, dtype=torch.bfloat16).to(DEV)
    w = randn(g, hid, K, dtype=torch.bfloat16, std=K ** -0.5).to(DEV)
    b = randn(g, hid, dtype=torch.bfloat16, std=0.02).to(DEV)
    x = randn(g, B, L, hid, dtype=torch.bfloat16).to(DEV)
    mod = randn(g, B, 3 * hid, dtype=torch.bfloat16).to(DEV)
    gate = mod[:, None, :].chunk(3, dim=-1)[2]
    out = torch.empty_like(x)
    tk.linear_into(a, w, b, out=out.view(B * L, hid), resid=x.view(B * L, hid), gate=gate)
    y32 = oracle.linear_ref_fp32(a, w, b).view(B, L, hid)
    # the two-op oracle (x + gate * y, modules/blocks.py:123) on the rounded product: y may sit on the
    # other side of a bf16 rounding boundary than the kernel's, which |gate| then magnifies
    want = oracle.gated_residual_ref(x, gate, y32.to(torch.bfloat16))
    torch.testing.assert_close(out, want, atol=4e-2, rtol=1e-2)
    # element-wise bound against the unrounded fp32 value: the kernel rounds y, gate * y and the sum,
    # each by at most half an ulp (2^-8 relative) of its own magnitude
    gy = gate.float() * y32
    want32 = x.float() + gy
    bound = 2.0 ** -8 * 1.01 * (2 * gy.abs() + want32.abs()) + 2e-3
    err = (out.float() - want32).abs()
    assert (err <= bound).all(), f"max excess {(err - bound).max().item()}"
    assert err.mean().item() < 6e-3


@pytest.mark.parametrize("B,L,H,mlp,bias,per_batch_pe", [(2, 256, 3, 1152, True, False), (1, 512, 2, 256, False, False),
                                                         (2, 256, 2, 256, True, True), (1, 4608, 24, 12288, True, False),
                                                         # ragged: rows and sequence length no multiple of the tile, tiles that
                                                         # hold the end of one batch element and the start of the next
                                                         (3, 300, 2, 256, True, True), (2, 421, 3, 1152, False, False),
                                                         (1, 333, 2, 256, True, False), (3, 4336, 24, 12288, True, False)])
def test_linear_qk_norm_rope_epilogue(B, L, H, mlp, bias, per_batch_pe):
    """linear1 with QKNorm + RoPE in the epilogue: q and k leave as [B,H,L,128], v and the GELU'd mlp
    columns as in the split epilogue. Checked against the oracle chain on the un-fused projection
    and against the preparation kernel the block otherwise runs."""
    D, hid = 128, H * 128
    M, N = B * L, 3 * hid + mlp
    g = seeded(L + H)
    x = randn(g, M, hid, dtype=torch.bfloat16).to(DEV)
    w = randn(g, N, hid, dtype=torch.bfloat16, std=hid ** -0.5).to(DEV)
    b = randn(g, N, dtype=torch.bfloat16, std=0.02).to(DEV) if bias else None
    qs = (torch.rand(D, generator=g) + 0.5).to(torch.bfloat16).to(DEV)
    ks = (torch.rand(D, generator=g) + 0.5).to(torch.bfloat16).to(DEV)
    pe = randn(g, B if per_batch_pe else 1, 1, L, D // 2, 2, 2).to(DEV)

    qkv = torch.zeros(M, 3 * hid, dtype=torch.bfloat16, device=DEV)
    both = torch.zeros(M, hid + mlp, dtype=torch.bfloat16, device=DEV)
    q = torch.empty(B, H, L, D, dtype=torch.bfloat16, device=DEV)
    k = torch.empty_like(q)
    assert qk_fusable(x, w, L, D) == (-(-M // 256) * (N // 256) >= 160)   # small ones are taken, just not preferred
    tk.linear_into(x, w, b, activation="GELU", act_begin=3 * hid, out=qkv, out2=both[:, hid:], split=3 * hid,
                   qk=dict(q_out=q, k_out=k, q_scale=qs, k_scale=ks, pe=pe, heads=H, seq_len=L, eps=1e-6))

    # un-fused: the same projection, then the preparation kernel
    qkv_u = torch.empty_like(qkv)
    both_u = torch.zeros_like(both)
    tk.linear_into(x, w, b, activation="GELU", act_begin=3 * hid, out=qkv_u, out2=both_u[:, hid:], split=3 * hid)
    assert torch.equal(qkv[:, 2 * hid:], qkv_u[:, 2 * hid:])           # v columns: same code path, same bits
    assert torch.equal(both, both_u)
    assert (qkv[:, :2 * hid] == 0).all()                               # q and k columns are not written
    heads = qkv_u.view(B, L, 3, H, D).permute(2, 0, 3, 1, 4)
    q_u, k_u, _ = tk.qkv_prep(heads[0], heads[1], None, pe=pe, q_scale_img=qs, k_scale_img=ks)
    # oracle chain on the bf16 projection
    qn = oracle.rms_norm_ref(heads[0].cpu(), qs.cpu())
    kn = oracle.rms_norm_ref(heads[1].cpu(), ks.cpu())
    rq, rk = oracle.apply_rope_ref(qn, kn, pe.cpu())

    def close(got, want, normed, atol, rtol):
        """atol + rtol |want|, plus what one bf16 ulp of a normalised value is worth behind the 2 x 2 matrix:
        where x * rstd falls on a rounding boundary two correct evaluations may round it either way, and
        the table here is random (entries of several units, rows that cancel), which magnifies that ulp."""
        xn = normed.float().reshape(*normed.shape[:-1], -1, 1, 2).abs()
        amp = (pe.cpu().float().abs() * xn).sum(-1).reshape(normed.shape)
        err = (got.cpu().float() - want.cpu().float()).abs()
        assert (err <= atol + rtol * want.cpu().float().abs() + 2.0 ** -7 * amp).all(), err.max().item()
        assert err.mean().item() < 2e-3

    close(q, q_u, qn, 1e-2, 1e-2)
    close(k, k_u, kn, 1e-2, 1e-2)
    close(q, rq, qn, 2e-2, 2e-2)
    close(k, rk, kn, 2e-2, 2e-2)


@pytest.mark.parametrize("M", [1, 2, 5, 8])
@pytest.mark.parametrize("N,K", [(9216, 3072), (18432, 3072), (40, 72), (33, 50)])
def test_linear_input_silu_is_modulation(M, N, K):
    """lin(silu(vec)) of Modulation (modules/blocks.py:62-67) as one launch: SiLU in fp32 rounded to bf16
    on the way in, bit-identical to the two-launch form and within tolerance of the oracle."""
    from triton_kernels.modules.blocks import _silu
    g = seeded(M + N + K)
    vec = randn(g, M, K, dtype=torch.bfloat16, std=2.0).to(DEV)
    w = randn(g, N, K, dtype=torch.bfloat16, std=K ** -0.5).to(DEV)
    b = randn(g, N, dtype=torch.bfloat16, std=0.02).to(DEV)
    fused = tk.linear_into(vec, w, b, in_activation="SiLU")
    two = tk.linear(_silu(vec), w, b)
    assert torch.equal(fused, two)
    ref32 = oracle.linear_ref_fp32(oracle.silu_ref(vec), w, b)
    torch.testing.assert_close(fused.float(), ref32, atol=2e-2, rtol=1e-2)


def test_linear_input_silu_needs_few_rows_and_modulation_uses_it():
    g = seeded(3)
    vec = randn(g, 9, 64, dtype=torch.bfloat16).to(DEV)
    w = randn(g, 32, 64, dtype=torch.bfloat16).to(DEV)
    with pytest.raises(AssertionError):
        tk.linear_into(vec, w, None, in_activation="SiLU")
    from triton_kernels.modules.blocks import Modulation
    torch.manual_seed(0)
    mod = Modulation(256, double=True).to(torch.bfloat16).to(DEV)
    for rows in (1, 3, 9):                                    # 9 rows: the two-launch form
        v = randn(g, rows, 256, dtype=torch.bfloat16).to(DEV)
        m1, m2 = mod(v)
        want = oracle.linear_ref_fp32(oracle.silu_ref(v), mod.lin.weight, mod.lin.bias)[:, None, :].chunk(6, dim=-1)
        for got, ref in zip((m1.shift, m1.scale, m1.gate, m2.shift, m2.scale, m2.gate), want):
            assert got.shape == (rows, 1, 256)
            torch.testing.assert_close(got.float(), ref, atol=2e-2, rtol=1e-2)
        mod.fused_silu = False
        u1, _ = mod(v)
        mod.fused_silu = True
        assert torch.equal(u1.scale, m1.scale)


@pytest.mark.parametrize("gated", [False, True])
def test_linear_head_and_tail_launches(gated):
    """4608 x 12288 outputs are 864 tiles of 256 x 256, 3.375 rounds of 256 CUs: the library launches the
    first 4096 rows on those tiles and the last 512 rows on 128-wide ones. Same results as one launch
    would give: compared with the fp32 product row block by row block."""
    g = seeded(77 + gated)
    M, N, K = 4608, 12288, 192
    a = randn(g, M, K, dtype=torch.bfloat16).to(DEV)
    w = randn(g, N, K, dtype=torch.bfloat16, std=K ** -0.5).to(DEV)
    b = randn(g, N, dtype=torch.bfloat16, std=0.02).to(DEV)
    if not gated:
        y = tk.linear(a, w, b, activation="GELU")
        ref32 = oracle.linear_ref_fp32(a, w, b, "GELU")
        assert ((y.float() - ref32).abs() <= half_ulp_bound(ref32)).all()
        return
    B, L = 9, 512                                               # the cut at row 4096 falls between batch elements
    x = randn(g, B, L, N, dtype=torch.bfloat16).to(DEV)
    gate = randn(g, B, 1, N, dtype=torch.bfloat16).to(DEV)
    out = torch.empty_like(x)
    tk.linear_into(a, w, b, out=out.view(M, N), resid=x.view(M, N), gate=gate)
    gy = gate.float() * oracle.linear_ref_fp32(a, w, b).view(B, L, N)
    want32 = x.float() + gy
    bound = 2.0 ** -8 * 1.01 * (2 * gy.abs() + want32.abs()) + 2e-3
    assert ((out.float() - want32).abs() <= bound).all()
