"""The raw `ops` kernels under their reference names and launch spelling, vs the oracle."""
import pytest
import torch

from oracle import flux_oracle as oracle
from triton_kernels import ops
from util import DEV, randn, seeded

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("numel", [1, 7, 3072, 100003])
def test_silu(dtype, numel):
    x = randn(seeded(numel), numel, dtype=dtype, std=3.0).to(DEV)
    y = torch.empty_like(x)
    ops.triton_silu[(1,)](x, y, numel, XBLOCK=1024)
    torch.testing.assert_close(y, oracle.silu_ref(x), atol=1e-2 if dtype == torch.bfloat16 else 1e-5, rtol=1e-2 if dtype == torch.bfloat16 else 1e-5)


@pytest.mark.parametrize("is_mod1", [True, False])
def test_modulation_scale_shift_and_gate(is_mod1):
    g = seeded(4)
    B, L, hid = 2, 50, 384
    x = randn(g, B, L, hid, dtype=torch.bfloat16).to(DEV)
    mod = randn(g, B, 6 * hid, dtype=torch.bfloat16).to(DEV)
    out = torch.empty_like(x)
    ops.triton_modulation_scale_shift[(1,)](x, mod, out, L * hid, hid, 6 * hid, is_mod1, XBLOCK=512)
    torch.testing.assert_close(out, oracle.modulation_scale_shift_ref(x, mod, is_mod1), atol=1e-2, rtol=1e-2)
    proj = randn(g, B, L, hid, dtype=torch.bfloat16).to(DEV)
    ops.triton_modulation_gate_proj(x, mod, proj, out, L * hid, hid, 6 * hid, XBLOCK=512)
    torch.testing.assert_close(out, oracle.modulation_gate_proj_ref(x, mod, proj), atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("B,H,D,Lt,Li", [(1, 24, 128, 512, 4096), (2, 3, 64, 5, 11), (1, 2, 128, 0, 33)])
def test_qkv_concat_bit_exact(B, H, D, Lt, Li):
    g = seeded(B + H + D + Lt + Li)
    hid = H * D
    txt = randn(g, B, max(Lt, 1), 3 * hid, dtype=torch.bfloat16).to(DEV)[:, :Lt]
    img = randn(g, B, Li, 3 * hid, dtype=torch.bfloat16).to(DEV)
    L = Lt + Li
    q, k, v = (torch.empty(B, H, L, D, dtype=torch.bfloat16, device=DEV) for _ in range(3))
    ops.triton_qkv_concat[(1,)](txt, img, q, k, v, L, H, D, hid, Lt,
                                Lt * 3 * hid if Lt else None, 3 * hid if Lt else None, Li * 3 * hid, 3 * hid,
                                H * L * D, L * D, D, XBLOCK=1024)
    rq, rk, rv = oracle.qkv_concat_ref(txt, img, H)
    assert torch.equal(q, rq) and torch.equal(k, rk) and torch.equal(v, rv)


def test_triton_linear_bias_suffix():
    g = seeded(6)
    M, N, K = 200, 320, 256
    a = randn(g, M, K, dtype=torch.bfloat16).to(DEV)
    w = randn(g, N, K, dtype=torch.bfloat16, std=K ** -0.5).to(DEV)
    c = randn(g, N, dtype=torch.bfloat16).to(DEV)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    b = w.t()                                                  # [K, N] view: stride_bk = 1, stride_bn = K
    ops.triton_linear[(1,)](a, b, c, out, M, N, K, a.stride(0), a.stride(1), b.stride(0), b.stride(1),
                            GROUP_M=8, EVEN_K=True, ALLOW_TF32=False, ACC_TYPE=None, B_PROLOGUE_CAST_TYPE=None,
                            BLOCK_M=128, BLOCK_N=128, BLOCK_K=32)
    torch.testing.assert_close(out.float(), oracle.linear_ref_fp32(a, w, c), atol=2e-2, rtol=0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,n,ld", [(1, 8, 8), (5, 384, 384), (300, 1024, 1280), (4608, 12288, 21504), (7, 100, 333)])
def test_gelu_tanh_strided_rows(dtype, rows, n, ld):
    """flux_gelu_tanh on a [rows, n] view of wider rows: nn.GELU(approximate="tanh") on the mlp half
    of linear1's output (modules/blocks.py:107,122)."""
    from triton_kernels.modules.blocks import _gelu_tanh
    wide = randn(seeded(rows + n), rows, ld, dtype=dtype, std=2.0).to(DEV)
    x = wide[:, ld - n:]
    assert x.is_contiguous() == (ld == n or rows == 1)
    y = _gelu_tanh(x)
    assert y.is_contiguous() and y.shape == x.shape
    ref = oracle.gelu_tanh_ref(x.float())
    if dtype == torch.float32:
        torch.testing.assert_close(y, ref, atol=2e-6, rtol=1e-5)
    else:
        assert ((y.float() - ref).abs() <= ref.abs() * 2.0 ** -8 * 1.01 + 1e-6).all()   # one rounding of the fp32 value
    # a 3-d view, as the block passes it
    if rows % 5 == 0:
        x3 = wide.view(5, rows // 5, ld)[..., ld - n:]
        assert torch.equal(_gelu_tanh(x3).view(rows, n), y)


@pytest.mark.parametrize("B,L,hid", [(1, 4608, 3072), (2, 77, 384), (3, 1, 8)])
def test_gated_residual_rounds_the_product(B, L, hid):
    """flux_gate_residual with round_product = 1: exactly what the two PyTorch ops x + gate * y of
    modules/blocks.py:123,166-171 produce in bf16 (product rounded, then the sum rounded)."""
    from triton_kernels.modules.blocks import _gated_residual
    g = seeded(B + L + hid)
    x = randn(g, B, L, hid, dtype=torch.bfloat16).to(DEV)
    y = randn(g, B, L, hid, dtype=torch.bfloat16).to(DEV)
    mod = randn(g, B, 1, 3 * hid, dtype=torch.bfloat16).to(DEV)
    gate = mod.chunk(3, dim=-1)[2]                              # a strided [B, 1, hid] chunk of the modulation vector
    out = _gated_residual(x, gate, y)
    assert torch.equal(out, oracle.gated_residual_ref(x, gate, y))
    # and it differs from the single-rounding form somewhere, i.e. the flag does something
    if B * L * hid > 10000:
        once = (x.float() + gate.float() * y.float()).to(torch.bfloat16)
        assert not torch.equal(out, once)
