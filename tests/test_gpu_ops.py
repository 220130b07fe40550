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
