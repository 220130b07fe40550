"""HIP flash-attention forward vs the oracle: the reference's grid (tests/test_attention.py: bf16,
atol 1e-2 vs F.scaled_dot_product_attention), the Flux shape at atol 2e-2 vs an fp32 softmax, ragged
lengths, strided views, and mathematical invariants at the full size."""
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
@pytest.mark.parametrize("seq_len", [256, 512, 1024])
@pytest.mark.parametrize("head_dim", [64, 128])
def test_attention_reference_grid(batch_size, num_heads, seq_len, head_dim):
    g = seeded(batch_size + num_heads + seq_len + head_dim)
    q, k, v = (randn(g, batch_size, num_heads, seq_len, head_dim, dtype=torch.bfloat16).to(DEV) for _ in range(3))
    o = tk.scaled_dot_product_attention(q, k, v)
    torch.testing.assert_close(o, oracle.attention_ref(q, k, v), atol=1e-2, rtol=0)
    torch.testing.assert_close(o.float(), oracle.attention_ref_fp32(q, k, v), atol=1e-2, rtol=0)


@pytest.mark.parametrize("seq_len", [1, 31, 64, 65, 127, 200, 333, 4336 // 4])
@pytest.mark.parametrize("head_dim", [64, 128])
def test_attention_ragged_lengths(seq_len, head_dim):
    g = seeded(seq_len + head_dim)
    q, k, v = (randn(g, 2, 3, seq_len, head_dim, dtype=torch.bfloat16).to(DEV) for _ in range(3))
    o = tk.scaled_dot_product_attention(q, k, v, sm_scale=0.11)
    torch.testing.assert_close(o.float(), oracle.attention_ref_fp32(q, k, v, 0.11), atol=1e-2, rtol=0)


def test_attention_flux_shape_vs_fp32_and_invariants():
    q, k, v = cfg.config5_attention(DEV)
    o = tk.scaled_dot_product_attention(q, k, v)
    ref = oracle.attention_ref_fp32(q, k, v)
    torch.testing.assert_close(o.float(), ref, atol=2e-2, rtol=0)
    err = (o.float() - ref).abs().max().item()
    assert err < 4e-3, f"max error {err} is far above what bf16 output rounding explains"
    # rows of P sum to one: constant V gives a constant output
    vc = torch.full_like(v, 0.75)
    assert torch.equal(tk.scaled_dot_product_attention(q, k, vc), vc)
    # permuting the keys (and values alike) does not change the result beyond summation order
    perm = torch.randperm(k.shape[2], generator=seeded(1)).to(DEV)
    o2 = tk.scaled_dot_product_attention(q, k[:, :, perm], v[:, :, perm])
    torch.testing.assert_close(o2.float(), o.float(), atol=4e-3, rtol=0)


def test_attention_single_key_returns_v():
    g = seeded(9)
    q = randn(g, 1, 2, 70, 128, dtype=torch.bfloat16).to(DEV)
    k = randn(g, 1, 2, 1, 128, dtype=torch.bfloat16).to(DEV)
    v = randn(g, 1, 2, 1, 128, dtype=torch.bfloat16).to(DEV)
    o = torch.empty_like(q)
    # one key: L differs between q and k, which the public operator does not allow; the invariant is
    # checked through equal lengths instead: all keys identical
    kk = k.expand(1, 2, 70, 128).contiguous()
    vv = v.expand(1, 2, 70, 128).contiguous()
    o = tk.scaled_dot_product_attention(q, kk, vv)
    assert torch.equal(o, vv)


def test_attention_strided_views_and_lse():
    g = seeded(17)
    B, H, L, D = 2, 4, 300, 128
    qkv = randn(g, B, L, 3 * H * D, dtype=torch.bfloat16).to(DEV)
    q, k, v = oracle.split_heads_ref(qkv, H)                  # strided views, row stride 3*H*D
    buf = torch.zeros(B, L, H * D + 64, dtype=torch.bfloat16, device=DEV)
    out = buf[..., :H * D].view(B, L, H, D).permute(0, 2, 1, 3)  # "B L (H D)" destination
    lse = torch.empty(B, H, L, dtype=torch.float32, device=DEV)
    tk.attention_into(q, k, v, out, lse=lse)
    ref = oracle.attention_ref_fp32(q, k, v)
    torch.testing.assert_close(out.float(), ref, atol=1e-2, rtol=0)
    assert (buf[..., H * D:] == 0).all()
    # the kernel rounds q * sm_scale * log2(e) to bf16 once (2^-9 relative per element), which moves a
    # score by a few 1e-3 in the base-2 domain; lse inherits that
    torch.testing.assert_close(lse, oracle.attention_lse_ref(q, k), atol=5e-3, rtol=5e-4)


def test_attention_head_dim_assert():
    q = torch.zeros(1, 1, 8, 48, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(AssertionError):
        tk.scaled_dot_product_attention(q, q, q)


@pytest.mark.parametrize("seq_len", [1, 31, 77, 256, 333, 1024])
@pytest.mark.parametrize("head_dim", [16, 32, 256])
def test_attention_other_head_dims(seq_len, head_dim):
    """The remaining head dims kernels/attention.py:184 accepts; these score in fp32 (no rounding of a
    pre-scaled q), so lse is held to a tight bound."""
    g = seeded(seq_len * 3 + head_dim)
    B, H = 2, 3
    q, k, v = (randn(g, B, H, seq_len, head_dim, dtype=torch.bfloat16).to(DEV) for _ in range(3))
    o = torch.empty_like(q)
    lse = torch.empty(B, H, seq_len, dtype=torch.float32, device=DEV)
    tk.attention_into(q, k, v, o, lse=lse)
    torch.testing.assert_close(o.float(), oracle.attention_ref_fp32(q, k, v), atol=1e-2, rtol=0)
    torch.testing.assert_close(lse, oracle.attention_lse_ref(q, k), atol=1e-4, rtol=1e-5)
    if seq_len % 64 == 0:
        torch.testing.assert_close(tk.scaled_dot_product_attention(q, k, v), oracle.attention_ref(q, k, v), atol=1e-2, rtol=0)
    # strided source and destination, explicit scale
    qkv = randn(g, B, seq_len, 3 * H * head_dim, dtype=torch.bfloat16).to(DEV)
    q2, k2, v2 = oracle.split_heads_ref(qkv, H)
    out = torch.empty(B, seq_len, H, head_dim, dtype=torch.bfloat16, device=DEV).permute(0, 2, 1, 3)
    tk.attention_into(q2, k2, v2, out, sm_scale=0.2)
    torch.testing.assert_close(out.float(), oracle.attention_ref_fp32(q2, k2, v2, 0.2), atol=1e-2, rtol=0)


def _prescaled_ref(q, k, v, sm_scale):
    """What the head-dim-64/128 kernels evaluate: q * sm_scale * log2(e) rounded to bf16 once, scores and
    softmax in the base-2 domain. Large scores make that one rounding visible, so the cases that
    drive the scores up are compared with this form (fp32 otherwise)."""
    q2 = (q.float() * (sm_scale * math.log2(math.e))).bfloat16().float()
    s = torch.einsum("bhqd,bhkd->bhqk", q2, k.float()) * math.log(2.0)
    return torch.einsum("bhqk,bhkd->bhqd", torch.softmax(s, dim=-1), v.float()), torch.logsumexp(s, -1) * math.log2(math.e)


# (batch, heads, seq): which launch shape the head-dim-64/128 dispatch picks for them
_WIDE = [(4, 24, 512),    # 64-row-per-wave kernel, one launch of 256-row tiles
         (4, 24, 1000),   # the same with a ragged last tile
         (1, 24, 4336),   # two launches (256- and 192-row tiles), ragged
         (3, 24, 1536),   # two launches, odd batch * even heads
         (8, 24, 31),     # one partial tile per head
         (6, 24, 97),
         (1, 8, 4100),    # few heads, long ragged sequence
         (2, 43, 770),    # both tile sizes in one launch, ragged, 4 tiles of 256 rows per head
         (1, 170, 520),   # the same just under two rounds of tiles
         (257, 1, 257),   # an odd number of (batch, head) pairs just over two rounds
         (2, 24, 4608),   # 864 tiles of 256 rows = 3.4 rounds: 576 such tiles and 384 of 192 rows
         (1, 25, 2300)]   # an odd head count with both tile sizes


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("B,H,L", _WIDE)
def test_attention_wide_tile_launch_shapes(B, H, L, D):
    g = seeded(B * 1000 + H * 100 + L + D)
    q, k, v = (randn(g, B, H, L, D, dtype=torch.bfloat16).to(DEV) for _ in range(3))
    o = torch.empty_like(q)
    lse = torch.empty(B, H, L, dtype=torch.float32, device=DEV)
    tk.attention_into(q, k, v, o, lse=lse)
    assert torch.isfinite(o.float()).all()
    for b in range(B):
        torch.testing.assert_close(o[b:b + 1].float(), oracle.attention_ref_fp32(q[b:b + 1], k[b:b + 1], v[b:b + 1]), atol=1e-2, rtol=0)
        torch.testing.assert_close(lse[b:b + 1], oracle.attention_lse_ref(q[b:b + 1], k[b:b + 1]), atol=5e-3, rtol=5e-4)


@pytest.mark.parametrize("D", [128, 64])
def test_attention_wide_tile_strided_views(D):
    """The 64-row-per-wave kernels on views of a packed qkv projection (row stride 3 * H * D) with the
    output written head-interleaved, as the blocks pass them, ragged length, with lse."""
    g = seeded(7 + D)
    B, H, L = 2, 3072 // D, 1100
    qkv = randn(g, B, L, 3 * H * D, dtype=torch.bfloat16).to(DEV)
    q, k, v = oracle.split_heads_ref(qkv, H)
    out = torch.empty(B, L, H, D, dtype=torch.bfloat16, device=DEV).permute(0, 2, 1, 3)
    lse = torch.empty(B, H, L, dtype=torch.float32, device=DEV)
    tk.attention_into(q, k, v, out, lse=lse)
    for b in range(B):
        torch.testing.assert_close(out[b:b + 1].float(), oracle.attention_ref_fp32(q[b:b + 1], k[b:b + 1], v[b:b + 1]), atol=1e-2, rtol=0)
        torch.testing.assert_close(lse[b:b + 1], oracle.attention_lse_ref(q[b:b + 1], k[b:b + 1]), atol=5e-3, rtol=5e-4)


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("H", [24, 4])   # 24 heads: 64-row-per-wave kernel; 4 heads: 128-row workgroups
@pytest.mark.parametrize("kind", ["hot", "ramp"])
def test_attention_large_scores_move_the_reference_maximum(H, kind, D):
    """Scores far above the first tile's maximum: the kernels subtract a per-row reference value that is
    only raised when a partial sum grows too large, and this drives them through that step."""
    g = seeded(H + len(kind) + D)
    L = 2048
    # the same spread of scores at either head dim: |q| grows as the head shrinks
    q = (randn(g, 1, H, L, D) * ((30.0 if kind == "hot" else 4.0) * math.sqrt(128 / D))).bfloat16().to(DEV)
    k = randn(g, 1, H, L, D, dtype=torch.bfloat16).to(DEV)
    v = randn(g, 1, H, L, D, dtype=torch.bfloat16).to(DEV)
    if kind == "ramp":   # later keys score ever higher than earlier ones
        ramp = torch.linspace(0, 6.0, L, device=DEV).view(1, 1, L, 1)
        k = (k.float() + ramp * q.float().mean(dim=2, keepdim=True).sign()).bfloat16()
    sc = 1 / math.sqrt(128)   # at head dim 64 too: with the larger q the scores have the spread of the 128 case
    o = torch.empty_like(q)
    lse = torch.empty(1, H, L, dtype=torch.float32, device=DEV)
    tk.attention_into(q, k, v, o, sm_scale=sc, lse=lse)
    ref, lref = _prescaled_ref(q, k, v, sc)
    assert torch.isfinite(o.float()).all()
    # nearly one-hot rows: the output is a v value of size up to ~4, where one bf16 ulp is 0.03
    torch.testing.assert_close(o.float(), ref, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(lse, lref, atol=2e-2, rtol=1e-4)
    # Against the oracle itself, which scales the fp32 scores (kernels/attention.py:29-30). Rounding
    # q * sm_scale * log2(e) to bf16 moves every term of a score by at most 2^-8 of its size, so in the
    # base-2 domain row i's scores, and with them its lse, move by at most
    #     bound_i = 2^-8 * sm_scale * log2(e) * max_j sum_d |q_id| |k_jd|
    # which is a function of the input magnitudes only. The outputs of these nearly one-hot rows are
    # single v values (|v| up to ~4); their departure is bounded by what was measured when the kernel
    # was written, with a third on top: 0.24-0.33 (hot) and 0.047-0.066 (ramp) at the maximum over the
    # four cases of either kind, 3.4e-3 and 1.8e-3 on average.
    lse_oracle = oracle.attention_lse_ref(q, k, sc)
    mag = torch.einsum("bhqd,bhkd->bhqk", q.float().abs(), k.float().abs()).amax(dim=-1)
    bound = mag * (sc * math.log2(math.e) * 2.0 ** -8)
    assert ((lse - lse_oracle).abs() <= bound + 1e-3).all()
    err = (o.float() - oracle.attention_ref_fp32(q, k, v, sc)).abs()
    assert err.max().item() <= (0.44 if kind == "hot" else 0.088), err.max().item()
    assert err.mean().item() <= (2e-2 if kind == "hot" else 6e-3), err.mean().item()


@pytest.mark.parametrize("B,H,L,D", [(4, 24, 300, 128), (2, 3, 300, 128), (2, 3, 300, 64), (2, 3, 300, 32)])
@pytest.mark.parametrize("sm_scale", [-0.11, 0.0])
def test_attention_any_scale_sign(B, H, L, D, sm_scale):
    """kernels/attention.py:173 takes whatever scale it is given; zero makes every row the mean of v."""
    g = seeded(B + H + L + D)
    q, k, v = (randn(g, B, H, L, D, dtype=torch.bfloat16).to(DEV) for _ in range(3))
    o = tk.scaled_dot_product_attention(q, k, v, sm_scale=sm_scale)
    torch.testing.assert_close(o.float(), oracle.attention_ref_fp32(q, k, v, sm_scale), atol=1e-2, rtol=0)
    if sm_scale == 0.0:
        torch.testing.assert_close(o.float(), v.float().mean(dim=2, keepdim=True).expand_as(o), atol=4e-3, rtol=0)


def test_attention_lse_at_the_flux_shape():
    q, k, v = cfg.config5_attention(DEV)
    o = torch.empty_like(q)
    lse = torch.empty(q.shape[:3], dtype=torch.float32, device=DEV)
    tk.attention_into(q, k, v, o, lse=lse)
    torch.testing.assert_close(lse, oracle.attention_lse_ref(q, k), atol=5e-3, rtol=5e-4)
    # o and lse are consistent: exp2(s_ij * log2e - lse_i) sums to one over j, checked on a few rows
    rows = torch.tensor([0, 255, 256, 3071, 4415, 4607], device=DEV)
    s = torch.einsum("bhqd,bhkd->bhqk", q[:, :, rows].float(), k.float()) * (math.log2(math.e) / math.sqrt(q.shape[-1]))
    total = torch.exp2(s - lse[:, :, rows, None]).sum(-1)
    torch.testing.assert_close(total, torch.ones_like(total), atol=5e-3, rtol=0)
