"""The committed fixture tests/golden/flux_small.npz (inputs and expected outputs of every op of the
path at small shapes; written by tests/golden/make_golden.py from the pinned CPU oracle).

CPU: the oracle still reproduces the fixture. GPU: the HIP kernels reproduce it through the C ABI,
bit-exact for the copy/concat path, within the tolerances of the path elsewhere (row-wise ops
atol 1e-2 rtol 1e-2 in bf16, linear and attention atol 2e-2 against the fp32 expectation).
"""
import pytest
import torch

from oracle import flux_oracle as oracle
from util import load_golden

G = load_golden()


def test_fixture_is_complete():
    want = {"rms_x", "rms_w", "rms_y", "ln_x", "ln_scale", "ln_shift", "ln_y", "rope_q", "rope_k", "rope_pe", "rope_oq",
            "rope_ok", "lin_a", "lin_w", "lin_b", "lin_y", "lin_y_gelu", "att_q", "att_k", "att_v", "att_o", "cat_txt",
            "cat_img", "cat_q", "cat_k", "cat_v"}
    assert want <= set(G)


def test_oracle_reproduces_fixture():
    assert torch.equal(oracle.rms_norm_ref(G["rms_x"], G["rms_w"], 1e-6), G["rms_y"])
    assert torch.equal(oracle.layer_norm_modulation_ref(G["ln_x"], G["ln_scale"], G["ln_shift"], 1e-6), G["ln_y"])
    oq, ok = oracle.apply_rope_ref(G["rope_q"], G["rope_k"], G["rope_pe"])
    assert torch.equal(oq, G["rope_oq"]) and torch.equal(ok, G["rope_ok"])
    torch.testing.assert_close(oracle.linear_ref_fp32(G["lin_a"], G["lin_w"], G["lin_b"], ""), G["lin_y"], atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(oracle.linear_ref_fp32(G["lin_a"], G["lin_w"], G["lin_b"], "GELU"), G["lin_y_gelu"], atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(oracle.attention_ref_fp32(G["att_q"], G["att_k"], G["att_v"]), G["att_o"], atol=1e-5, rtol=1e-5)
    cq, ck, cv = oracle.qkv_concat_ref(G["cat_txt"], G["cat_img"], 2)
    assert torch.equal(cq, G["cat_q"]) and torch.equal(ck, G["cat_k"]) and torch.equal(cv, G["cat_v"])


@pytest.mark.gpu
def test_hip_kernels_reproduce_fixture():
    import triton_kernels as tk

    d = {k: v.cuda() for k, v in G.items()}
    torch.testing.assert_close(tk.rms_norm(d["rms_x"], d["rms_w"]).cpu(), G["rms_y"], atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(tk.layer_norm_modulation(d["ln_x"], d["ln_scale"], d["ln_shift"], 1e-6).cpu(), G["ln_y"],
                               atol=1e-2, rtol=1e-2)
    oq, ok = tk.apply_rope(d["rope_q"], d["rope_k"], d["rope_pe"])
    torch.testing.assert_close(oq.cpu(), G["rope_oq"], atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(ok.cpu(), G["rope_ok"], atol=1e-2, rtol=1e-2)
    y = tk.linear(d["lin_a"], d["lin_w"], d["lin_b"])
    torch.testing.assert_close(y.float().cpu(), G["lin_y"], atol=2e-2, rtol=2 ** -8)
    y = tk.linear(d["lin_a"], d["lin_w"], d["lin_b"], activation="GELU")
    torch.testing.assert_close(y.float().cpu(), G["lin_y_gelu"], atol=2e-2, rtol=2 ** -8)
    o = tk.scaled_dot_product_attention(d["att_q"], d["att_k"], d["att_v"])
    torch.testing.assert_close(o.float().cpu(), G["att_o"], atol=2e-2, rtol=0)
    tq, tk_, tv = d["cat_txt"].view(1, 8, 3, 2, 64).permute(2, 0, 3, 1, 4)    # [B,H,L,D] views, read in place
    iq, ik, iv = d["cat_img"].view(1, 16, 3, 2, 64).permute(2, 0, 3, 1, 4)
    cq, ck, cv = tk.qkv_prep(iq, ik, iv, tq, tk_, tv)
    assert torch.equal(cq.cpu(), G["cat_q"]) and torch.equal(ck.cpu(), G["cat_k"]) and torch.equal(cv.cpu(), G["cat_v"])
