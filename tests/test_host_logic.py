"""Host-side behaviour of the Python operator layer that can be checked without a GPU: the public
names, the exceptions the reference raises, the no-CPU-fallback rule, state-dict compatibility and
the launch spelling of the raw ops."""
import os

import pytest
import torch

import triton_kernels as tk
from triton_kernels import flux, modules, ops
from triton_kernels.kernels.utils import calculate_settings
from triton_kernels.ops._launch import HipOp


def test_public_names():
    for name in ("apply_rope", "layer_norm_modulation", "linear", "rms_norm", "scaled_dot_product_attention",
                 "apply_rope_torch", "apply_rope_torch_compile", "layer_norm_modulation_torch",
                 "layer_norm_modulation_torch_compile", "rms_norm_torch", "rms_norm_torch_compile",
                 "DoubleStreamBlock", "QKNorm", "RMSNorm", "SingleStreamBlock"):
        assert hasattr(tk, name), name
    for name in ("triton_linear", "triton_modulation_scale_shift", "triton_modulation_gate_proj", "triton_qkv_concat", "triton_silu"):
        assert isinstance(getattr(ops, name), HipOp)
    assert {"SingleStreamBlock", "DoubleStreamBlock"} <= set(dir(flux))


def test_calculate_settings():
    assert calculate_settings(128) == (128, 4)
    assert calculate_settings(3072) == (4096, 8)
    assert calculate_settings(8192)[1] == 16 and calculate_settings(65536) == (65536, 32)
    with pytest.raises(RuntimeError):
        calculate_settings(65537)


def test_no_cpu_fallback():
    x = torch.randn(2, 8, 16)
    with pytest.raises(RuntimeError, match="GPU"):
        tk.rms_norm(x, torch.ones(16))
    with pytest.raises(RuntimeError, match="GPU"):
        tk.layer_norm_modulation(x, torch.zeros(2, 1, 16), torch.zeros(2, 1, 16))
    with pytest.raises(RuntimeError, match="GPU"):
        tk.apply_rope(x[None], x[None], torch.zeros(1, 1, 8, 8, 2, 2))
    with pytest.raises(RuntimeError, match="GPU"):
        tk.linear(x.bfloat16(), torch.zeros(4, 16, dtype=torch.bfloat16), None)
    q = torch.zeros(1, 1, 8, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        tk.scaled_dot_product_attention(q, q, q)


def test_reference_error_behaviour():
    x = torch.randn(2, 8, 16)
    with pytest.raises(AssertionError):
        tk.rms_norm(x, torch.ones(8))                                  # last dims differ
    with pytest.raises(AssertionError):
        tk.layer_norm_modulation(x, torch.zeros(3, 1, 16), torch.zeros(2, 1, 16))
    with pytest.raises(AssertionError):
        tk.linear(x.bfloat16(), torch.zeros(4, 8, dtype=torch.bfloat16), None)    # incompatible dimensions
    with pytest.raises(AssertionError):
        tk.linear(x.bfloat16(), torch.zeros(4, 16), None)                          # incompatible dtypes
    with pytest.raises(KeyError):
        tk.linear(x, torch.zeros(4, 16), None)                                     # fp32: no tile plan, as in the reference
    with pytest.raises(KeyError):
        tk.linear(x.bfloat16(), torch.zeros(4, 16, dtype=torch.bfloat16), None, activation="RELU")
    q = torch.zeros(1, 1, 8, 48, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        tk.scaled_dot_product_attention(q, q, q)                                   # head dim not in {16..256}
    with pytest.raises(RuntimeError):
        tk.rms_norm(torch.zeros(1, 70000), torch.ones(70000))                      # wider than 65536


def test_functional_names_are_plain_torch():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 3, 16, generator=g)
    w = torch.rand(16, generator=g)
    assert torch.equal(tk.rms_norm_torch(x, w), tk.rms_norm_torch_compile(x, w))
    sc, sh = torch.randn(2, 1, 16, generator=g), torch.randn(2, 1, 16, generator=g)
    torch.testing.assert_close(tk.layer_norm_modulation_torch(x, sc, sh),
                               torch.nn.functional.layer_norm(x, (16,)) * (1 + sc) + sh)
    pe = torch.randn(1, 1, 3, 8, 2, 2, generator=g)
    q, k = tk.apply_rope_torch(x[None], x[None], pe)
    assert torch.equal(q, k) and q.shape == (1, 2, 3, 16)


def test_state_dicts_are_interchangeable():
    single_keys = {"linear1.weight", "linear1.bias", "linear2.weight", "linear2.bias", "norm.query_norm.scale",
                   "norm.key_norm.scale", "modulation.lin.weight", "modulation.lin.bias"}
    ref, hip = flux.SingleStreamBlock(64, 4), tk.SingleStreamBlock(64, 4)
    assert set(ref.state_dict()) == set(hip.state_dict()) == single_keys
    hip.load_state_dict(ref.state_dict())
    ref_d, hip_d = flux.DoubleStreamBlock(64, 4, 4.0), tk.DoubleStreamBlock(64, 4, 4.0)
    assert set(ref_d.state_dict()) == set(hip_d.state_dict())
    for s in ("img", "txt"):
        for key in (f"{s}_mod.lin.weight", f"{s}_attn.qkv.weight", f"{s}_attn.norm.query_norm.scale", f"{s}_attn.proj.bias",
                    f"{s}_mlp.0.weight", f"{s}_mlp.2.bias"):
            assert key in hip_d.state_dict()
        assert f"{s}_attn.qkv.bias" not in hip_d.state_dict()          # qkv_bias defaults to False
    hip_d.load_state_dict(ref_d.state_dict())
    assert {k: v.shape for k, v in ref_d.state_dict().items()} == {k: v.shape for k, v in hip_d.state_dict().items()}
    assert isinstance(modules.MLP(8, 32)[1], torch.nn.Identity)


def test_linear_launch_metadata_matches_the_reference_hook():
    """kernels/linear.py:9-19 of the reference: name with the problem size, flops16 = 2 M N K, bytes = A + W + C."""
    import sys
    import triton_kernels.kernels.linear  # noqa: F401  (the package re-exports the function under the same name)
    lin = sys.modules["triton_kernels.kernels.linear"]
    md = lin.linear_launch_metadata(4608, 21504, 3072)
    assert md["name"].endswith("[M=4608, N=21504, K=3072]")
    assert md["flops16"] == 2.0 * 4608 * 21504 * 3072
    assert md["bytes"] == 2 * (4608 * 3072 + 21504 * 3072 + 4608 * 21504)
    assert lin.launch_hook is None


def test_hip_op_launch_spelling():
    calls = []
    op = HipOp(lambda a, b, scale=1: calls.append((a, b, scale)) or "ok", "demo")
    assert op[(4,)](1, 2, XBLOCK=128, num_warps=4) == "ok"
    assert op(3, 4, scale=2, BLOCK_M=64) == "ok"
    assert calls == [(1, 2, 1), (3, 4, 2)]


def test_seeded_inputs_are_reproducible():
    from triton_kernels import testing as cfg

    a1, w1, b1 = cfg.config4("cpu", "mlp_in", m=8)
    a2, w2, b2 = cfg.config4("cpu", "mlp_in", m=8)
    assert torch.equal(a1, a2) and torch.equal(w1, w2) and torch.equal(b1, b2)
    assert a1.dtype == torch.bfloat16 and w1.shape == (12288, 3072)
    pe = cfg.flux_pe(4, 2)
    assert pe.shape == (1, 1, 8, 64, 2, 2) and pe.dtype == torch.float32
    from oracle import flux_oracle as oracle
    assert torch.equal(pe, oracle.embed_nd_ref(oracle.flux_ids(4, 2, 2)))    # package builder == oracle builder


def test_bench_reads_traffic_from_the_committed_summary_and_refuses_more_gpus():
    """bench.py takes roofline.traffic from the counter summary under profiles/ (not from a literal), and
    a run on more than one GPU exits with a message."""
    import importlib.util
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(root, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    traffic = bench.linear1_traffic_bytes()
    text = open(os.path.join(root, "profiles", "gemm_linear1_linear2_4608_hbm_traffic.md")).read()
    line = next(l for l in text.splitlines() if l.startswith("linear1_traffic_bytes_per_launch:"))
    assert traffic == int(line.split(":")[1].split()[0])
    algorithmic = 2 * (4608 * 3072 + 21504 * 3072 + 4608 * 21504)          # A, W and Y once, bf16
    assert algorithmic < traffic < 8 * algorithmic
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)
