"""Single- and double-stream Flux block: HIP-kernel block against the plain-PyTorch block.

What the reference's scripts/single_triton.py and scripts/double_triton.py do, at their shapes
(batch 3; single: 4336 tokens; double: 4080 img + 256 txt tokens; hidden 3072, 24 heads): both
blocks share one state dict, the outputs are compared, then each block is timed over 100 passes
after 5 warm-up passes. The reference scripts build fp32 tensors, which its bf16-only linear
(kernels/linear.py:105-114) rejects, and compare at atol 1e-5; here the blocks run in bf16, the
dtype the kernels are written for, and are compared at the tolerance of tests/test_blocks.py:43
(atol 0.1).

    python triton-kernels_amd/benchmarks/blocks.py --block single
    python triton-kernels_amd/benchmarks/blocks.py --block double --batch 1 --img-len 4096 --txt-len 512
"""
import argparse
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import triton_kernels as tk  # noqa: E402
from triton_kernels import flux  # noqa: E402


def build_pair(kind, hidden, heads, mlp_ratio, device, dtype=torch.bfloat16, seed=0):
    torch.manual_seed(seed)
    names = {"single": "SingleStreamBlock", "double": "DoubleStreamBlock"}
    plain = getattr(flux, names[kind])(hidden_size=hidden, num_heads=heads, mlp_ratio=mlp_ratio)
    hip = getattr(tk, names[kind])(hidden_size=hidden, num_heads=heads, mlp_ratio=mlp_ratio)
    hip.load_state_dict(plain.state_dict())
    return plain.to(dtype).to(device), hip.to(dtype).to(device)


def make_inputs(kind, batch, seq_len, img_len, txt_len, hidden, heads, device, dtype=torch.bfloat16):
    head_dim = hidden // heads
    vec = torch.randn(batch, hidden, device=device, dtype=dtype)
    if kind == "single":
        pe = torch.randn(1, 1, seq_len, head_dim // 2, 2, 2, device=device)
        return dict(x=torch.randn(batch, seq_len, hidden, device=device, dtype=dtype), vec=vec, pe=pe)
    pe = torch.randn(1, 1, img_len + txt_len, head_dim // 2, 2, 2, device=device)
    return dict(img=torch.randn(batch, img_len, hidden, device=device, dtype=dtype),
                txt=torch.randn(batch, txt_len, hidden, device=device, dtype=dtype), vec=vec, pe=pe)


def time_block(block, inputs, warmup, runs):
    with torch.no_grad():
        for _ in range(warmup):
            block(**inputs)
        beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        beg.record()
        for _ in range(runs):
            block(**inputs)
        end.record()
        end.synchronize()
    return beg.elapsed_time(end) / runs


def compare(plain, hip, inputs, atol):
    with torch.no_grad():
        want, got = plain(**inputs), hip(**inputs)
    want = want if isinstance(want, tuple) else (want,)
    got = got if isinstance(got, tuple) else (got,)
    worst = 0.0
    for w, g in zip(want, got):
        torch.testing.assert_close(g, w, atol=atol, rtol=0)
        worst = max(worst, (g.float() - w.float()).abs().max().item())
    return worst


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--block", default="single", choices=["single", "double"])
    ap.add_argument("--batch", type=int, default=3)
    ap.add_argument("--seq-len", type=int, default=4336, help="single block: tokens")
    ap.add_argument("--img-len", type=int, default=4080, help="double block: image tokens")
    ap.add_argument("--txt-len", type=int, default=256, help="double block: text tokens")
    ap.add_argument("--hidden", type=int, default=3072)
    ap.add_argument("--heads", type=int, default=24)
    ap.add_argument("--mlp-ratio", type=float, default=4.0)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--runs", type=int, default=100)
    ap.add_argument("--atol", type=float, default=0.1)
    ap.add_argument("--no-baseline", action="store_true", help="skip timing the plain PyTorch block (for kernel traces of the HIP one)")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("blocks.py needs a GPU: the HIP kernels have no CPU path")
    dev = torch.device("cuda", 0)
    plain, hip = build_pair(args.block, args.hidden, args.heads, args.mlp_ratio, dev)
    inputs = make_inputs(args.block, args.batch, args.seq_len, args.img_len, args.txt_len,
                         args.hidden, args.heads, dev)
    worst = compare(plain, hip, inputs, args.atol)
    print(f"max |hip - baseline| = {worst:.4f} (atol {args.atol})")
    if not args.no_baseline:
        print(f"baseline block time: {time_block(plain, inputs, args.warmup, args.runs):.3f} ms per pass")
    print(f"     hip block time: {time_block(hip, inputs, args.warmup, args.runs):.3f} ms per pass")


if __name__ == "__main__":
    main()
