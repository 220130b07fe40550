"""Sequence-length sweeps of the five operators, HIP kernels next to the PyTorch ops on the same GPU.

Covers what the reference's benchmarks/*.py measure (rms_norm.py, layer_norm.py, rope.py, linear.py,
attention.py): batch 4, 24 heads x 128 (hidden 3072), seq_len 256..4096 in steps of 256 (linear:
64..2048 in steps of 64), forward, and backward for rms_norm. The reference reports
"GB/s" = 2 * numel(x) * element_size / time for every operator (benchmarks/rms_norm.py:49,
benchmarks/linear.py:38, benchmarks/attention.py:37); that column is kept under the same name, and
the GEMM and attention rows also carry TFLOP/s, the figure their roofline is stated in.

    python triton-kernels_amd/benchmarks/sweep.py --op all --out results
    python triton-kernels_amd/benchmarks/sweep.py --op attention --seq-lens 1024 4096

One CSV per operator and mode is written to <out>/<fwd|bwd>/<name>.csv, columns
seq_len, then per provider <provider>_ms, <provider>_gbps[, <provider>_tflops].
"""
import argparse
import csv
import os
import statistics
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import triton_kernels as tk  # noqa: E402

HEADS, HEAD_DIM, HIDDEN = 24, 128, 3072


class Timer:
    """Median time of one call with the caches cold: a buffer larger than the 256 MB Infinity Cache is
    overwritten before every timed call."""

    def __init__(self, device, reps, warmup, flush_mb=512):
        self.reps, self.warmup = reps, warmup
        self.flush = torch.empty(flush_mb << 20, dtype=torch.uint8, device=device) if flush_mb else None

    def __call__(self, fn):
        for _ in range(self.warmup):
            fn()
        torch.cuda.synchronize()
        times = []
        for _ in range(self.reps):
            if self.flush is not None:
                self.flush.zero_()
            beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            beg.record()
            fn()
            end.record()
            end.synchronize()
            times.append(beg.elapsed_time(end))
        return statistics.median(times)


def _rms_norm(batch, seq_len, dev, mode, dtype):
    x = torch.randn(batch, HEADS, seq_len, HEAD_DIM, device=dev, dtype=dtype)
    scale = torch.randn(HEAD_DIM, device=dev, dtype=dtype)
    fwd = {"hip": lambda: tk.rms_norm(x, scale), "torch": lambda: tk.rms_norm_torch(x, scale)}
    if mode == "bwd":
        x.requires_grad_(True)
        scale.requires_grad_(True)
        dy = torch.randn_like(x)
        outs = {name: f() for name, f in fwd.items()}
        fns = {name: (lambda y=y: y.backward(dy, retain_graph=True)) for name, y in outs.items()}
    else:
        fns = fwd
    return fns, 2 * x.numel() * x.element_size(), None


def _layer_norm(batch, seq_len, dev, mode, dtype):
    x = torch.randn(batch, seq_len, HIDDEN, device=dev, dtype=dtype)
    scale = torch.randn(batch, 1, HIDDEN, device=dev, dtype=dtype)
    shift = torch.randn(batch, 1, HIDDEN, device=dev, dtype=dtype)
    fns = {"hip": lambda: tk.layer_norm_modulation(x, scale, shift),
           "torch": lambda: tk.layer_norm_modulation_torch(x, scale, shift)}
    return fns, 2 * x.numel() * x.element_size(), None


def _rope(batch, seq_len, dev, mode, dtype):
    q = torch.randn(batch, HEADS, seq_len, HEAD_DIM, device=dev, dtype=dtype)
    k = torch.randn_like(q)
    pe = torch.randn(1, 1, seq_len, HEAD_DIM // 2, 2, 2, device=dev)
    fns = {"hip": lambda: tk.apply_rope(q, k, pe), "torch": lambda: tk.apply_rope_torch(q, k, pe)}
    return fns, 2 * q.numel() * q.element_size(), None


def _linear(batch, seq_len, dev, mode, dtype):
    x = torch.randn(batch, seq_len, HIDDEN, device=dev, dtype=torch.bfloat16)
    w = torch.randn(HIDDEN, HIDDEN, device=dev, dtype=torch.bfloat16)
    b = torch.randn(HIDDEN, device=dev, dtype=torch.bfloat16)
    fns = {"hip": lambda: tk.linear(x, w, b), "torch": lambda: torch.nn.functional.linear(x, w, b)}
    return fns, 2 * x.numel() * x.element_size(), 2.0 * batch * seq_len * HIDDEN * HIDDEN


def _attention(batch, seq_len, dev, mode, dtype):
    q = torch.randn(batch, HEADS, seq_len, HEAD_DIM, device=dev, dtype=torch.bfloat16)
    k, v = torch.randn_like(q), torch.randn_like(q)
    fns = {"hip": lambda: tk.scaled_dot_product_attention(q, k, v),
           "torch": lambda: torch.nn.functional.scaled_dot_product_attention(q, k, v)}
    return fns, 2 * q.numel() * q.element_size(), 4.0 * batch * HEADS * seq_len * seq_len * HEAD_DIM


_STEP256 = [256 * i for i in range(1, 17)]
OPS = {
    # name: (builder, default seq_lens, modes, csv name as in the reference's plot_name)
    "rms_norm": (_rms_norm, _STEP256, ("fwd", "bwd"), "rms-norm"),
    "layer_norm": (_layer_norm, _STEP256, ("fwd",), "layer-norm-modulation"),
    "rope": (_rope, _STEP256, ("fwd",), "apply-rope"),
    "linear": (_linear, [64 * i for i in range(1, 33)], ("fwd",), "linear"),
    "attention": (_attention, _STEP256, ("fwd",), "attention"),
}


def run_op(name, mode, seq_lens, batch, timer, device, out_dir=None, echo=print, dtype=torch.bfloat16):
    builder, default_lens, modes, csv_name = OPS[name]
    if mode not in modes:
        raise ValueError(f"{name} has no {mode} benchmark")
    rows = []
    for seq_len in seq_lens or default_lens:
        fns, nbytes, flops = builder(batch, seq_len, device, mode, dtype)
        row = {"seq_len": seq_len}
        for provider, fn in fns.items():
            ms = timer(fn)
            row[f"{provider}_ms"] = round(ms, 5)
            row[f"{provider}_gbps"] = round(nbytes / ms * 1e-6, 1)
            if flops is not None:
                row[f"{provider}_tflops"] = round(flops / ms * 1e-9, 1)
        rows.append(row)
        del fns
    cols = list(rows[0])
    echo(f"{csv_name} ({mode}), batch {batch}" + (f", {dtype}" if flops is None else ", torch.bfloat16") + ":")
    echo("  " + "  ".join(f"{c:>13}" for c in cols))
    for row in rows:
        echo("  " + "  ".join(f"{row[c]:>13}" for c in cols))
    if out_dir:
        os.makedirs(os.path.join(out_dir, mode), exist_ok=True)
        with open(os.path.join(out_dir, mode, csv_name + ".csv"), "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=cols)
            w.writeheader()
            w.writerows(rows)
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--op", default="all", choices=["all", *OPS])
    ap.add_argument("--mode", default="all", choices=["all", "fwd", "bwd"])
    ap.add_argument("--seq-lens", type=int, nargs="*", default=None)
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"],
                    help="element type of the three row-wise operators (the reference's scripts feed them "
                         "fp32, the Flux block bf16); linear and attention are bf16 only")
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--out", default=None, help="directory for the CSV files")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("sweep.py needs a GPU: the HIP kernels have no CPU path")
    dev = torch.device("cuda", 0)
    timer = Timer(dev, args.reps, args.warmup)
    for name in (OPS if args.op == "all" else [args.op]):
        for mode in OPS[name][2]:
            if args.mode in ("all", mode):
                run_op(name, mode, args.seq_lens, args.batch, timer, dev, args.out,
                       dtype=torch.float32 if args.dtype == "fp32" else torch.bfloat16)


if __name__ == "__main__":
    main()
