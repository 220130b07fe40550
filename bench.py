#!/usr/bin/env python3
"""Benchmark of the Flux single-stream block on the HIP kernel set (one MI355X).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--settle-ms S] [--no-kernels] [--no-cpu] [--json-out FILE]
    python bench.py --only KERNEL [--launches N]      one row of the kernel table by itself (for rocprofv3)

A step is one forward pass of the single-stream block at 4608 tokens (512 txt + 64x64 img),
hidden 3072, 24 heads, bf16, batch 1, on synthetic seeded inputs that are resident in HBM before
the timed region. Prints ONE JSON line: block latency (the headline `value`), the roofline
fraction of the dominant kernel (linear1, timed live with events inside the timed steps), a table
of per-kernel throughputs against their rooflines (`kernels`), and the PyTorch CPU path timed on
the host cores of the same machine (`cpu_baseline`).

From idle this GPU needs some 40 ms of sustained load before its clocks settle (the first 10 block
passes run 12-17 % slower than the 40th), so the timed region is preceded by a clock-settle phase
of fixed duration (--settle-ms, default 80 ms of block passes, untimed, reported as `settle_ms`)
whatever --warmup says. The per-kernel table gives every kernel 50 ms of its own launches first.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(ROOT, "triton-kernels_amd"), ROOT):
    if _p not in sys.path:
        sys.path.insert(0, _p)

METRIC = "Flux single-block ms @4608 tok bf16; per-kernel GB/s & TFLOP/s vs roofline"
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
BLOCK_GFLOP = 1304.65       # linear1 + attention + linear2 + modulation projection
LINEAR1_FLOP = 2.0 * 4608 * 21504 * 3072

TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "gemm_linear1_linear2_4608_hbm_traffic.md")


def linear1_traffic_bytes():
    """Fabric-side bytes of one linear1 launch (what the L2s fetch from / write to Infinity Cache +
    HBM), read from the committed rocprofv3 summary: FETCH_SIZE and WRITE_SIZE per dispatch, each
    scaled by what the same counter reads for a plain copy of known size. None when the summary
    does not carry the figure."""
    try:
        for line in open(TRAFFIC_SUMMARY):
            if line.startswith("linear1_traffic_bytes_per_launch:"):
                return int(line.split(":")[1].strip())
    except OSError:
        pass
    return None


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--settle-ms", type=float, default=80.0, help="untimed block passes for this long before the warm-up")
    ap.add_argument("--only", default=None, help="run one row of the per-kernel table by itself, then exit")
    ap.add_argument("--launches", type=int, default=20, help="launches timed with --only")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--json-out", default=None, help="also write the result, indented, to this file")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run plain device-to-device copies of 256 MiB (reference for scaling FETCH_SIZE / "
                         "WRITE_SIZE counter readings), then exit")
    return ap.parse_args()


# --------------------------------------------------------------------------------------------------
# per-kernel measurements through the C ABI, with rotating buffer sets so that the 256 MB Infinity
# Cache cannot serve what is reported as HBM traffic
# --------------------------------------------------------------------------------------------------
def _time_launches(torch, launches, reps=7, min_launches=48):
    """launches: list of zero-argument callables (one per buffer set). A timed region is at least
    min_launches launches back to back inside one event pair, cycling through the buffer sets, so
    that the idle gap in front of a region (synchronisation, event creation) does not weigh on a
    region of only a few short launches. Returns the median time per launch in microseconds."""
    t_end = time.perf_counter() + 0.05     # warm-up: the clocks settle under sustained load only
    while True:
        for f in launches:
            f()
        torch.cuda.synchronize()
        if time.perf_counter() >= t_end:
            break
    per = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        cycles = -(-min_launches // len(launches))
        a.record()
        for _ in range(cycles):
            for f in launches:
                f()
        b.record()
        torch.cuda.synchronize()
        per.append(a.elapsed_time(b) * 1e3 / (cycles * len(launches)))
    return statistics.median(per)


def kernel_cases(torch, extra=False):
    """Yields (name, bound, work, note, build) for every row of the per-kernel table; build() allocates
    the rotating buffer sets and returns (launches, keepalive). extra=True adds rows that only
    `--only` runs: the same copy and RMSNorm at sixteen times the size, where launch, ramp-up and
    tail no longer weigh on the rate."""
    import triton_kernels as tk
    from triton_kernels import _native as nv
    from triton_kernels import testing as cfg

    lib = nv.lib()
    dev = torch.device("cuda:0")
    st = nv.stream_ptr(dev)

    def n_sets(bytes_per_set):
        return max(3, int(600e6 // bytes_per_set) + 1)

    def check(rc):
        nv.check(rc, "bench")

    # What a plain device-to-device copy reaches at the sizes of the row-wise kernels below (the
    # practical HBM ceiling of this machine for read-once / write-once traffic, launch included).
    for mb in (27, 81, 432) if extra else (27, 81):
        n = mb * 1024 * 1024 // 2

        def build(n=n):
            sets = [(torch.empty(n, dtype=torch.bfloat16, device=dev).normal_(), torch.empty(n, dtype=torch.bfloat16, device=dev))
                    for _ in range(n_sets(4 * n))]
            return [(lambda a=a, y=y: y.copy_(a)) for a, y in sets], sets
        yield f"copy_{mb}MiB_reference", "hbm", 4 * n, "torch copy_ (device-to-device), same rotation", build

    # C1: QK RMSNorm, x [1,24,4608,128]
    def build_rms():
        x, w = cfg.config1(dev)
        B_, H_, L_, D_ = x.shape
        sets = [(x.clone(), torch.empty_like(x)) for _ in range(n_sets(2 * x.numel() * 2))]
        return [(lambda a=a, y=y: check(lib.flux_rms_norm(a.data_ptr(), w.data_ptr(), y.data_ptr(), None, B_, H_, L_, D_,
                                                           a.stride(0), a.stride(1), a.stride(2), 0, 0, 1e-6, st)))
                for a, y in sets], (sets, w)
    yield "rms_norm_qk", "hbm", 2 * (24 * 4608 * 128) * 2 + 256, "", build_rms

    if extra:
        def build_rms16():
            x, w = cfg.config1(dev)
            x = x.expand(16, -1, -1, -1).contiguous()
            B_, H_, L_, D_ = x.shape
            sets = [(x.clone(), torch.empty_like(x)) for _ in range(3)]
            return [(lambda a=a, y=y: check(lib.flux_rms_norm(a.data_ptr(), w.data_ptr(), y.data_ptr(), None, B_, H_, L_, D_,
                                                               a.stride(0), a.stride(1), a.stride(2), 0, 0, 1e-6, st)))
                    for a, y in sets], (sets, w)
        yield "rms_norm_qk_x16", "hbm", 16 * 2 * (24 * 4608 * 128) * 2 + 256, "x [16,24,4608,128]", build_rms16

    # C2: LayerNorm + modulation, x [1,4608,3072]
    def build_ln():
        x, sc, sh = cfg.config2(dev)
        sets = [(x.clone(), torch.empty_like(x)) for _ in range(n_sets(2 * x.numel() * 2))]
        return [(lambda a=a, y=y: check(lib.flux_layer_norm_modulation(a.data_ptr(), sc.data_ptr(), sh.data_ptr(), y.data_ptr(),
                                                                        1, x.shape[1], x.shape[2], x.shape[2], 0, 1e-6, st)))
                for a, y in sets], (sets, sc, sh)
    yield "layer_norm_modulation", "hbm", 2 * (4608 * 3072) * 2 + 2 * 3072 * 2, "", build_ln

    # C3: RoPE alone, concat alone, RoPE + concat fused (argument structs are prepared once per buffer set)
    Lt, Li = 512, 4096
    Ltot = Lt + Li
    qk_elems = 24 * Ltot * 128
    pe_bytes = Ltot * 64 * 4 * 4

    def prep_args(pe, tq, tk_, tv, iq, ik, iv, oq, ok, ov, with_pe, lt):
        a = nv.QkvPrepArgs()
        for name, t_, i_, o_ in (("q", tq, iq, oq), ("k", tk_, ik, ok), ("v", tv, iv, ov)):
            if o_ is None:
                continue
            setattr(a, f"{name}_img", nv.src4(i_))
            if lt:
                setattr(a, f"{name}_txt", nv.src4(t_))
            setattr(a, f"{name}_out", o_.data_ptr())
        if with_pe:
            a.pe = pe.data_ptr()
        a.B, a.H, a.Lt, a.Li, a.D = 1, 24, lt, Ltot - lt, 128
        a.dtype = a.scale_dtype = 0
        a.eps = 1e-6
        return a

    def build_rope():
        txt, img, pe = cfg.config3(dev)
        full_q = torch.cat((txt[0], img[0]), 2)
        full_k = torch.cat((txt[1], img[1]), 2)
        keep, launches = [pe], []
        for _ in range(n_sets(4 * qk_elems * 2)):
            q_, k_ = full_q.clone(), full_k.clone()
            oq, ok = torch.empty_like(q_), torch.empty_like(k_)
            a = prep_args(pe, None, None, None, q_, k_, None, oq, ok, None, True, 0)
            keep.append((q_, k_, oq, ok, a))
            launches.append(lambda a=a: check(lib.flux_qkv_prep(ctypes.byref(a), st)))
        return launches, keep
    yield "rope_apply", "hbm", 4 * qk_elems * 2 + pe_bytes, "", build_rope

    for name, with_pe, work in (("qkv_concat", False, 6 * qk_elems * 2),
                                ("rope_concat_fused", True, 6 * qk_elems * 2 + pe_bytes)):
        def build(with_pe=with_pe):
            txt, img, pe = cfg.config3(dev)
            keep, launches = [pe], []
            for _ in range(n_sets(6 * qk_elems * 2)):
                t_ = [t.clone() for t in txt]
                i_ = [t.clone() for t in img]
                o_ = [torch.empty(1, 24, Ltot, 128, dtype=torch.bfloat16, device=dev) for _ in range(3)]
                a = prep_args(pe, t_[0], t_[1], t_[2], i_[0], i_[1], i_[2], o_[0], o_[1], o_[2], with_pe, Lt)
                keep.append((t_, i_, o_, a))
                launches.append(lambda a=a: check(lib.flux_qkv_prep(ctypes.byref(a), st)))
            return launches, keep
        yield name, "hbm", work, "", build

    # C4 / C5: GEMMs (MFMA-bound; three rotating sets keep operands out of L2 between launches)
    for name, which, act, (M, N, K) in (("linear_mlp_in_gelu", "mlp_in", "GELU", (4608, 12288, 3072)),
                                        ("linear_proj_out", "proj_out", "", (4608, 3072, 15360)),
                                        ("linear1_block", "linear1", "", (4608, 21504, 3072))):
        def build(which=which, act=act, M=M, N=N):
            a_, w_, b_ = cfg.config4(dev, which)
            sets = [(a_.clone(), w_.clone(), torch.empty(M, N, dtype=torch.bfloat16, device=dev)) for _ in range(3)]
            return [(lambda s=s: tk.linear_into(s[0], s[1], b_, activation=act, out=s[2])) for s in sets], (sets, b_)
        note = ("bias-only epilogue; inside the block the same product carries the q/k norm + RoPE and GELU epilogues, "
                "timed there as roofline.launch_us") if name == "linear1_block" else ""
        yield name, "mfma", 2.0 * M * N * K, note, build

    # C5: attention forward
    def build_attn():
        q, k, v = cfg.config5_attention(dev)
        sets = [(q.clone(), k.clone(), v.clone(), torch.empty_like(q)) for _ in range(3)]
        return [(lambda s=s: tk.attention_into(s[0], s[1], s[2], s[3])) for s in sets], sets
    yield "attention_fwd", "mfma", 4.0 * 24 * 4608 * 4608 * 128, "", build_attn


def _entry(us, bound, work, note=""):
    if bound == "hbm":
        ach, peak, unit = work / us / 1e3, HBM_PEAK_GBS, "GB/s"
    else:
        ach, peak, unit = work / us / 1e6, MFMA_PEAK_TFLOPS, "TFLOP/s"
    return {"us": round(us, 2), "bound": bound, "achieved": round(ach, 1), "unit": unit,
            "frac": round(ach / peak, 4), "work": work, **({"note": note} if note else {})}


def kernel_table(torch):
    out = {}
    for name, bound, work, note, build in kernel_cases(torch):
        launches, keep = build()
        out[name] = _entry(_time_launches(torch, launches), bound, work, note)
        del launches, keep
    return out


def run_only(torch, which, n_launches):
    """One row of the table by itself: 50 ms of its launches to settle the clocks, then n_launches
    launches inside one event pair. This is the command the rocprofv3 summaries under profiles/ wrap."""
    for name, bound, work, note, build in kernel_cases(torch, extra=True):
        if name != which:
            continue
        launches, keep = build()
        t_end = time.perf_counter() + 0.05
        while time.perf_counter() < t_end:
            for f in launches:
                f()
            torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(n_launches):
            launches[i % len(launches)]()
        b.record()
        torch.cuda.synchronize()
        res = _entry(a.elapsed_time(b) * 1e3 / n_launches, bound, work, note)
        print(json.dumps({"only": name, "launches_timed": n_launches, **res}))
        return
    names = [c[0] for c in kernel_cases(torch, extra=True)]
    print(f"bench.py --only: unknown kernel {which!r}; one of {names}", file=sys.stderr)
    sys.exit(2)


# --------------------------------------------------------------------------------------------------
# CPU baseline: the oracle's single-stream block on the host cores (reported, not a target)
# --------------------------------------------------------------------------------------------------
def cpu_baseline(torch):
    from oracle import flux_oracle as oracle
    from triton_kernels import testing as cfg

    x, vec, pe, sd = cfg.config5_block("cpu")
    times = []
    with torch.no_grad():
        for i in range(4):
            t0 = time.perf_counter()
            oracle.single_stream_block_ref(sd, x, vec, pe, 24)
            t1 = time.perf_counter()
            if i > 0:
                times.append((t1 - t0) * 1e3)
    return {
        "value": round(statistics.median(times), 1), "unit": "ms", "cores": torch.get_num_threads(), "kind": "port",
        "sample": "oracle single_stream_block_ref (plain PyTorch, bf16) on the same seeded 4608-token inputs: "
                  "1 warm-up + 3 timed passes, median; host has %d logical CPUs" % (os.cpu_count() or 0),
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; the kernel path has no collective and --gpus must be 1 "
              f"(got {args.gpus})", file=sys.stderr)
        sys.exit(2)

    import torch

    import triton_kernels as tk
    from triton_kernels import testing as cfg

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibrate_copy:
        n = 256 * 1024 * 1024
        srcs = [torch.full((n,), i, dtype=torch.uint8, device=dev) for i in range(4)]
        dst = torch.empty(n, dtype=torch.uint8, device=dev)
        for a in srcs * 2:
            dst.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "8 device-to-device copies", "bytes_read_per_copy": n, "bytes_written_per_copy": n}))
        return

    if args.only:
        run_only(torch, args.only, args.launches)
        return

    x, vec, pe, sd = cfg.config5_block(dev)
    blk = tk.SingleStreamBlock(3072, 24).to(torch.bfloat16).to(dev)
    blk.load_state_dict(sd)

    # Events around the stages of the fused forward inside the timed steps, through the hook the module
    # exposes for this. They are recorded on torch's current stream, which is the stream every HIP
    # kernel here is launched on. linear1 (N = 21504) is the dominant kernel.
    stage_events = {"linear1": [], "attention": [], "linear2": []}
    open_ev = {}

    def hook(stage, edge):
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        if edge == "begin":
            open_ev[stage] = e
        else:
            stage_events[stage].append((open_ev.pop(stage), e))

    with torch.no_grad():
        # clock-settle phase: block passes for a fixed time, whatever --warmup says
        t_s = time.perf_counter()
        settle_passes = 0
        while (time.perf_counter() - t_s) * 1e3 < args.settle_ms:
            for _ in range(8):
                blk(x, vec, pe)
            torch.cuda.synchronize()
            settle_passes += 8
        settle_ms = (time.perf_counter() - t_s) * 1e3
        for _ in range(args.warmup):
            blk(x, vec, pe)
        torch.cuda.synchronize()
        blk.stage_hook = hook
        t0 = time.perf_counter()
        for _ in range(args.steps):
            y = blk(x, vec, pe)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        blk.stage_hook = None
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    stage_us = {k: statistics.mean(e0.elapsed_time(e1) for e0, e1 in v) * 1e3 for k, v in stage_events.items()}
    l1_us = stage_us["linear1"]
    l1_tflops = LINEAR1_FLOP / l1_us / 1e6
    assert torch.isfinite(y.float()).all()

    result = {
        "metric": METRIC,
        "value": round(ms_per_step, 4),
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_ms": round(settle_ms, 1),
        "settle_passes": settle_passes,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "flux single-stream block forward, batch 1, 4608 tokens (512 txt + 64x64 img), "
                               "hidden 3072, 24 heads x 128, mlp 12288, seeded N(0,1) inputs, N(0,1/fan_in) weights"},
        "block_tflops": round(BLOCK_GFLOP / ms_per_step, 1),
        "block_frac_of_mfma_peak": round(BLOCK_GFLOP / ms_per_step / MFMA_PEAK_TFLOPS, 4),
        "roofline": {
            "kernel": "gemm_nt_ring_kernel<4,false> (linear1: 4608 x 21504 x 3072, bias, split qkv / GELU(mlp) epilogue)",
            "bound": "mfma", "achieved": round(l1_tflops, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(l1_tflops / MFMA_PEAK_TFLOPS, 4), "traffic": linear1_traffic_bytes(),
            "launch_us": round(l1_us, 1), "launches_timed": len(stage_events["linear1"]),
        },
        "block_stage_us": {k: round(v, 1) for k, v in stage_us.items()},
    }
    if not args.no_kernels:
        result["kernels"] = kernel_table(torch)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(torch)
    if args.json_out:
        with open(args.json_out, "w") as f:
            json.dump(result, f, indent=1)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
