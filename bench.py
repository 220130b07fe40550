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
SWEEP_MULTS = (1, 2, 4, 8, 16)
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
    ap.add_argument("--sweep", action="store_true",
                    help="row-wise kernels and a hand-written copy at 1, 2, 4, 8 and 16 times the Flux shape, with the "
                         "least-squares fit t = t0 + bytes / rate per kernel; then exit")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-graph", action="store_true", help="skip the captured-graph replay of the same block")
    ap.add_argument("--no-double", action="store_true", help="skip the extra timing of the double-stream block")
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

    # The same kernels on 2, 4, 8 and 16 times the rows (batch 2 .. 16), for the fit t = t0 + bytes / rate
    # that separates launch, ramp-up and tail from the steady rate (--sweep, --only).
    if extra:
        for mult in SWEEP_MULTS[1:]:
            def build_rms_n(mult=mult):
                x, w = cfg.config1(dev)
                x = x.expand(mult, -1, -1, -1).contiguous()
                B_, H_, L_, D_ = x.shape
                sets = [(x.clone(), torch.empty_like(x)) for _ in range(n_sets(2 * x.numel() * 2))]
                return [(lambda a=a, y=y: check(lib.flux_rms_norm(a.data_ptr(), w.data_ptr(), y.data_ptr(), None, B_, H_, L_, D_,
                                                                   a.stride(0), a.stride(1), a.stride(2), 0, 0, 1e-6, st)))
                        for a, y in sets], (sets, w)
            yield f"rms_norm_qk_x{mult}", "hbm", mult * 2 * (24 * 4608 * 128) * 2 + 256, f"x [{mult},24,4608,128]", build_rms_n

    # C2: LayerNorm + modulation, x [1,4608,3072]
    def build_ln():
        x, sc, sh = cfg.config2(dev)
        sets = [(x.clone(), torch.empty_like(x)) for _ in range(n_sets(2 * x.numel() * 2))]
        return [(lambda a=a, y=y: check(lib.flux_layer_norm_modulation(a.data_ptr(), sc.data_ptr(), sh.data_ptr(), y.data_ptr(),
                                                                        1, x.shape[1], x.shape[2], x.shape[2], 0, 1e-6, st)))
                for a, y in sets], (sets, sc, sh)
    yield "layer_norm_modulation", "hbm", 2 * (4608 * 3072) * 2 + 2 * 3072 * 2, "", build_ln

    if extra:
        for mult in SWEEP_MULTS[1:]:
            def build_ln_n(mult=mult):
                x, sc, sh = cfg.config2(dev)
                x = x.expand(mult, -1, -1).contiguous()
                sc, sh = sc.expand(mult, -1, -1).contiguous(), sh.expand(mult, -1, -1).contiguous()
                sets = [(x.clone(), torch.empty_like(x)) for _ in range(n_sets(2 * x.numel() * 2))]
                return [(lambda a=a, y=y: check(lib.flux_layer_norm_modulation(a.data_ptr(), sc.data_ptr(), sh.data_ptr(), y.data_ptr(),
                                                                                mult, x.shape[1], x.shape[2], x.shape[2], 0, 1e-6, st)))
                        for a, y in sets], (sets, sc, sh)
            yield (f"layer_norm_modulation_x{mult}", "hbm", mult * (2 * (4608 * 3072) * 2 + 2 * 3072 * 2), f"x [{mult},4608,3072]",
                   build_ln_n)

    # C3: RoPE alone, concat alone, RoPE + concat fused (argument structs are prepared once per buffer set)
    Lt, Li = 512, 4096
    Ltot = Lt + Li
    qk_elems = 24 * Ltot * 128
    pe_bytes = Ltot * 64 * 4 * 4

    def prep_args(pe, tq, tk_, tv, iq, ik, iv, oq, ok, ov, with_pe, lt, batch=1):
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
        a.B, a.H, a.Lt, a.Li, a.D = batch, 24, lt, Ltot - lt, 128
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

    if extra:
        # the fused RoPE + concat at 2 .. 16 times the rows, and the same gather kernel as a plain copy of
        # q alone (no table, no norm): a hand-written copy of the same structure as the row-wise kernels
        for mult in SWEEP_MULTS[1:]:
            def build_fused_n(mult=mult):
                txt, img, pe = cfg.config3(dev)
                keep, launches = [pe], []
                for _ in range(n_sets(mult * 6 * qk_elems * 2)):
                    t_ = [t.expand(mult, -1, -1, -1).contiguous() for t in txt]
                    i_ = [t.expand(mult, -1, -1, -1).contiguous() for t in img]
                    o_ = [torch.empty(mult, 24, Ltot, 128, dtype=torch.bfloat16, device=dev) for _ in range(3)]
                    a = prep_args(pe, t_[0], t_[1], t_[2], i_[0], i_[1], i_[2], o_[0], o_[1], o_[2], True, Lt, batch=mult)
                    keep.append((t_, i_, o_, a))
                    launches.append(lambda a=a: check(lib.flux_qkv_prep(ctypes.byref(a), st)))
                return launches, keep
            yield f"rope_concat_fused_x{mult}", "hbm", mult * 6 * qk_elems * 2 + pe_bytes, f"batch {mult}", build_fused_n
        for mult in SWEEP_MULTS:
            def build_copy_n(mult=mult):
                x, _ = cfg.config1(dev)
                keep, launches = [], []
                for _ in range(n_sets(mult * 2 * qk_elems * 2)):
                    q_ = x.expand(mult, -1, -1, -1).clone(memory_format=torch.contiguous_format)   # a buffer of its own per set
                    oq = torch.empty_like(q_)
                    a = prep_args(None, None, None, None, q_, None, None, oq, None, None, False, 0, batch=mult)
                    keep.append((q_, oq, a))
                    launches.append(lambda a=a: check(lib.flux_qkv_prep(ctypes.byref(a), st)))
                return launches, keep
            yield (f"hand_copy_x{mult}", "hbm", mult * 2 * qk_elems * 2,
                   f"flux_qkv_prep as a plain copy of q [{mult},24,4608,128] (no table, no norm)", build_copy_n)

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

    # the same launch on the views the fused block passes: v read in place inside the qkv projection
    # (row stride 9216 elements), o written in "L (H D)" order into the [L, 15360] buffer linear2 reads
    def build_attn_views():
        q, k, v = cfg.config5_attention(dev)
        sets = []
        for _ in range(3):
            qkv = torch.empty(1, 4608, 3 * 3072, dtype=torch.bfloat16, device=dev)
            v_view = qkv.view(1, 4608, 3, 24, 128).permute(2, 0, 3, 1, 4)[2]
            v_view.copy_(v)
            both = torch.empty(1, 4608, 3072 + 12288, dtype=torch.bfloat16, device=dev)
            o_view = both[..., :3072].view(1, 4608, 24, 128).permute(0, 2, 1, 3)
            sets.append((q.clone(), k.clone(), v_view, o_view, qkv, both))
        return [(lambda s=s: tk.attention_into(s[0], s[1], s[2], s[3])) for s in sets], sets
    yield ("attention_fwd_block_views", "mfma", 4.0 * 24 * 4608 * 4608 * 128,
           "v at row stride 9216 inside qkv, o at row stride 15360 into the concat buffer, as in the fused block", build_attn_views)

    # head dim 64 at the same hidden size (the reference's test grid is D in {64, 128}, tests/test_attention.py:7-21)
    def build_attn64():
        g = torch.Generator().manual_seed(1064)
        mk = lambda: torch.randn((1, 48, 4608, 64), generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
        sets = [(mk(), mk(), mk(), torch.empty(1, 48, 4608, 64, dtype=torch.bfloat16, device=dev)) for _ in range(3)]
        return [(lambda s=s: tk.attention_into(s[0], s[1], s[2], s[3])) for s in sets], sets
    yield "attention_fwd_d64", "mfma", 4.0 * 48 * 4608 * 4608 * 64, "B1 H48 L4608 D64", build_attn64

    # linear2 as the block runs it: bias and the gated residual x + gate * y in the epilogue, the
    # residual rows cold (twelve rotating copies, more than the Infinity Cache holds)
    def build_lin2_gated():
        a_, w_, b_ = cfg.config4(dev, "proj_out")
        g = torch.Generator().manual_seed(1077)
        gate = (torch.randn((1, 1, 3072), generator=g) * 0.5).to(torch.bfloat16).to(dev)
        xs = [torch.randn((4608, 3072), generator=g).to(torch.bfloat16).to(dev) for _ in range(12)]
        outs = [torch.empty(4608, 3072, dtype=torch.bfloat16, device=dev) for _ in range(3)]
        return [(lambda i=i: tk.linear_into(a_, w_, b_, out=outs[i % 3], resid=xs[i], gate=gate)) for i in range(12)], (a_, w_, b_, xs, outs, gate)
    yield ("linear2_gated_residual", "mfma", 2.0 * 4608 * 3072 * 15360,
           "proj_out with the block's epilogue: bias, then x + gate * y", build_lin2_gated)


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


def run_sweep(torch):
    """Times the row-wise kernels and the hand-written copy at every size of SWEEP_MULTS and fits
    t = t0 + bytes / rate: t0 is what a launch costs whatever its size (launch, ramp-up, tail), rate the
    steady HBM rate of the kernel. Prints one JSON object."""
    fams = {"rms_norm_qk": [], "layer_norm_modulation": [], "rope_concat_fused": [], "hand_copy": []}
    for name, bound, work, note, build in kernel_cases(torch, extra=True):
        fam = next((f for f in fams if name == f or name.startswith(f + "_x")), None)
        if fam is None:
            continue
        launches, keep = build()
        us = _time_launches(torch, launches, reps=5, min_launches=24)
        fams[fam].append((work, us))
        del launches, keep
        torch.cuda.empty_cache()
    out = {}
    for fam, pts in fams.items():
        pts.sort()
        n = len(pts)
        sx, sy = sum(b for b, _ in pts), sum(t for _, t in pts)
        sxx, sxy = sum(b * b for b, _ in pts), sum(b * t for b, t in pts)
        slope = (n * sxy - sx * sy) / (n * sxx - sx * sx)      # us per byte
        t0 = (sy - slope * sx) / n
        rate = 1.0 / slope / 1e3                                 # GB/s
        out[fam] = {"points": [{"bytes": b, "us": round(t, 2), "GBps": round(b / t / 1e3, 1)} for b, t in pts],
                    "t0_us": round(t0, 2), "steady_GBps": round(rate, 1), "steady_frac_of_peak": round(rate / HBM_PEAK_GBS, 4)}
    print(json.dumps({"sweep": out}))


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


def double_block(torch, steps):
    """The fused double-stream block (4096 img + 512 txt tokens, same hidden size, the txt chain on the
    block's side stream), timed like the headline: an extra key, not the metric."""
    import triton_kernels as tk
    from triton_kernels.testing import flux_pe
    dev = "cuda"
    g = torch.Generator().manual_seed(5)
    blk = tk.DoubleStreamBlock(3072, 24, mlp_ratio=4.0, qkv_bias=True).to(torch.bfloat16)
    for prm in blk.parameters():
        prm.data = (torch.randn(prm.shape, generator=g) * (prm.shape[-1] ** -0.5 if prm.dim() > 1 else 0.1)).to(torch.bfloat16)
    blk = blk.to(dev)
    img = torch.randn(1, 4096, 3072, generator=g).bfloat16().to(dev)
    txt = torch.randn(1, 512, 3072, generator=g).bfloat16().to(dev)
    vec = torch.randn(1, 3072, generator=g).bfloat16().to(dev)
    pe = flux_pe().to(dev)
    with torch.no_grad():
        for _ in range(40):
            out = blk(img=img, txt=txt, vec=vec, pe=pe)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = blk(img=img, txt=txt, vec=vec, pe=pe)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    assert torch.isfinite(out[0].float()).all() and torch.isfinite(out[1].float()).all()
    ms = (t1 - t0) * 1e3 / steps
    return {"ms_per_step": round(ms, 4), "steps": steps, "block_frac_of_mfma_peak": round(BLOCK_GFLOP / ms / MFMA_PEAK_TFLOPS, 4),
            "workload": "flux double-stream block forward, batch 1, 4096 img + 512 txt tokens, hidden 3072, 24 heads x 128"}


def graph_replay(torch, blk, x, vec, pe, y_eager, steps):
    """The same block pass captured once into a HIP graph and replayed `steps` times: what the launch
    gaps of the eager pass cost. Not the headline (that stays the eager number). The library allocates
    nothing and records no memset, so capture is legal; every replay is compared with the eager result."""
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(3):
                blk(x, vec, pe)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(g):
            y_g = blk(x, vec, pe)
        worst = 0.0
        for _ in range(3):   # replays with eager work and synchronisations in between, each one checked
            g.replay()
            torch.cuda.synchronize()
            worst = max(worst, (y_g.float() - y_eager.float()).abs().max().item())
            with torch.no_grad():
                blk(x, vec, pe)
            torch.cuda.synchronize()
        for _ in range(10):
            g.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            g.replay()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        return {"ms_per_step": round(ms, 4), "steps": steps, "max_abs_diff_vs_eager": worst}
    except Exception as e:  # capture is an extra: report why it did not run, keep the headline
        return {"error": f"{type(e).__name__}: {e}"[:300]}


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
    if args.sweep:
        run_sweep(torch)
        return

    x, vec, pe, sd = cfg.config5_block(dev)
    blk = tk.SingleStreamBlock(3072, 24).to(torch.bfloat16).to(dev)
    blk.load_state_dict(sd)

    # Events around the stages of the fused forward inside the timed steps, through the hook the module
    # exposes for this. They are recorded on torch's current stream, which is the stream every HIP
    # kernel here is launched on. linear1 (N = 21504) is the dominant kernel.
    stage_events = {"modulation": [], "layer_norm": [], "linear1": [], "attention": [], "linear2": []}
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
        # the timed region: exactly `steps` passes of the block and nothing else
        t0 = time.perf_counter()
        for _ in range(args.steps):
            y = blk(x, vec, pe)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        # the same passes again with an event pair around every stage, on the stream the kernels run on:
        # stage times and the roofline of the dominant kernel. Ten event records per pass are not free on
        # every box (nothing on some, 0.1 ms per pass on others), so they stay out of the headline.
        blk.stage_hook = hook
        t2 = time.perf_counter()
        for _ in range(args.steps):
            blk(x, vec, pe)
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        blk.stage_hook = None
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    ms_per_step_staged = (t3 - t2) * 1e3 / args.steps
    stage_us = {k: statistics.mean(e0.elapsed_time(e1) for e0, e1 in v) * 1e3 for k, v in stage_events.items()}
    # what the five stages leave of a pass: launch gaps between dependent kernels, allocator calls
    # (and, in the instrumented passes, the event records)
    gap_us = ms_per_step * 1e3 - sum(stage_us.values())
    graph = None if args.no_graph else graph_replay(torch, blk, x, vec, pe, y, args.steps)
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
        "ms_per_step_with_stage_events": round(ms_per_step_staged, 4),
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
        "launch_gap_us": round(gap_us, 1),
        "launch_gap_share": round(gap_us / (ms_per_step * 1e3), 4),
    }
    if graph is not None:
        result["graph_replay"] = graph
    if not args.no_double:
        result["double_block"] = double_block(torch, args.steps)
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
