#!/usr/bin/env python3
"""Benchmark of the banded-matmul hot path on one MI355X.

A step is one pass of the chain the reference's callers run (reference
tests/test_attention.py:48-72) at the Longformer shape the headline metric is quoted on:

    A = window_matmul(q, k^T, w) -> P = softmax(A, -1) -> O = unwindow_matmul(P, v, w)
    backward with dO ~ N(0,1)  (grad_a, grad_v, softmax backward, grad_q, grad_k)

bf16 storage, float32 accumulation, B=96 M=4096 N=64 w=256, seeded synthetic inputs that
are resident in HBM before the timed region starts.  The value reported is whole-step
throughput on the band FLOPs (6 band units per step; the torch softmax adds no FLOPs to
the count but its time is inside the step).  Next to it:

  roofline       the slowest of the six kernels, timed alone with HIP events on the stream
                 it is launched on (median of the launches), priced against the 8 TB/s HBM
                 peak on its algorithmic bytes (each operand touched once);
  cpu_baseline   the C restatement of the reference's scalar CPU path (and, where it is
                 built, the reference's own compiled CPU path beside it), one thread, on a
                 slice of the batch;
  other_configs  per-kernel timings, band softmax and fused attention at the other shapes
                 the targets are stated on: the narrow window (w = 8), the wide head
                 (N = 128, w = 512, float16) and the float32 band that covers the sequence.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c4|c5|c5_w33_bf16|...] [--no-cpu] [--no-others]
       python bench.py --kernels-only [--shape B M N w] [--dtype bf16|fp16|fp32|fp64] [--family auto|wide|staged|strided]
"""
import argparse
import hashlib
import json
import os
import statistics
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(REPO, "pytorch-window-matmul_amd")
for _p in (REPO, PKG):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0      # MI355X published HBM3E bandwidth
MFMA_PEAK_TFLOPS = 2500.0  # dense bf16 / fp16 matrix peak
FP32_PEAK_TFLOPS = 157.3   # float32 matrix peak
FP64_PEAK_TFLOPS = 78.6    # float64 matrix peak

WORKLOADS = {
    "c3": dict(B=96, M=4096, N=64, w=256, dtype="bf16", qk_scale=0.125, backward=True,
               label="B96 M4096 N64 w256 bf16, window->softmax->unwindow, fwd+bwd"),
    "c2": dict(B=96, M=16384, N=64, w=8, dtype="bf16", qk_scale=1.0, backward=False,
               label="B96 M16384 N64 w8 bf16, window->softmax->unwindow, fwd"),
    "c4": dict(B=16, M=32768, N=128, w=512, dtype="fp16", qk_scale=1.0, backward=True,
               label="B16 M32768 N128 w512 fp16, window->softmax->unwindow, fwd+bwd"),
    "c5": dict(B=7, M=3001, N=80, w=1500, dtype="fp32", qk_scale=1.0, backward=True,
               label="B7 M3001 N80 w1500 fp32, window->softmax->unwindow, fwd+bwd"),
}
# the other windows and storage type of the ragged configuration (per-kernel figures on the default run)
for _w in (1, 33, 1500):
    for _dt in ("fp32", "bf16"):
        if (_w, _dt) != (1500, "fp32"):
            WORKLOADS[f"c5_w{_w}_{_dt}"] = dict(
                B=7, M=3001, N=80, w=_w, dtype=_dt, qk_scale=1.0, backward=True,
                label=f"B7 M3001 N80 w{_w} {_dt}, window->softmax->unwindow, fwd+bwd")
# a single long sequence and a single short one (launches with far fewer tiles than CUs; --kernels-only
# runs for the kernel trace in profiles/, not part of the default run)
WORKLOADS["one_sequence_16k"] = dict(B=1, M=16384, N=128, w=1024, dtype="bf16", qk_scale=1.0, backward=True,
                                     label="B1 M16384 N128 w1024 bf16, window->softmax->unwindow, fwd+bwd")
WORKLOADS["one_sequence_4k"] = dict(B=1, M=4096, N=128, w=256, dtype="bf16", qk_scale=1.0, backward=True,
                                    label="B1 M4096 N128 w256 bf16, window->softmax->unwindow, fwd+bwd")
# source files the dominant kernel of the headline configuration can come from (the wide-band 16-bit
# family, its shared headers and the dispatcher that picks it): the digest of these guards the HBM
# traffic figure stored in profiles/config3_bf16_hbm_traffic.md
TRAFFIC_SOURCES = ("wm_mfma.hip", "wm_mfma_common.hpp", "wm_common.hpp", "wm_types.hpp", "wm_api.hip")


def band_unit_flops(B, M, N, w):
    valid = M * (2 * w + 1) - w * (w + 1) if w <= M - 1 else M * M
    return 2.0 * B * N * valid


def kernel_bytes(B, M, N, w, es):
    """Algorithmic HBM bytes of one launch, every operand touched once."""
    W = 2 * w + 1
    band, mat = B * M * W * es, B * M * N * es
    return band + 2 * mat  # P1: X, Y in, band out;  P2 / P3: band, Y in, C out


def kernel_source_digest():
    h = hashlib.sha256()
    for name in TRAFFIC_SOURCES:
        with open(os.path.join(PKG, "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profiled_traffic(kernel_label):
    """HBM bytes per launch of the dominant kernel as measured with rocprofv3 counters (FETCH_SIZE and
    WRITE_SIZE runs, scaled by a copy of known size), read from the committed summary.  The summary
    names the digest of the kernel sources it was measured on: when the sources have changed since,
    the stored figure says nothing about this run and None is returned."""
    path = os.path.join(REPO, "profiles", "config3_bf16_hbm_traffic.md")
    prim = {"P1": "p1", "P2": "p2", "P3": "p3"}.get(kernel_label[-3:-1])
    value, digest = None, None
    try:
        for line in open(path):
            parts = line.split()
            if len(parts) == 3 and parts[0] == "traffic_bytes_per_launch" and parts[1] == prim:
                value = int(parts[2])
            if len(parts) == 2 and parts[0] == "kernel_source_digest":
                digest = parts[1]
    except OSError:
        return None, None
    if digest != kernel_source_digest():
        return None, digest
    return value, digest


def time_gpu(fn, iters, warmup, settle_ms=0.0):
    """Median duration of one launch, each launch bracketed by its own pair of HIP events on the
    current stream (so that the gap between dependent launches is not counted as kernel time).
    The untimed launches before it go on until `settle_ms` of GPU time have passed: after a pause
    (host-side input generation between workloads) the first 10 ms of a run of launches are a clock
    transient, 300 rising to 400 and settling at 310 us per launch for the band-out product at
    B16 M32768 N128 w512, and a median over 10 launches taken inside it is not the kernel's rate."""
    import torch

    for _ in range(warmup):
        fn()
    if settle_ms > 0:
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(1000):  # bounded: a launch that takes no time cannot spin here
            for _ in range(4):
                fn()
            stop.record()
            stop.synchronize()
            if start.elapsed_time(stop) >= settle_ms:
                break
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    torch.cuda.synchronize()
    for start, stop in pairs:
        start.record()
        fn()
        stop.record()
    torch.cuda.synchronize()
    return statistics.median(a.elapsed_time(b) for a, b in pairs)  # ms


def time_steps(fn, steps, warmup):
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def cpu_baseline(cfg, seconds_budget=20.0):
    """Times the C restatement of the reference's scalar CPU path on one thread over a batch slice, and
    the reference's own compiled CPU path beside it where that build is present."""
    import torch

    import oracle

    torch.set_num_threads(1)
    M, N, w = cfg["M"], cfg["N"], cfg["w"]
    rnd = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32, "fp64": torch.float64}[cfg["dtype"]]

    def run(impl, budget):
        g = torch.Generator().manual_seed(0)

        def rounded(*shape, scale=1.0):
            return (torch.randn(*shape, generator=g) * scale).to(rnd).float()

        done, elapsed, flops = 0, 0.0, 0.0
        while elapsed < budget and done < cfg["B"]:
            q, k, v, go = (rounded(1, M, N, scale=s) for s in (cfg["qk_scale"], cfg["qk_scale"], 1.0, 1.0))
            kt = k.transpose(1, 2).contiguous()
            t0 = time.perf_counter()
            att = impl.window_matmul_forward(q, kt, w)
            probs = att.softmax(-1)
            impl.unwindow_matmul_forward(probs, v, w)
            units = 2
            if cfg["backward"]:
                ga, _ = impl.unwindow_matmul_backward(probs, v, w, go)
                impl.window_matmul_backward(q, kt, w, ga)
                units = 6
            elapsed += time.perf_counter() - t0
            done += 1
            flops += units * band_unit_flops(1, M, N, w)
        return flops / elapsed / 1e12, done, elapsed

    ref = oracle.reference_module()
    value, done, elapsed = run(oracle, seconds_budget * (0.35 if ref is not None else 0.5))
    out = {
        "value": value,
        "unit": "TFLOP/s",
        "cores": 1,
        "kind": "port",
        "sample": f"{done} of {cfg['B']} batch elements at full M, N, w; float32 copies of the rounded inputs; "
                  f"{elapsed:.1f} s of CPU time (softmax between the ops included, as on the GPU)",
        "host_cpus": os.cpu_count(),
    }
    if ref is not None:
        rvalue, rdone, relapsed = run(ref, seconds_budget * 0.15)
        out["reference_cpu_path"] = {"value": rvalue, "unit": "TFLOP/s", "cores": 1,
                                     "sample": f"{rdone} batch elements, {relapsed:.1f} s; the reference's own "
                                               "scalar kernels compiled from its sources"}
    return out


class Bench:
    """Tensors and launches of one configuration."""

    def __init__(self, cfg, family):
        import torch

        import wm_ctypes as abi

        self.cfg, self.abi, self.torch, self.fam = cfg, abi, torch, family
        self.B, self.M, self.N, self.w = cfg["B"], cfg["M"], cfg["N"], cfg["w"]
        self.dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32,
                      "fp64": torch.float64}[cfg["dtype"]]
        self.es = torch.empty((), dtype=self.dtype).element_size()
        self.dev = torch.device("cuda:0")
        self.g = torch.Generator().manual_seed(0)
        self.q, self.k = self.synth(cfg["qk_scale"]), self.synth(cfg["qk_scale"])
        self.v, self.go = self.synth(), self.synth()
        self.unit = band_unit_flops(self.B, self.M, self.N, self.w)

    def synth(self, scale=1.0):
        return (self.torch.randn(self.B, self.M, self.N, generator=self.g) * scale).to(self.dtype).to(self.dev)

    def kernels(self, iters, settle_ms=30.0):
        """Per-kernel timing through the C ABI (one launch per call), same tensors, same stream.
        `settle_ms` of untimed launches precede every timing (0 for profiler passes, which want
        few launches and say how many they saw)."""
        torch, abi, cfg, w, fam = self.torch, self.abi, self.cfg, self.w, self.fam
        B, M, N, es = self.B, self.M, self.N, self.es
        out = {}
        with torch.no_grad():
            q, k, v, go = self.q.detach(), self.k.detach(), self.v.detach(), self.go
            kt = k.transpose(1, 2)
            att = abi.window_forward(q, kt, w)
            probs = torch.softmax(att, dim=-1)
            ga = None
            launches = {
                "window_fwd(P1)": lambda: abi.window_forward(q, kt, w, fam, out=att),
                "unwindow_fwd(P2)": lambda: abi.unwindow_forward(probs, v, w, fam),
            }
            if cfg["backward"]:
                ga = torch.randn(B, M, 2 * w + 1, generator=self.g).to(self.dtype).to(self.dev)
                launches.update({
                    "grad_a(P1)": lambda: abi.unwindow_backward(probs, v, w, go, fam, want_v=False),
                    "grad_v(P3)": lambda: abi.unwindow_backward(probs, v, w, go, fam, want_a=False),
                    "grad_q(P2)": lambda: abi.window_backward(q, kt, w, ga, fam, want_k=False),
                    "grad_k(P3)": lambda: abi.window_backward(q, kt, w, ga, fam, want_q=False),
                })
            kb = kernel_bytes(B, M, N, w, es)
            per_kernel = {}
            if cfg["backward"] and B * M <= (1 << 16):
                # a problem this small pays for launches, not arithmetic: the two backward ops as their callers
                # issue them (both gradients from one call; the library makes that one launch where it can)
                launches.update({
                    "unwindow_bwd(both)": lambda: abi.unwindow_backward(probs, v, w, go, fam),
                    "window_bwd(both)": lambda: abi.window_backward(q, kt, w, ga, fam),
                })
            for name, fn in launches.items():
                ms = single = time_gpu(fn, iters, 3, settle_ms)
                if single < 0.05:
                    # a launch this short is mostly the event pair around it (14-25 us): time trains of
                    # 20 back-to-back launches between one pair instead and report the single-launch
                    # figure beside it
                    ms = time_gpu(lambda: [fn() for _ in range(20)], iters, 1, 0.0) / 20
                per_kernel[name] = {"ms": round(ms, 4), "GBps": round(kb / ms / 1e6, 1),
                                    "hbm_frac": round(kb / ms / 1e6 / HBM_PEAK_GBS, 4),
                                    "TFLOPs": round(self.unit / ms / 1e9, 1)}
                if ms is not single:
                    per_kernel[name]["single_launch_ms"] = round(single, 4)
            out["kernels"], out["algorithmic_bytes_per_launch"] = per_kernel, kb
            out["softmax_fwd_ms"] = round(time_gpu(lambda: torch.softmax(att, dim=-1), iters, 3, settle_ms), 4)
            band_bytes = att.numel() * es
            sm_out = torch.empty_like(att)
            bs_fwd = time_gpu(lambda: abi.band_softmax_forward(att, 1.0, out=sm_out), iters, 3, settle_ms)
            bs_bwd = time_gpu(lambda: abi.band_softmax_backward(probs, ga if ga is not None else att, 1.0, out=sm_out),
                              iters, 3, settle_ms)
            out["band_softmax"] = {"fwd_ms": round(bs_fwd, 4), "fwd_GBps": round(2 * band_bytes / bs_fwd / 1e6, 1),
                                   "bwd_ms": round(bs_bwd, 4), "bwd_GBps": round(3 * band_bytes / bs_bwd / 1e6, 1)}
            # the fused kernels are 16-bit only (N a multiple of 16 up to 128); other shapes run the chain of separate ops
            if es == 2 and abi.lib().wm_window_attention_supported(M, N, w, abi.DTYPES[self.dtype], 1.0):
                fo, flse = abi.attention_forward(q, k, v, w, 1.0)
                fwd = time_gpu(lambda: abi.attention_forward(q, k, v, w, 1.0), iters, 3, settle_ms)
                fused = {"fwd_ms": round(fwd, 4), "fwd_TFLOPs": round(2 * self.unit / fwd / 1e9, 1),
                         "fwd_mfma_frac": round(2 * self.unit / fwd / 1e9 / MFMA_PEAK_TFLOPS, 4),
                         "fwd_hbm_frac": round((4 * B * M * N * es + 4 * B * M) / fwd / 1e6 / HBM_PEAK_GBS, 4)}
                # (a forward-only workload gets the backward of a training step as well: its band is so
                # narrow that the step is bound by the eight tensors it reads and writes, q k v o dO dq dk dv)
                bwd = time_gpu(lambda: abi.attention_backward(q, k, v, fo, flse, go, w, 1.0), iters, 3, settle_ms)
                fused.update({"bwd_ms": round(bwd, 4), "bwd_TFLOPs": round(4 * self.unit / bwd / 1e9, 1),
                              "bwd_mfma_frac": round(4 * self.unit / bwd / 1e9 / MFMA_PEAK_TFLOPS, 4),
                              "bwd_hbm_frac": round((8 * B * M * N * es + 4 * B * M) / bwd / 1e6 / HBM_PEAK_GBS, 4),
                              "step_mfma_frac": round(6 * self.unit / (fwd + bwd) / 1e9 / MFMA_PEAK_TFLOPS, 4)})
                out["fused_attention"] = fused
                del fo, flse
            # device-to-device copy of the band as the achievable-bandwidth yardstick
            scratch = torch.empty_like(att)
            copy_ms = time_gpu(lambda: scratch.copy_(att), iters, 3, settle_ms)
            out["copy_yardstick_GBps"] = round(2 * att.numel() * es / copy_ms / 1e6, 1)
            out["copy_bytes_each_way"] = att.numel() * es
        both = {n: per_kernel.pop(n) for n in list(per_kernel) if n.endswith("(both)")}
        if both:
            out["backward_ops"] = {n: {"ms": x["ms"], "single_launch_ms": x.get("single_launch_ms", x["ms"])} for n, x in both.items()}
        dom = max(per_kernel, key=lambda n: per_kernel[n]["ms"])
        out["slowest_kernel"] = dom
        if per_kernel[dom]["ms"] < 0.03:
            out["note"] = ("launches of 10-20 us in trains of 20: what is timed is the rate at which the host "
                           "(Python, one output allocation per call) issues them, not the kernels")
        # float32 and float64 are bound by their matrix rate once a launch has more FLOP per algorithmic
        # byte than the ridge of that rate against 8 TB/s (19.7 and 9.8 FLOP/B); 16-bit storage never gets
        # there (ridge 312 FLOP/B) and narrow windows are streams in every type
        name, peak = {torch.float32: ("float32", FP32_PEAK_TFLOPS), torch.float64: ("float64", FP64_PEAK_TFLOPS)}.get(
            self.dtype, ("16-bit", MFMA_PEAK_TFLOPS))
        if self.unit / out["algorithmic_bytes_per_launch"] > peak * 1e12 / (HBM_PEAK_GBS * 1e9):
            out["bound"] = "mfma (%s matrix peak %.1f TFLOP/s)" % (name, peak)
            out["slowest_kernel_frac"] = round(per_kernel[dom]["TFLOPs"] / peak, 4)
        else:
            out["bound"] = "hbm"
            out["slowest_kernel_frac"] = per_kernel[dom]["hbm_frac"]
        return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--shape", type=int, nargs=4, metavar=("B", "M", "N", "w"),
                    help="time this shape instead of a named workload (forward + backward)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp16", "fp32", "fp64"],
                    help="storage type for --shape")
    ap.add_argument("--family", default="auto", choices=["auto", "wide", "staged", "strided"],
                    help="kernel family for the per-kernel timings: the library's choice, the wide-band MFMA "
                         "kernels even for a narrow band, the library's choice without the kernels that load "
                         "their tiles straight into LDS, or the strided kernels (A/B measurements)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-others", action="store_true", help="skip the per-kernel timings at the other configurations")
    ap.add_argument("--kernels-only", action="store_true",
                    help="launch each of the six kernels --steps times and a reference copy, nothing else "
                         "(for rocprofv3 counter passes)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (the path shards over the batch "
                 "dimension with no communication, which one GPU cannot show)")

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    import wm_ctypes as abi
    from window_matmul import band_softmax, unwindow_matmul, window_attention, window_matmul

    cfg = WORKLOADS[args.workload]
    if args.shape:
        sb, sm, sn, sw = args.shape
        cfg = dict(B=sb, M=sm, N=sn, w=sw, dtype=args.dtype, qk_scale=sn ** -0.25, backward=True,
                   label=f"B{sb} M{sm} N{sn} w{sw} {args.dtype}, window->softmax->unwindow, fwd+bwd")
        args.workload = "custom"
    fam = {"auto": 0, "wide": abi.NO_NARROW_BAND, "staged": abi.NO_LDS_DIRECT, "strided": abi.FORCE_STRIDED}[args.family]
    iters = max(args.steps, 10)
    bench = Bench(cfg, fam)
    B, M, N, w = bench.B, bench.M, bench.N, bench.w

    if args.kernels_only:
        k = bench.kernels(iters, settle_ms=0.0)
        print(json.dumps({"workload": cfg["label"], "family": args.family, "kernels": k["kernels"],
                          "backward_ops": k.get("backward_ops"),
                          "fused_attention": k.get("fused_attention"), "band_softmax": k["band_softmax"],
                          "copy_yardstick_GBps": k["copy_yardstick_GBps"],
                          "copy_bytes_each_way": k["copy_bytes_each_way"]}), flush=True)
        return

    q, k, v, go = bench.q, bench.k, bench.v, bench.go
    if cfg["backward"]:  # forward-only workloads are inference: no autograd graph is recorded
        q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)

    def step(softmax=lambda att: torch.softmax(att, dim=-1)):
        att = window_matmul(q, k.transpose(1, 2), w)
        probs = softmax(att)
        out = unwindow_matmul(probs, v, w)
        if cfg["backward"]:
            q.grad = k.grad = v.grad = None
            out.backward(go)
        return out

    def fused_step():  # the whole chain as one call: fused kernels, the band never reaches memory
        out = window_attention(q, k, v, w, scale=1.0)
        if cfg["backward"]:
            q.grad = k.grad = v.grad = None
            out.backward(go)
        return out

    units = 6 if cfg["backward"] else 2
    flops = units * bench.unit
    ms_per_step = time_steps(step, args.steps, args.warmup)
    # the same chain with this library's band softmax in place of torch's (one changed line in
    # caller code; reported beside the drop-in figure, never as `value`)
    band_ms_per_step = time_steps(lambda: step(band_softmax), args.steps, args.warmup)
    fused_ms_per_step = time_steps(fused_step, args.steps, args.warmup)

    kern = bench.kernels(iters)
    per_kernel, kb = kern["kernels"], kern["algorithmic_bytes_per_launch"]
    dom = kern["slowest_kernel"]
    achieved = per_kernel[dom]["GBps"]
    traffic, digest = profiled_traffic(dom) if args.workload == "c3" else (None, None)
    fused = dict(kern.get("fused_attention") or {})
    fused.update({"ms_per_step": round(fused_ms_per_step, 4), "TFLOPs": round(flops / fused_ms_per_step / 1e9, 2),
                  "mfma_frac": round(flops / fused_ms_per_step / 1e9 / MFMA_PEAK_TFLOPS, 4),
                  "note": "same chain as one call, window_matmul.window_attention (autograd step); band FLOPs "
                          "credited as for the separate ops (recomputation in the backward not counted); "
                          "fractions against 2.5 PFLOP/s"})
    band = dict(kern["band_softmax"])
    band.update({"ms_per_step": round(band_ms_per_step, 4), "TFLOPs": round(flops / band_ms_per_step / 1e9, 2),
                 "note": "same chain with window_matmul.band_softmax replacing torch.softmax"})
    result = {
        "metric": "fwd+bwd TFLOP/s & HBM GB/s, window+unwindow, B96 M4096 N64 w256 bf16" if args.workload == "c3"
                  else f"band TFLOP/s, window+unwindow, {cfg['label']}",
        "value": round(flops / ms_per_step / 1e9, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": cfg["label"], "B": B, "M": M, "N": N, "w": w,
                   "band_gflop_per_step": round(flops / 1e9, 2)},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_source": "profiles/config3_bf16_hbm_traffic.md, kernel sources %s" % digest
                                       if traffic is not None else
                                       "not measured in this run; the committed counter summary is for other kernel sources",
                     "kernel": dom, "algorithmic_bytes_per_launch": kb, "median_launch_ms": per_kernel[dom]["ms"]},
        "kernels": per_kernel,
        "softmax_fwd_ms": kern["softmax_fwd_ms"],
        "band_softmax": band,
        "fused_attention": fused,
        "copy_yardstick_GBps": kern["copy_yardstick_GBps"],
        "kernel_sum_GBps": round(len(per_kernel) * kb / sum(x["ms"] for x in per_kernel.values()) / 1e6, 1),
    }
    del bench, q, k, v, go
    torch.cuda.empty_cache()
    if not args.no_others and args.workload == "c3":
        others = {}
        for name in ["c2", "c4", "c5"] + sorted(n for n in WORKLOADS if n.startswith("c5_")):
            ocfg = WORKLOADS[name]
            ob = Bench(ocfg, 0)
            others[name] = {"workload": ocfg["label"], **ob.kernels(10)}
            del ob
            torch.cuda.empty_cache()
        result["other_configs"] = others
        # the two stated targets, next to the roofline so that they are read with it: fused forward +
        # backward at this shape against half the dense bf16 matrix peak, and the slowest kernel of the
        # narrow-window configuration against 0.7 of the HBM peak
        result["roofline"]["targets"] = {
            "c3_fused_step_mfma_frac": fused.get("mfma_frac"),
            "c3_fused_step_kernels_only_mfma_frac": fused.get("step_mfma_frac"),
            "c3_fused_fwd_mfma_frac": fused.get("fwd_mfma_frac"),
            "c3_fused_bwd_mfma_frac": fused.get("bwd_mfma_frac"),
            "c3_fused_target_mfma_frac": 0.5,
            "c2_slowest_kernel": others["c2"]["slowest_kernel"],
            "c2_slowest_kernel_hbm_frac": others["c2"]["slowest_kernel_frac"],
            "c2_target_hbm_frac": 0.7,
        }
    result["cpu_baseline"] = None if args.no_cpu else cpu_baseline(cfg)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
