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

  roofline      the slowest of the six kernels, timed alone with HIP events on the stream
                it is launched on, priced against the 8 TB/s HBM peak on its algorithmic
                bytes (each operand touched once);
  cpu_baseline  the reference's own scalar CPU path (oracle/_ref, where built) or its C
                restatement, one thread, on a slice of the batch.

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c4] [--no-cpu]
       python bench.py --kernels-only [--shape B M N w] [--dtype bf16|fp16|fp32] [--family auto|wide|strided]
"""
import argparse
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(REPO, "pytorch-window-matmul_amd")
for _p in (REPO, PKG):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

WORKLOADS = {
    # name: (B, M, N, w, dtype, qk_scale, backward)
    "c3": dict(B=96, M=4096, N=64, w=256, dtype="bf16", qk_scale=0.125, backward=True,
               label="B96 M4096 N64 w256 bf16, window->softmax->unwindow, fwd+bwd"),
    "c2": dict(B=96, M=16384, N=64, w=8, dtype="bf16", qk_scale=1.0, backward=False,
               label="B96 M16384 N64 w8 bf16, window->softmax->unwindow, fwd"),
    "c4": dict(B=16, M=32768, N=128, w=512, dtype="fp16", qk_scale=1.0, backward=True,
               label="B16 M32768 N128 w512 fp16, window->softmax->unwindow, fwd+bwd"),
}


def band_unit_flops(B, M, N, w):
    valid = M * (2 * w + 1) - w * (w + 1) if w <= M - 1 else M * M
    return 2.0 * B * N * valid


def kernel_bytes(B, M, N, w, es):
    """Algorithmic HBM bytes of one launch, every operand touched once."""
    W = 2 * w + 1
    band, mat = B * M * W * es, B * M * N * es
    return band + 2 * mat  # P1: X, Y in, band out;  P2 / P3: band, Y in, C out


def profiled_traffic(kernel_label):
    """HBM bytes per launch of the dominant kernel as measured with rocprofv3 counters (FETCH_SIZE and
    WRITE_SIZE runs, scaled by a copy of known size); read from the committed summary, None if absent."""
    path = os.path.join(REPO, "profiles", "config3_bf16_hbm_traffic.md")
    prim = {"P1": "p1", "P2": "p2", "P3": "p3"}.get(kernel_label[-3:-1])
    try:
        for line in open(path):
            parts = line.split()
            if len(parts) == 3 and parts[0] == "traffic_bytes_per_launch" and parts[1] == prim:
                return int(parts[2])
    except OSError:
        pass
    return None


def time_gpu(fn, iters, warmup):
    """Mean duration of one launch, each launch bracketed by its own pair of HIP events on the
    current stream (so that the gap between dependent launches is not counted as kernel time)."""
    import torch

    for _ in range(warmup):
        fn()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    torch.cuda.synchronize()
    for start, stop in pairs:
        start.record()
        fn()
        stop.record()
    torch.cuda.synchronize()
    return sum(a.elapsed_time(b) for a, b in pairs) / iters  # ms


def cpu_baseline(cfg, seconds_budget=20.0):
    """Times the reference CPU path (or its restatement) on one thread over a batch slice."""
    import torch

    import oracle

    torch.set_num_threads(1)
    ref = oracle.reference_module()
    kind = "reference" if ref is not None else "port"
    impl = ref if ref is not None else oracle
    M, N, w = cfg["M"], cfg["N"], cfg["w"]
    g = torch.Generator().manual_seed(0)
    rnd = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[cfg["dtype"]]

    def rounded(*shape, scale=1.0):
        return (torch.randn(*shape, generator=g) * scale).to(rnd).float()

    slice_b, done, elapsed = 1, 0, 0.0
    flops = 0.0
    while elapsed < seconds_budget * 0.5 and done < cfg["B"]:
        q, k, v, go = (rounded(slice_b, M, N, scale=s) for s in (cfg["qk_scale"], cfg["qk_scale"], 1.0, 1.0))
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
        done += slice_b
        flops += units * band_unit_flops(slice_b, M, N, w)
    return {
        "value": flops / elapsed / 1e12,
        "unit": "TFLOP/s",
        "cores": 1,
        "kind": kind,
        "sample": f"{done} of {cfg['B']} batch elements at full M, N, w; float32 copies of the rounded inputs; "
                  f"{elapsed:.1f} s of CPU time (softmax between the ops included, as on the GPU)",
        "host_cpus": os.cpu_count(),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--shape", type=int, nargs=4, metavar=("B", "M", "N", "w"),
                    help="time this shape instead of a named workload (forward + backward)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp16", "fp32"],
                    help="storage type for --shape")
    ap.add_argument("--family", default="auto", choices=["auto", "wide", "strided"],
                    help="kernel family for the per-kernel timings: the library's choice, the wide-band MFMA "
                         "kernels even for a narrow band, or the strided kernels (A/B measurements)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
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
    fam = {"auto": 0, "wide": abi.NO_NARROW_BAND, "strided": abi.FORCE_STRIDED}[args.family]
    B, M, N, w = cfg["B"], cfg["M"], cfg["N"], cfg["w"]
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[cfg["dtype"]]
    es = 4 if dtype == torch.float32 else 2
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)

    def synth(scale=1.0):
        return (torch.randn(B, M, N, generator=g) * scale).to(dtype).to(dev)

    q, k, v, go = synth(cfg["qk_scale"]), synth(cfg["qk_scale"]), synth(), synth()
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

    units = 6 if cfg["backward"] else 2
    flops = units * band_unit_flops(B, M, N, w)
    ms_per_step = float("nan")
    if not args.kernels_only:
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
        # the same chain with this library's band softmax in place of torch's (one changed line
        # in caller code; reported beside the drop-in figure, never as `value`)
        for _ in range(args.warmup):
            step(band_softmax)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step(band_softmax)
        torch.cuda.synchronize()
        band_ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

        # and the whole chain as one call: fused kernels, the band never reaches memory
        def fused_step():
            out = window_attention(q, k, v, w, scale=1.0)
            if cfg["backward"]:
                q.grad = k.grad = v.grad = None
                out.backward(go)
            return out

        for _ in range(args.warmup):
            fused_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fused_step()
        torch.cuda.synchronize()
        fused_ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # per-kernel timing through the C ABI (one launch per call), same tensors, same stream
    with torch.no_grad():
        kt = k.detach().transpose(1, 2)
        att = abi.window_forward(q.detach(), kt, w)
        probs = torch.softmax(att, dim=-1)
        ga = torch.randn(B, M, 2 * w + 1, generator=g).to(dtype).to(dev) if cfg["backward"] else None
        qd, vd = q.detach(), v.detach()
        launches = {
            "window_fwd(P1)": lambda: abi.window_forward(qd, kt, w, fam, out=att),
            "unwindow_fwd(P2)": lambda: abi.unwindow_forward(probs, vd, w, fam),
        }
        if cfg["backward"]:
            launches.update({
                "grad_a(P1)": lambda: abi.unwindow_backward(probs, vd, w, go, fam, want_v=False),
                "grad_v(P3)": lambda: abi.unwindow_backward(probs, vd, w, go, fam, want_a=False),
                "grad_q(P2)": lambda: abi.window_backward(qd, kt, w, ga, fam, want_k=False),
                "grad_k(P3)": lambda: abi.window_backward(qd, kt, w, ga, fam, want_q=False),
            })
        kb = kernel_bytes(B, M, N, w, es)
        per_kernel = {}
        for name, fn in launches.items():
            ms = time_gpu(fn, max(args.steps, 10), 3)
            per_kernel[name] = {"ms": round(ms, 4), "GBps": round(kb / ms / 1e6, 1),
                                "TFLOPs": round(band_unit_flops(B, M, N, w) / ms / 1e9, 1)}
        softmax_ms = time_gpu(lambda: torch.softmax(att, dim=-1), max(args.steps, 10), 3)
        band_bytes = att.numel() * es
        sm_out = torch.empty_like(att)
        bs_fwd_ms = time_gpu(lambda: abi.band_softmax_forward(att, 1.0, out=sm_out), max(args.steps, 10), 3)
        bs_bwd_ms = time_gpu(lambda: abi.band_softmax_backward(probs, ga if ga is not None else att, 1.0, out=sm_out),
                             max(args.steps, 10), 3)
        del sm_out
        fused_fwd_ms = fused_bwd_ms = None
        if es == 2:  # the fused kernels are 16-bit only; float32 runs the chain of separate ops
            fo, flse = abi.attention_forward(qd, k.detach(), vd, w, 1.0)
            fused_fwd_ms = time_gpu(lambda: abi.attention_forward(qd, k.detach(), vd, w, 1.0), max(args.steps, 10), 3)
            if cfg["backward"]:
                fused_bwd_ms = time_gpu(lambda: abi.attention_backward(qd, k.detach(), vd, fo, flse, go, w, 1.0),
                                        max(args.steps, 10), 3)
            del fo, flse
        # device-to-device copy of the band as the achievable-bandwidth yardstick
        scratch = torch.empty_like(att)
        copy_ms = time_gpu(lambda: scratch.copy_(att), 20, 3)
        copy_gbs = 2 * att.numel() * es / copy_ms / 1e6
    dom = max(per_kernel, key=lambda n: per_kernel[n]["ms"])
    achieved = per_kernel[dom]["GBps"]
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
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": profiled_traffic(dom) if args.workload == "c3" else None, "kernel": dom,
                     "algorithmic_bytes_per_launch": kb, "avg_launch_ms": per_kernel[dom]["ms"]},
        "kernels": per_kernel,
        "softmax_fwd_ms": round(softmax_ms, 4),
        "band_softmax": None if args.kernels_only else {
            "ms_per_step": round(band_ms_per_step, 4), "TFLOPs": round(flops / band_ms_per_step / 1e9, 2),
            "fwd_ms": round(bs_fwd_ms, 4), "fwd_GBps": round(2 * band_bytes / bs_fwd_ms / 1e6, 1),
            "bwd_ms": round(bs_bwd_ms, 4), "bwd_GBps": round(3 * band_bytes / bs_bwd_ms / 1e6, 1),
            "note": "same chain with window_matmul.band_softmax replacing torch.softmax"},
        "fused_attention": None if args.kernels_only else {
            "ms_per_step": round(fused_ms_per_step, 4), "TFLOPs": round(flops / fused_ms_per_step / 1e9, 2),
            "fwd_ms": None if fused_fwd_ms is None else round(fused_fwd_ms, 4),
            "bwd_ms": None if fused_bwd_ms is None else round(fused_bwd_ms, 4),
            "mfma_frac": round(flops / fused_ms_per_step / 1e9 / 2500.0, 4),
            "note": "same chain as one call, window_matmul.window_attention; band FLOPs credited as for the "
                    "separate ops (recomputation in the backward not counted); mfma_frac against 2.5 PFLOP/s"},
        "copy_yardstick_GBps": round(copy_gbs, 1),
        "kernel_sum_GBps": round(len(per_kernel) * kb / sum(v["ms"] for v in per_kernel.values()) / 1e6, 1),
    }
    if args.kernels_only:
        print(json.dumps({"workload": cfg["label"], "family": args.family, "kernels": per_kernel,
                          "copy_yardstick_GBps": round(copy_gbs, 1),
                          "copy_bytes_each_way": att.numel() * es}), flush=True)
        return
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(cfg)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
