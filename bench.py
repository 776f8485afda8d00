#!/usr/bin/env python3
"""Benchmark of the QLM 4-bit hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|adamw|decode|train]

Prints ONE JSON line. A "step" is one pass of a hot-path kernel set over one batch of synthetic
input that is already resident in HBM. Workloads (shapes from BASELINE.json `configs`):
  train   32-expert top-2 layer, D=768 F=2048, 8192 bf16 tokens, Zipf(1.1) load: grouped
          dequant-GEMM forward + dgrad + wgrad (TFLOP/s, bound: bf16 MFMA)
  decode  same layer weights x 8 distinct layers, 1/4/16 tokens top-2: grouped dequant-GEMV
          (GB/s of packed weights of the experts hit, bound: HBM)
  adamw   Integer AdamW + requantisation over 120*2^20 4-bit weights (GB/s, bound: HBM)
Each workload reports its own roofline object; the top-level `value`/`roofline` are the first
workload that ran in the order train, decode, adamw. `cpu_baseline` times the reference's own CPU
backend (oracle/_ref, kind "reference") or the repository's C restatement (kind "port") on a bounded
sample on this host's cores; it is a reported baseline, not the target.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="all", choices=["all", "adamw", "decode", "train"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--adamw-weights", type=int, default=120 * 2 ** 20)
    ap.add_argument("--render-p", type=int, default=0, help="adamw: also write the fp32 view P (4 B/weight more)")
    return ap.parse_args()


def timed(torch, fn, steps, warmup):
    """W untimed calls, then K timed ones bracketed by synchronize; per-call HIP-event times are
    taken on the stream the kernels run on (torch's current stream, handed to the library)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    per = sorted(a.elapsed_time(b) for a, b in evs)
    return {"wall_ms": wall, "event_ms_avg": sum(per) / len(per), "event_ms_med": per[len(per) // 2], "event_ms_min": per[0]}


# --------------------------------------------------------------------------------------------- adamw
def bench_adamw(torch, q, args):
    import numpy as np
    from cudalm_c_amd.binding import SPAN_DTYPE
    dev = torch.device("cuda:0")
    nq = (args.adamw_weights // 128) * 128
    ng = nq // 128
    g = torch.Generator(device=dev); g.manual_seed(0)
    d = torch.randint(-128, 128, (nq // 2,), dtype=torch.int8, device=dev, generator=g)
    # keep digits inside [-7,7]: clear the forbidden nibble value -8 (0x8) in both halves
    du = d.view(torch.uint8)
    lo = du & 15; hi = du >> 4
    lo = torch.where(lo == 8, torch.zeros_like(lo), lo); hi = torch.where(hi == 8, torch.zeros_like(hi), hi)
    d = (lo | (hi << 4)).view(torch.int8)
    r = torch.randint(-64, 65, (nq,), dtype=torch.int8, device=dev, generator=g)
    m8 = torch.randint(-127, 128, (nq,), dtype=torch.int8, device=dev, generator=g)
    v8 = torch.randint(0, 256, (nq,), dtype=torch.int16, device=dev, generator=g).to(torch.uint8)
    s = (0.02 * 3 / 7) * (0.5 + torch.rand(ng, device=dev, generator=g))
    m8s = (3e-3 / 127) * (0.5 + torch.rand(ng, device=dev, generator=g))
    v8s = (3e-3 / 255) * (0.5 + torch.rand(ng, device=dev, generator=g))
    G = 1e-3 * torch.randn(nq, device=dev, generator=g)
    P = torch.empty(nq, device=dev) if args.render_p else None
    tab = np.zeros(1, dtype=SPAN_DTYPE)
    tab[0] = (0, 0, 0, nq, 0, ng, float(s.mean()), 0)
    sp = torch.from_numpy(tab.view(np.uint8)).to(dev)
    stream = torch.cuda.current_stream().cuda_stream
    state = {"t": 0}
    b1, b2 = 0.9, 0.95

    def step():
        state["t"] += 1
        t = state["t"]
        bc1 = 1.0 - b1 ** t; bc2 = 1.0 - b2 ** t
        q.step(P, G, d, r, s, m8, m8s, v8, v8s, sp, 1, 128, 7, 3e-4, b1, b2, 0.1, 1.0, None,
               1.0 / bc1, 1.0 / bc2 ** 0.5, 0, t, 1, None, 1, 0, ng, 0, stream)

    tm = timed(torch, step, args.steps, args.warmup)
    bytes_per_w = 11.0 + 20.0 / 128 + (4.0 if args.render_p else 0.0)
    algo_bytes = nq * bytes_per_w
    gbs = algo_bytes / (tm["event_ms_avg"] * 1e-3) / 1e9
    return {
        "workload": "C4 integer AdamW sweep, %d weights, group 128, 4-bit packed, P %s" % (nq, "rendered" if args.render_p else "not rendered"),
        "metric": "int-AdamW GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": tm["wall_ms"], "dtype": "u8+f32",
        "kernel_ms": tm, "weights_per_s": nq / (tm["event_ms_avg"] * 1e-3),
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                     "traffic": None, "kernel": "k_qlmx_step<adam>", "bytes_per_weight": bytes_per_w},
    }


def cpu_adamw(args):
    """Reference CPU Integer AdamW on a bounded sample (same distributions, 16M weights)."""
    import numpy as np
    from oracle.binding import Oracle, Ref, have_ref, make_spans
    orc = Oracle()
    threads = min(16, os.cpu_count() or 1)
    kind = "reference" if have_ref() else "port"
    lib = Ref(threads=threads) if kind == "reference" else orc
    orc.set_threads(threads)
    nq = 16 * 2 ** 20
    tab, _, ng = make_spans([nq], 128)
    d = orc.digits(nq, 0, 1); r = orc.int8(nq, 0, 2, -64, 64); m8 = orc.int8(nq, 0, 3, -127, 127)
    v8 = orc.u8(nq, 0, 4, 0, 255)
    s = orc.uniform(ng, 0, 5, 0.5, 1.5) * np.float32(0.02 * 3 / 7)
    m8s = orc.uniform(ng, 0, 6, 0.5, 1.5) * np.float32(3e-3 / 127)
    v8s = orc.uniform(ng, 0, 7, 0.5, 1.5) * np.float32(3e-3 / 255)
    tab["sref"] = float(s.mean())
    G = orc.normal(nq, 0, 8, 1e-3)
    P = np.zeros(nq, np.float32)
    reps, t_used = 0, 0.0
    lib.step(P, G, d, r, s, m8, m8s, v8, v8s, tab, 128, 7, 3e-4, 0.9, 0.95, 0.1, 1.0, None, 10.0, 4.47, 0, 1, 1, None, 1, 0, ng)
    while t_used < 8.0 and reps < 50:
        t0 = time.perf_counter()
        lib.step(P, G, d, r, s, m8, m8s, v8, v8s, tab, 128, 7, 3e-4, 0.9, 0.95, 0.1, 1.0, None, 10.0, 4.47, 0, 2 + reps, 1, None, 1, 0, ng)
        t_used += time.perf_counter() - t0
        reps += 1
    gbs = nq * 15.16 * reps / t_used / 1e9
    return {"value": gbs, "unit": "GB/s", "cores": threads, "kind": kind,
            "sample": "Integer AdamW (P rendered, 15.16 B/weight) over %d weights x %d steps, %s" % (nq, reps, "cpu_kern.h cpu_qlm_step" if kind == "reference" else "oracle/qlm_oracle.c"),
            "weights_per_s": nq * reps / t_used}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU's share of the path; --gpus must be 1 "
              "(no collective, IPC or multi-rank code exists in it)", file=sys.stderr)
        sys.exit(2)
    import torch
    from __graft_entry__ import load_package
    pkg = load_package()
    q = pkg.load()           # raises if libqlmx.so is missing or no gfx950 device
    torch.cuda.set_device(0)
    want = ["train", "decode", "adamw"] if args.workload == "all" else [args.workload]
    runners = {"adamw": bench_adamw}
    results = {}
    for w in want:
        if w in runners:
            results[w] = runners[w](torch, q, args)
    first = next(results[w] for w in ["train", "decode", "adamw"] if w in results)
    line = {
        "metric": "QLM expert dequant-GEMM TFLOP/s & GB/s (% roofline); int-AdamW GB/s",
        "value": first["value"], "unit": first["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": first["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": first["dtype"], "data": "synthetic",
        "config": {"workload": first["workload"]},
        "roofline": first["roofline"],
        "workloads": results,
        "device": q.call("qlmx_device_name").decode(),
    }
    if not args.no_cpu:
        if "adamw" in results:
            line["cpu_baseline"] = cpu_adamw(args)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
