#!/usr/bin/env python3
"""Benchmark of the QLM 4-bit hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|adamw|decode|train|train5|codec|glue]

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
Defaults: 30 warm-up and 100 timed steps. The device takes some 20 ms of load to reach the clock it then
holds; with 3 + 20 steps of 1 ms the timed region would lie inside that ramp and read 8 % low, so every
measurement is preceded by 40 ms of the same calls, untimed, in addition to the W warm-up steps.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SETTLE_MS = 40.0               # untimed load in front of every measurement (clock ramp, see the docstring)
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--workload", default="all", choices=["all", "adamw", "decode", "train", "train5", "c5", "layer", "codec", "glue", "copy"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--fwd-math", default="f16", choices=["f16", "bf16x2"],
                    help="train, c5: forward GEMMs on the fp16 matrix core (one MFMA per product, 2e-4 relative L2) or as bf16 hi+lo (two, 3e-6)")
    ap.add_argument("--bwd", default="pair", choices=["pair", "serial", "streams"],
                    help="train, c5: the two grouped GEMMs of every backward flush as one launch (qlmx_pair_begin / qlmx_pair_end), "
                         "one after the other, or the weight gradient on the library's side stream beside the input gradient")
    ap.add_argument("--step-only", action="store_true", help="train: skip the per-launch repetitions, so that a kernel trace holds nothing but steps; "
                    "layer: time the merged layer only (no pass-by-pass forms, no glue-only run)")
    ap.add_argument("--adamw-weights", type=int, default=120 * 2 ** 20)
    ap.add_argument("--render-p", type=int, default=0, help="adamw: also write the fp32 view P (4 B/weight more)")
    return ap.parse_args()


def timed(torch, fn, steps, warmup):
    """W untimed calls, then exactly K timed ones bracketed by synchronize. One pair of HIP events on the
    stream the kernels run on (torch's current stream, handed to the library) spans the K calls: an
    event between two calls would itself leave the GPU idle for some 6 us and be charged to the step."""
    # the device reaches the clock it then holds only after some 20 ms of load: keep it busy with the same
    # call for SETTLE_MS first, whatever W is, so that a short run does not time the ramp
    t_end = time.perf_counter() + SETTLE_MS * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return {"wall_ms": wall, "event_ms_avg": a.elapsed_time(b) / steps}


def step_spread(torch, fn, steps):
    """Duration of every single step of `steps` more (an event behind each: some 6 us of idle GPU per step ride along,
    which is why the mean comes from timed() and only the spread from here): a stall that a mean would hide shows as max."""
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    ev[0].record()
    for i in range(steps):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    ms = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(steps))
    return {"min": ms[0], "p50": ms[len(ms) // 2], "p99": ms[min(len(ms) - 1, (len(ms) * 99) // 100)], "max": ms[-1],
            "note": "per-step events: each adds a few us of idle GPU to its step"}



# --------------------------------------------------------------------------------------------- train
def zipf_counts(E, tokens, topk, seed=0):
    """Per-expert row counts when every token draws `topk` distinct experts with p_e ~ (e+1)^-1.1
    (Gumbel top-k = sampling without replacement)."""
    import numpy as np
    rng = np.random.default_rng(seed)
    logp = -1.1 * np.log(np.arange(E) + 1.0)
    keys = logp[None, :] + rng.gumbel(size=(tokens, E))
    top = np.argsort(-keys, axis=1)[:, :topk]
    return np.bincount(top.ravel(), minlength=E).astype(int)


def bench_train(torch, q, args, E=32, D=768, F=2048, tokens=8192, topk=2, label="C3 train layer"):
    from cudalm_c_amd.binding import ACT_BF16, MATH_MFMA, MATH_MFMA_F16
    FWD = MATH_MFMA if args.fwd_math == "bf16x2" else MATH_MFMA_F16
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev); g.manual_seed(0)
    cnt = zipf_counts(E, tokens, topk)
    rows = int(cnt.sum())
    off = [0]
    for c in cnt:
        off.append(off[-1] + int(c))
    group = 128
    nw = E * D * F

    def packed():
        b = torch.randint(0, 256, (nw // 2,), dtype=torch.int16, device=dev, generator=g).to(torch.uint8)
        lo = b & 15; hi = b >> 4
        lo = torch.where(lo == 8, torch.zeros_like(lo), lo); hi = torch.where(hi == 8, torch.zeros_like(hi), hi)
        return (lo | (hi << 4)).view(torch.int8)

    # one digit array holding w1 | w3 | w2 back to back, like consecutive spans of a layer
    d = torch.cat([packed(), packed(), packed()])
    s = (0.02 * 3 / 7) * (0.5 + torch.rand(3 * nw // group, device=dev, generator=g))
    o1, o3, o2 = 0, nw, 2 * nw

    def bf16(n, scale=1.0):
        return (scale * torch.randn(n, device=dev, generator=g)).to(torch.bfloat16)

    Xp, ap, dyp = bf16(rows * D), bf16(rows * F), bf16(rows * D)
    dgp, dup = bf16(rows * F), bf16(rows * F)
    gp = torch.empty(rows * F, device=dev); up = torch.empty(rows * F, device=dev); yp = torch.empty(rows * D, device=dev)
    dap = torch.empty(rows * F, device=dev); dXp = torch.empty(rows * D, device=dev)
    G = torch.zeros(3 * nw, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def probs(A, a_w, B, b_w, Cm, c_w, wbase, per_expert_c=False):
        items = []
        for e in range(E):
            m = int(cnt[e])
            items.append((A.data_ptr() + off[e] * a_w * 2, (B.data_ptr() + off[e] * b_w * 2) if B is not None else None,
                          (Cm.data_ptr() + (wbase + e * D * F) * 4) if per_expert_c else (Cm.data_ptr() + off[e] * c_w * 4),
                          wbase + e * D * F, (wbase + e * D * F) // group, m, 0.0))
        return items

    P = q.problems
    p_w13 = P(probs(Xp, D, None, 0, gp, F, o1) + probs(Xp, D, None, 0, up, F, o3))
    p_w2 = P(probs(ap, F, None, 0, yp, D, o2))
    p_d2 = P(probs(dyp, D, None, 0, dap, F, o2))
    p_d1 = P(probs(dgp, F, None, 0, dXp, D, o1))
    it3 = probs(dup, F, None, 0, dXp, D, o3)
    p_d3 = P([(a, b, c, wq, wg, m, 1.0) for (a, b, c, wq, wg, m, _) in it3])
    p_g2 = P(probs(ap, F, dyp, D, G, 0, o2, True))
    p_g13 = P(probs(Xp, D, dgp, F, G, 0, o1, True) + probs(Xp, D, dup, F, G, 0, o3, True))
    # the order of moe_forward / moe_backward (cudalm.cu:4211-4225, 4333-4335, 4362-4366): each backward flush
    # holds the weight gradient and the input gradient of the same operands
    def mk(st):
        return [
            ("fwd w1,w3 (nn)", lambda: q.gemm_nn(d, s, group, p_w13, 2 * E, D, F, ACT_BF16, FWD, st), 2),
            ("fwd w2 (nn)", lambda: q.gemm_nn(d, s, group, p_w2, E, F, D, ACT_BF16, FWD, st), 1),
            ("wgrad w2 (nt)", lambda: q.gemm_nt(p_g2, E, F, D, ACT_BF16, MATH_MFMA, st), 1),
            ("dgrad w2 (tn)", lambda: q.gemm_tn(d, s, group, p_d2, E, D, F, ACT_BF16, MATH_MFMA, st), 1),
            ("wgrad w1,w3 (nt)", lambda: q.gemm_nt(p_g13, 2 * E, D, F, ACT_BF16, MATH_MFMA, st), 2),
            ("dgrad w1,w3 (tn pair)", lambda: q.gemm_tn_pair(d, s, group, p_d1, p_d3, E, F, D, ACT_BF16, MATH_MFMA, st), 2),
        ]
    calls = mk(stream)
    unit = 2.0 * rows * D * F            # flops of one expert GEMM over all rows

    def step():
        for _, fn, _n in calls:
            fn()

    if args.bwd == "streams":
        # each backward flush (cudalm.cu:4333-4335, 4362-4366) with its weight gradient on the library's side
        # stream beside its input gradient: they read the same operands and write different outputs
        side = mk(q.side_fork(stream)); q.side_join(stream)      # the handle is the same at every fork

        def step():
            calls[0][1](); calls[1][1]()
            q.side_fork(stream); side[2][1](); calls[3][1](); q.side_join(stream)
            q.side_fork(stream); side[4][1](); calls[5][1](); q.side_join(stream)
    elif args.bwd == "pair":
        # each backward flush as one launch: the tiles of its weight gradient and of its input gradient in one grid
        def step():
            calls[0][1](); calls[1][1]()
            q.pair_begin(stream); calls[2][1](); calls[3][1](); q.pair_end(stream)
            q.pair_begin(stream); calls[4][1](); calls[5][1](); q.pair_end(stream)

    tm = timed(torch, step, args.steps, args.warmup)
    spread = step_spread(torch, step, args.steps)
    per = {}
    for name, fn, ng in ([] if args.step_only else calls):
        t1 = timed(torch, fn, max(5, args.steps // 2), 2)
        per[name] = {"ms": t1["event_ms_avg"], "tflops": ng * unit / (t1["event_ms_avg"] * 1e-3) / 1e12}
    # beside the step: the forward's gate|up GEMMs with the SwiGLU in their epilogue, against the two-launch form
    act = torch.empty(rows * F, dtype=torch.bfloat16, device=dev)
    g_gate = P(probs(Xp, D, None, 0, gp, F, o1))
    g_up = P([(None, act.data_ptr() + off[e] * F * 2, up.data_ptr() + off[e] * F * 4, o3 + e * D * F, (o3 + e * D * F) // group, int(cnt[e]), 0.0)
              for e in range(E)])
    extra = {}
    for name, fn in [] if args.step_only else [("fwd w1,w3 + SwiGLU, one launch", lambda: q.gemm_nn_swiglu(d, s, group, g_gate, g_up, E, D, F, ACT_BF16, FWD, stream)),
                     ("SwiGLU kernel alone", lambda: q.swiglu(gp, up, act, rows * F, ACT_BF16, stream))]:
        extra[name] = {"ms": timed(torch, fn, max(5, args.steps // 2), 2)["event_ms_avg"]}
    flops = 9 * unit
    tf = flops / (tm["event_ms_avg"] * 1e-3) / 1e12
    dom = max(per, key=lambda k: per[k]["ms"]) if per else "not timed"
    return {
        "workload": "%s: E=%d top-%d D=%d F=%d, %d bf16 tokens -> %d expert rows, Zipf(1.1) load (max %d, min %d rows); "
                    "fwd+dgrad+wgrad = 9 grouped GEMMs in %s" % (label, E, topk, D, F, tokens, rows, int(cnt.max()), int(cnt.min()),
                       {"pair": "4 launches (each backward flush -- weight gradient and input gradient of the same operands -- is one grid)",
                        "streams": "6 launches, the weight gradient of each backward flush on a second stream beside its input gradient",
                        "serial": "6 launches"}[args.bwd]),
        "bwd": args.bwd,
        "metric": "QLM expert dequant-GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": tm["wall_ms"],
        "dtype": "bf16" if args.fwd_math == "bf16x2" else "bf16 (fwd: fp16 MFMA)",
        "kernel_ms": tm, "step_ms_spread": spread, "per_launch": per, "beside_the_step": extra, "gflop_per_step": flops / 1e9,
        "roofline": {"bound": "mfma", "achieved": tf, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tf / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": None, "kernel": "k_gemm_nn_h, k_gemm_tn_lds, k_gemm_nt_lds (every launch of the step; slowest on its own: %s)" % dom,
                     "note": "algorithmic flops only; forward math: " + ("bf16 hi+lo weight split, two MFMAs per product" if args.fwd_math == "bf16x2" else
                             "fp16 matrix core, bf16 activations converted exactly, weights rounded once to fp16 (2e-4 relative L2), one MFMA per product")},
    }


# --------------------------------------------------------------------------------------------- layer
def bench_layer(torch, q, args, E=32, D=768, F=2048, tokens=8192, topk=2):
    """One whole MoE expert layer at config 3's shape, forward + backward with the recomputed forward (stash off), router
    outputs given, grouping on the device. Three ways:
      separate  the reference's call order pass by pass (moe_forward / moe_backward, cudalm.cu:4193-4228, 4299-4371),
                every glue step a kernel of its own;
      fused     the same passes with the glue folded into the GEMMs (gather -> w1|w3 -> SwiGLU, w2 -> gated scatter,
                dgrad w2 -> SwiGLU gradient, paired dgrad -> scatter-add);
      merged    all K passes as one expert-grouped list of K*N rows (the reference's merged top-K, cudalm.cu:3532-3561,
                4048-4110): every GEMM once per layer, the passes combined per token in pass order, glue folded in
                where one launch may still name a token once.
    What stays a kernel of its own when fused: the token matrix to bf16 once, the gather that feeds the weight gradient,
    the gate gradient and (merged) the two combines."""
    import numpy as np
    from cudalm_c_amd.binding import ACT_BF16, MATH_MFMA, MATH_MFMA_F16
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev); g.manual_seed(0)
    N, K, group = tokens, topk, 128
    nw = E * D * F
    stream = torch.cuda.current_stream().cuda_stream

    def packed():
        b = torch.randint(0, 256, (nw // 2,), dtype=torch.int16, device=dev, generator=g).to(torch.uint8)
        lo = b & 15; hi = b >> 4
        lo = torch.where(lo == 8, torch.zeros_like(lo), lo); hi = torch.where(hi == 8, torch.zeros_like(hi), hi)
        return (lo | (hi << 4)).view(torch.int8)
    d = torch.cat([packed(), packed(), packed()])
    s = (0.02 * 3 / 7) * (0.5 + torch.rand(3 * nw // group, device=dev, generator=g))
    # Zipf(1.1) routing without replacement, pass-major assignment, gates U(0.1, 0.6)
    logp = -1.1 * np.log(np.arange(E) + 1.0)
    keys = logp[None, :] + np.random.default_rng(0).gumbel(size=(N, E))
    top = np.argsort(-keys, axis=1)[:, :K]
    assign = torch.from_numpy(np.ascontiguousarray(top.T).astype(np.int32).reshape(-1)).to(dev)
    gate = 0.1 + 0.5 * torch.rand(K * N, device=dev, generator=g)
    x = torch.randn(N * D, device=dev, generator=g).to(torch.bfloat16).float()
    dout = torch.randn(N * D, device=dev, generator=g).to(torch.bfloat16).float()
    bf = torch.bfloat16
    KN = K * N
    xb = torch.empty(N * D, dtype=bf, device=dev)
    Xp, ap = torch.empty(KN * D, dtype=bf, device=dev), torch.empty(KN * F, dtype=bf, device=dev)
    gp, up, yp = torch.empty(KN * F, device=dev), torch.empty(KN * F, device=dev), torch.empty(KN * D, device=dev)
    dyp, dgp, dup = torch.empty(KN * D, dtype=bf, device=dev), torch.empty(KN * F, dtype=bf, device=dev), torch.empty(KN * F, dtype=bf, device=dev)
    dap, dXp = torch.empty(KN * F, device=dev), torch.empty(KN * D, device=dev)
    out, dx, dgate = torch.zeros(N * D, device=dev), torch.zeros(N * D, device=dev), torch.zeros(KN, device=dev)
    G = torch.zeros(3 * nw, device=dev)
    ident = torch.arange(N, dtype=torch.int32, device=dev)
    P = q.problems

    class Lists:
        """the grouped lists of one way of running the layer: K lists of N rows, or one of K*N"""
        def __init__(self, merged):
            self.R, self.n = (KN, 1) if merged else (N, K)
            self.perm = torch.empty(KN, dtype=torch.int32, device=dev); self.off = torch.empty(self.n * (E + 1), dtype=torch.int32, device=dev)
            ws = torch.empty(q.moe_perm_workspace(self.R, E, self.n), dtype=torch.uint8, device=dev)
            q.moe_perm(assign, self.R, E, self.n, self.perm, self.off, ws, stream)
            self.offh = self.off.cpu().numpy().reshape(self.n, E + 1)
            self.tok, self.inv = self.perm, None
            if merged:
                self.tok, self.inv = torch.empty(KN, dtype=torch.int32, device=dev), torch.empty(KN, dtype=torch.int32, device=dev)
                q.moe_merge_rows(self.perm, N, K, self.tok, self.inv, stream)
            self.T = [self.tables(k) for k in range(self.n)]

        def probs(self, k, A, a_cols, C, c_cols, wbase, B=None, b_cols=0, beta=0.0, out_expert=False, idx_a=False, idx_c=False):
            o = self.offh[k]; items = []
            for e in range(E):
                ne, oe = int(o[e + 1] - o[e]), int(o[e])
                a = self.tok.data_ptr() + (k * self.R + oe) * 4 if idx_a else A.data_ptr() + oe * a_cols * 2
                b = None if B is None else B.data_ptr() + oe * b_cols * 2
                if idx_c:       c = self.tok.data_ptr() + (k * self.R + oe) * 4
                elif C is None: c = None
                else:           c = C.data_ptr() + ((wbase + e * D * F) * 4 if out_expert else oe * c_cols * 4)
                items.append((a, b, c, wbase + e * D * F, (wbase + e * D * F) // group, ne, beta))
            return items

        def tables(self, k):
            pr = self.probs
            return dict(
                w13=P(pr(k, Xp, D, gp, F, 0) + pr(k, Xp, D, up, F, nw)),
                w1=P(pr(k, Xp, D, gp, F, 0)), w3=P(pr(k, Xp, D, up, F, nw, B=ap, b_cols=F)),
                w1g=P(pr(k, None, 0, None, F, 0, idx_a=True)), w3o=P(pr(k, Xp, D, None, F, nw, B=ap, b_cols=F)),
                w2=P(pr(k, ap, F, yp, D, 2 * nw)), w2s=P(pr(k, ap, F, None, 0, 2 * nw, idx_c=True)),
                g2=P(pr(k, ap, F, G, 0, 2 * nw, B=dyp, b_cols=D, beta=1.0, out_expert=True)),
                d2=P(pr(k, dyp, D, dap, F, 2 * nw)), d2s=P(pr(k, dyp, D, gp, F, 2 * nw)),
                g13=P(pr(k, Xp, D, G, 0, 0, B=dgp, b_cols=F, beta=1.0, out_expert=True) + pr(k, Xp, D, G, 0, nw, B=dup, b_cols=F, beta=1.0, out_expert=True)),
                d1=P(pr(k, dgp, F, dXp, D, 0)), d3=P(pr(k, dup, F, dXp, D, nw)),
                d1s=P(pr(k, dgp, F, None, 0, 0, idx_c=True)), d3s=P(pr(k, dup, F, None, 0, nw, idx_c=True)))

    def layer(L, fused, merged):
        R = L.R
        if fused: q.moe_gather(x, ident, xb, N, D, ACT_BF16, stream)               # the token matrix as bf16, once per layer
        for k in range(L.n):                                                          # forward
            T, tok, gk = L.T[k], L.tok[k * R:(k + 1) * R], gate[k * N:(k + 1) * N]
            if fused: q.gemm_nn_gather_swiglu(d, s, group, T["w1g"], T["w3o"], E, D, F, xb, stream)
            else:
                q.moe_gather(x, tok, Xp, R, D, ACT_BF16, stream)
                q.gemm_nn(d, s, group, T["w13"], 2 * E, D, F, ACT_BF16, MATH_MFMA_F16, stream)
                q.swiglu(gp, up, ap, R * F, ACT_BF16, stream)
            if merged:
                q.gemm_nn(d, s, group, T["w2"], E, F, D, ACT_BF16, MATH_MFMA_F16, stream)
                q.moe_combine(yp, L.inv, gate, out, N, K, D, stream)
            elif fused: q.gemm_nn_scatter(d, s, group, T["w2s"], E, F, D, out, gk, stream)
            else:
                q.gemm_nn(d, s, group, T["w2"], E, F, D, ACT_BF16, MATH_MFMA_F16, stream)
                q.moe_scatter_gate(yp, tok, gk, out, N, D, stream)
        for k in range(L.n):                                                          # backward
            T, tok, gk = L.T[k], L.tok[k * R:(k + 1) * R], gate[k * N:(k + 1) * N]
            q.moe_gather(x, tok, Xp, R, D, ACT_BF16, stream)                          # the weight gradient reads the grouped rows
            if fused: q.gemm_nn_swiglu(d, s, group, T["w1"], T["w3"], E, D, F, ACT_BF16, MATH_MFMA_F16, stream)
            else:
                q.gemm_nn(d, s, group, T["w13"], 2 * E, D, F, ACT_BF16, MATH_MFMA_F16, stream)
                q.swiglu(gp, up, ap, R * F, ACT_BF16, stream)
            q.gemm_nn(d, s, group, T["w2"], E, F, D, ACT_BF16, MATH_MFMA_F16, stream)
            if merged: q.moe_dgate_merged(dout, yp, L.perm, gate, dgate, dyp, N, K, D, ACT_BF16, stream)
            else:      q.moe_dgate(dout, yp, tok, gk, dgate[k * N:(k + 1) * N], dyp, N, D, ACT_BF16, stream)
            # each backward flush (weight gradient + input gradient of the same operands) is one grid
            q.pair_begin(stream)
            q.gemm_nt(T["g2"], E, F, D, ACT_BF16, MATH_MFMA, stream)
            if fused: q.gemm_tn_swiglu_bwd(d, s, group, T["d2s"], E, D, F, gp, up, dgp, dup, stream)
            else:     q.gemm_tn(d, s, group, T["d2"], E, D, F, ACT_BF16, MATH_MFMA, stream)
            q.pair_end(stream)
            if not fused: q.swiglu_bwd(gp, up, dap, dgp, dup, R * F, ACT_BF16, stream)
            q.pair_begin(stream)
            q.gemm_nt(T["g13"], 2 * E, D, F, ACT_BF16, MATH_MFMA, stream)
            if fused and not merged: q.gemm_tn_pair_scatter(d, s, group, T["d1s"], T["d3s"], E, F, D, dx, stream)
            else:                    q.gemm_tn_pair(d, s, group, T["d1"], T["d3"], E, F, D, ACT_BF16, MATH_MFMA, stream)
            q.pair_end(stream)
            if merged:      q.moe_combine(dXp, L.inv, None, dx, N, K, D, stream)
            elif not fused: q.moe_scatter_add(dXp, tok, dx, N, D, stream)

    steps, warmup = max(5, args.steps // 4), max(2, args.warmup // 4)
    per_pass, one_list = Lists(False), Lists(True)
    nil = {"event_ms_avg": None}
    t_sep = nil if args.step_only else timed(torch, lambda: layer(per_pass, False, False), steps, warmup)
    t_fus = nil if args.step_only else timed(torch, lambda: layer(per_pass, True, False), steps, warmup)
    t_mrg = timed(torch, lambda: layer(one_list, True, True), steps, warmup)
    spread = step_spread(torch, lambda: layer(one_list, True, True), steps)

    def glue_only():
        """the kernels of the merged layer that are not GEMMs: token matrix to bf16, the gather for the weight gradient,
        the gate gradient, the two combines"""
        L = one_list
        q.moe_gather(x, ident, xb, N, D, ACT_BF16, stream)
        q.moe_combine(yp, L.inv, gate, out, N, K, D, stream)
        q.moe_gather(x, L.tok, Xp, L.R, D, ACT_BF16, stream)
        q.moe_dgate_merged(dout, yp, L.perm, gate, dgate, dyp, N, K, D, ACT_BF16, stream)
        q.moe_combine(dXp, L.inv, None, dx, N, K, D, stream)
    t_glue = nil if args.step_only else timed(torch, glue_only, steps, warmup)
    flops = K * 12 * 2.0 * N * D * F                       # per pass: 3 forward GEMMs, 3 recomputed in the backward, 3 dgrad, 3 wgrad
    tf = flops / (t_mrg["event_ms_avg"] * 1e-3) / 1e12
    return {"workload": "C3 whole expert layer, forward + backward with the recomputed forward (%d tokens top-%d, E=%d D=%d F=%d): GEMMs and glue" % (N, K, E, D, F),
            "metric": "layer TFLOP/s (12 GEMMs per token and pass incl. the recomputed forward; all passes as one grouped list, glue folded in)",
            "value": tf, "unit": "TFLOP/s", "ms_per_step": t_mrg["wall_ms"], "dtype": "bf16 (fwd: fp16 MFMA)", "steps": steps, "warmup": warmup,
            "gflop_per_step": flops / 1e9, "step_ms_spread": spread,
            "glue_ms": {"the five kernels of the merged layer that are not GEMMs, timed on their own": t_glue["event_ms_avg"]},
            "layer_ms": {"pass by pass, glue as separate kernels": t_sep["event_ms_avg"], "pass by pass, glue folded into the GEMMs": t_fus["event_ms_avg"],
                         "all passes as one list, glue folded in": t_mrg["event_ms_avg"]},
            "roofline": {"bound": "mfma", "achieved": tf, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tf / MFMA_BF16_PEAK_TFLOPS, "traffic": None,
                         "kernel": "whole layer: 8 grouped GEMM launches (k_gemm_nn_h, k_gemm_nn_h_swiglu, k_gemm_tn_lds, k_gemm_nt_lds) + 5 glue kernels",
                         "note": "algorithmic flops only (12 GEMMs per token and pass, the recomputed forward included); glue time is inside the step"}}


# --------------------------------------------------------------------------------------------- c5
def bench_c5(torch, q, args, L=8, E=64, D=2048, F=1408, tokens=32768, topk=4):
    """Config 5 whole: 8 layers x (E=64, top-4, D=2048, F=1408), 131072 expert rows per layer with Zipf(1.1) loads
    (a different draw per layer): every layer's 9 expert GEMMs in the order of moe_forward / moe_backward
    (cudalm.cu:4211-4225, 4333-4366) over that layer's own 553.6 M packed weights, the weight gradients written
    into one fp32 G of 4.43 G elements; then one Integer AdamW step (cudalm.cu:6082-6103) over all 4.43 G weights.
    A step of this workload is heavy (about 0.1 s), so it is timed over max(3, K // 10) steps after max(1, W // 10)
    warm-up steps; both figures are in the result."""
    import numpy as np
    from cudalm_c_amd.binding import ACT_BF16, MATH_MFMA, MATH_MFMA_F16, SPAN_DTYPE
    FWD = MATH_MFMA if args.fwd_math == "bf16x2" else MATH_MFMA_F16
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev); g.manual_seed(0)
    group = 128
    EDF = E * D * F
    nlayer = 3 * EDF
    nq = L * nlayer
    ng = nq // group
    rows = tokens * topk
    steps, warmup = max(3, args.steps // 10), max(1, args.warmup // 10)

    def chunks(n, fn, dtype):
        out = torch.empty(n, dtype=dtype, device=dev)
        for i in range(0, n, 1 << 30):
            m = min(1 << 30, n - i)
            out[i:i + m] = fn(m)
        return out

    def packed(m):
        b = torch.randint(0, 256, (m,), dtype=torch.int16, device=dev, generator=g).to(torch.uint8)
        lo = b & 15; hi = b >> 4
        lo = torch.where(lo == 8, torch.zeros_like(lo), lo); hi = torch.where(hi == 8, torch.zeros_like(hi), hi)
        return (lo | (hi << 4)).view(torch.int8)

    d = chunks(nq // 2, packed, torch.int8)
    s = (0.02 * 3 / 7) * (0.5 + torch.rand(ng, device=dev, generator=g))
    G = torch.zeros(nq, device=dev)

    def bf16(n):
        return torch.randn(n, device=dev, generator=g).to(torch.bfloat16)

    Xp, ap, dyp, dgp, dup = bf16(rows * D), bf16(rows * F), bf16(rows * D), bf16(rows * F), bf16(rows * F)
    gp = torch.empty(rows * F, device=dev); up = torch.empty(rows * F, device=dev); yp = torch.empty(rows * D, device=dev)
    dap = torch.empty(rows * F, device=dev); dXp = torch.empty(rows * D, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    P = q.problems
    calls = []
    loads = []
    for l in range(L):
        cnt = zipf_counts(E, tokens, topk, seed=100 + l)
        loads.append((int(cnt.max()), int(cnt.min())))
        off = np.concatenate([[0], np.cumsum(cnt)]).astype(int)
        o1, o3, o2 = l * nlayer, l * nlayer + EDF, l * nlayer + 2 * EDF

        def items(A, a_w, B, b_w, Cm, c_w, wbase, per_expert_c=False, beta=0.0):
            return [(A.data_ptr() + int(off[e]) * a_w * 2, (B.data_ptr() + int(off[e]) * b_w * 2) if B is not None else None,
                     (Cm.data_ptr() + (wbase + e * D * F) * 4) if per_expert_c else (Cm.data_ptr() + int(off[e]) * c_w * 4),
                     wbase + e * D * F, (wbase + e * D * F) // group, int(cnt[e]), beta) for e in range(E)]

        p_w13 = P(items(Xp, D, None, 0, gp, F, o1) + items(Xp, D, None, 0, up, F, o3))
        p_w2 = P(items(ap, F, None, 0, yp, D, o2))
        p_g2 = P(items(ap, F, dyp, D, G, 0, o2, True))
        p_d2 = P(items(dyp, D, None, 0, dap, F, o2))
        p_g13 = P(items(Xp, D, dgp, F, G, 0, o1, True) + items(Xp, D, dup, F, G, 0, o3, True))
        p_d1 = P(items(dgp, F, None, 0, dXp, D, o1)); p_d3 = P(items(dup, F, None, 0, dXp, D, o3, beta=1.0))
        calls.append(lambda st, p_w13=p_w13, p_w2=p_w2, p_g2=p_g2, p_d2=p_d2, p_g13=p_g13, p_d1=p_d1, p_d3=p_d3: [
            (lambda: q.gemm_nn(d, s, group, p_w13, 2 * E, D, F, ACT_BF16, FWD, st)),
            (lambda: q.gemm_nn(d, s, group, p_w2, E, F, D, ACT_BF16, FWD, st)),
            (lambda: q.gemm_nt(p_g2, E, F, D, ACT_BF16, MATH_MFMA, st)),
            (lambda: q.gemm_tn(d, s, group, p_d2, E, D, F, ACT_BF16, MATH_MFMA, st)),
            (lambda: q.gemm_nt(p_g13, 2 * E, D, F, ACT_BF16, MATH_MFMA, st)),
            (lambda: q.gemm_tn_pair(d, s, group, p_d1, p_d3, E, F, D, ACT_BF16, MATH_MFMA, st)),
        ])
    main_calls = [mk(stream) for mk in calls]
    if args.bwd == "streams":
        side_st = q.side_fork(stream); q.side_join(stream)       # the handle is the same at every fork
        side_calls = [mk(side_st) for mk in calls]

        def gemms():
            # each backward flush with its weight gradient on the library's side stream beside its input gradient
            for m, sd in zip(main_calls, side_calls):
                m[0](); m[1]()
                q.side_fork(stream); sd[2](); m[3](); q.side_join(stream)
                q.side_fork(stream); sd[4](); m[5](); q.side_join(stream)
    elif args.bwd == "pair":
        def gemms():
            for m in main_calls:
                m[0](); m[1]()
                q.pair_begin(stream); m[2](); m[3](); q.pair_end(stream)
                q.pair_begin(stream); m[4](); m[5](); q.pair_end(stream)
    else:
        def gemms():
            for m in main_calls:
                for fn in m:
                    fn()

    tg = timed(torch, gemms, steps, warmup)
    flops = L * 9 * 2.0 * rows * D * F
    tf = flops / (tg["event_ms_avg"] * 1e-3) / 1e12
    del Xp, ap, dyp, dgp, dup, gp, up, yp, dap, dXp

    # ---- the optimizer step over every weight of the stack ----
    def ri(lo, hi, dtype):
        return lambda m: torch.randint(lo, hi, (m,), dtype=torch.int16, device=dev, generator=g).to(dtype)
    r = chunks(nq, ri(-64, 65, torch.int8), torch.int8)
    m8 = chunks(nq, ri(-127, 128, torch.int8), torch.int8)
    v8 = chunks(nq, ri(0, 256, torch.uint8), torch.uint8)
    m8s = (3e-3 / 127) * (0.5 + torch.rand(ng, device=dev, generator=g))
    v8s = (3e-3 / 255) * (0.5 + torch.rand(ng, device=dev, generator=g))
    tab = np.zeros(3 * L, dtype=SPAN_DTYPE)
    smean = float(s.mean())
    for i in range(3 * L):
        tab[i] = (i * EDF, i * EDF, i * EDF, EDF, i * (EDF // group), EDF // group, smean, 0)
    sp = torch.from_numpy(tab.view(np.uint8)).to(dev)
    gscale = 1e-3 / max(float(G[:1 << 24].std()), 1e-20)      # the weight gradients just computed, brought to the ~1e-3 scale the config names
    state = {"t": 0}
    b1, b2 = 0.9, 0.95

    def step():
        state["t"] += 1
        t = state["t"]
        q.step(None, G, d, r, s, m8, m8s, v8, v8s, sp, 3 * L, group, 7, 3e-4, b1, b2, 0.1, gscale, None,
               1.0 / (1.0 - b1 ** t), 1.0 / (1.0 - b2 ** t) ** 0.5, 0, t, 1, None, 1, 0, ng, 0, stream)

    ta = timed(torch, step, steps, warmup)
    bytes_per_w = 11.0 + 20.0 / 128
    gbs = nq * bytes_per_w / (ta["event_ms_avg"] * 1e-3) / 1e9
    return {
        "workload": "C5 whole stack: %d layers x (E=%d top-%d D=%d F=%d), %d bf16 tokens -> %d expert rows per layer, Zipf(1.1) load per layer "
                    "(max/min rows %s); fwd+dgrad+wgrad = %d grouped GEMMs in %d launches, then one Integer AdamW step over %d weights"
                    % (L, E, topk, D, F, tokens, rows, "/".join("%d:%d" % x for x in loads[:2]) + "...", 9 * L, (4 if args.bwd == "pair" else 6) * L, nq),
        "bwd": args.bwd,
        "metric": "QLM expert dequant-GEMM TFLOP/s", "value": tf, "unit": "TFLOP/s", "ms_per_step": tg["wall_ms"] + ta["wall_ms"],
        "dtype": "bf16" if args.fwd_math == "bf16x2" else "bf16 (fwd: fp16 MFMA)",
        "steps": steps, "warmup": warmup,
        "gemm": {"ms": tg["event_ms_avg"], "tflops": tf, "tflop_per_step": flops / 1e12},
        "adamw": {"ms": ta["event_ms_avg"], "gbs": gbs, "weights": nq, "weights_per_s": nq / (ta["event_ms_avg"] * 1e-3), "bytes_per_weight": bytes_per_w},
        "roofline": {"bound": "mfma", "achieved": tf, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tf / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": None, "kernel": "k_gemm_nn_h, k_gemm_tn_lds, k_gemm_nt_lds (all %d launches)" % ((4 if args.bwd == "pair" else 6) * L),
                     "note": "the device holds 1.33-1.39 GHz under this load (profiles/k_gemm_lds_train_c5.txt); the peak is that of 2.4 GHz"},
        "roofline_adamw": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": None,
                           "kernel": "k_qlmx_step<adam>, one launch over all %d weights" % nq},
    }


# --------------------------------------------------------------------------------------------- decode
def bench_decode(torch, q, args, E=32, D=768, F=2048, topk=2, layers=8):
    """8 distinct layers (8 x 80 MB of packed weights > the 256 MB last-level cache) decoded back to
    back for T = 1, 4, 16 tokens; bytes counted = digits + scales of the distinct experts hit."""
    import numpy as np
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev); g.manual_seed(0)
    group = 128
    nw = E * D * F
    per_expert = 3 * D * F // 2 + 3 * D * F // group * 4

    def packed(n):
        b = torch.randint(0, 256, (n // 2,), dtype=torch.int16, device=dev, generator=g).to(torch.uint8)
        lo = b & 15; hi = b >> 4
        lo = torch.where(lo == 8, torch.zeros_like(lo), lo); hi = torch.where(hi == 8, torch.zeros_like(hi), hi)
        return (lo | (hi << 4)).view(torch.int8)

    ds = [packed(3 * nw) for _ in range(layers)]
    ss = [(0.02 * 3 / 7) * (0.5 + torch.rand(3 * nw // group, device=dev, generator=g)) for _ in range(layers)]
    stream = torch.cuda.current_stream().cuda_stream
    out_all = {}
    for T in (1, 4, 16):
        x = torch.randn(T * D, device=dev, generator=g)
        asn, gates, hits = [], [], 0
        for l in range(layers):
            logits = torch.randn(T, E, device=dev, generator=g)
            p = torch.softmax(logits, dim=1)
            top = torch.topk(p, topk, dim=1)
            a = top.indices.t().contiguous().to(torch.int32)          # pass-major [K][T]
            asn.append(a.view(-1)); gates.append(top.values.t().contiguous().view(-1))
            hits += int(torch.unique(a).numel())
        out = torch.zeros(T * D, device=dev)

        def step():
            for l in range(layers):
                q.decode_forward(x, asn[l], gates[l], out, ds[l], ss[l], group, 0, nw, 2 * nw, T, topk, E, D, F, stream)

        tm = timed(torch, step, args.steps, args.warmup)
        res = {"ms_8_layers": tm["event_ms_avg"], "distinct_expert_hits": hits, "bytes": hits * per_expert,
               "gbs": hits * per_expert / (tm["event_ms_avg"] * 1e-3) / 1e9}
        # beside it: the same sequence with the layer's inputs taken as fp16 pairs (qlmx_decode_math(1); 3.7e-4
        # against the fp32 reference instead of 4e-7); the figures of the line are the default fp32 loop's
        q.call("qlmx_decode_math", 1)
        try:
            th = timed(torch, step, args.steps, args.warmup)
            res["fp16_inputs_ms_8_layers"] = th["event_ms_avg"]
        finally:
            q.call("qlmx_decode_math", 0)
        # the same 8-layer sequence replayed as one HIP graph (no launch gaps from the host)
        try:
            gr = torch.cuda.CUDAGraph()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                st2 = side.cuda_stream
                for l in range(layers):
                    q.decode_forward(x, asn[l], gates[l], out, ds[l], ss[l], group, 0, nw, 2 * nw, T, topk, E, D, F, st2)
                side.synchronize()
                with torch.cuda.graph(gr, stream=side):
                    for l in range(layers):
                        q.decode_forward(x, asn[l], gates[l], out, ds[l], ss[l], group, 0, nw, 2 * nw, T, topk, E, D, F, st2)
            torch.cuda.current_stream().wait_stream(side)
            tg = timed(torch, gr.replay, args.steps, args.warmup)
            res["graph_ms_8_layers"] = tg["event_ms_avg"]
            res["graph_gbs"] = hits * per_expert / (tg["event_ms_avg"] * 1e-3) / 1e9
        except Exception as e:      # graph capture is an extra; the eager figure stands on its own
            res["graph_error"] = str(e)[:200]
        out_all["T%d" % T] = res
    head = out_all["T16"]
    gbs = max(head["gbs"], head.get("graph_gbs", 0.0))
    return {
        "workload": "C2 decode: %d layers x (E=%d top-%d D=%d F=%d), T=16 tokens per step (T=1,4 listed beside); one launch per layer: grouping, w1|w3, SwiGLU, w2, gated combine"
                    % (layers, E, topk, D, F),
        "metric": "QLM expert dequant-GEMV GB/s", "value": gbs, "unit": "GB/s", "ms_per_step": min(head["ms_8_layers"], head.get("graph_ms_8_layers", 1e9)),
        "dtype": "u8+f32", "by_tokens": out_all, "bytes_per_expert_hit": per_expert,
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": None,
                     "kernel": "k_decode_fused (one launch per layer; figure is the whole 8-layer sequence)"},
    }

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
                     "traffic": None, "kernel": "k_qlmx_step_wide (Adam, eight groups per wavefront)", "bytes_per_weight": bytes_per_w},
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
    while t_used < 10.0 and reps < 5000:
        t0 = time.perf_counter()
        lib.step(P, G, d, r, s, m8, m8s, v8, v8s, tab, 128, 7, 3e-4, 0.9, 0.95, 0.1, 1.0, None, 10.0, 4.47, 0, 2 + reps, 1, None, 1, 0, ng)
        t_used += time.perf_counter() - t0
        reps += 1
    gbs = nq * 15.16 * reps / t_used / 1e9
    return {"value": gbs, "unit": "GB/s", "cores": threads, "cpu": cpu_model(), "kind": kind,
            "sample": "Integer AdamW (P rendered, 15.16 B/weight) over %d weights x %d steps, %s" % (nq, reps, "cpu_kern.h cpu_qlm_step" if kind == "reference" else "oracle/qlm_oracle.c"),
            "weights_per_s": nq * reps / t_used}


# --------------------------------------------------------------------------------------- codec, glue
def _stream_result(name, kernel, entries, note):
    """entries: list of (label, algorithmic bytes per launch, timing). The reported value is the slowest-rated entry's GB/s."""
    per = {lab: {"ms": tm["event_ms_avg"], "bytes": b, "gbs": b / (tm["event_ms_avg"] * 1e-3) / 1e9} for lab, b, tm in entries}
    tot_b = sum(b for _, b, _ in entries); tot_ms = sum(tm["event_ms_avg"] for _, _, tm in entries)
    gbs = tot_b / (tot_ms * 1e-3) / 1e9
    return {"workload": name, "metric": "streaming GB/s (algorithmic bytes of all listed launches / their summed time)", "value": gbs,
            "unit": "GB/s", "ms_per_step": tot_ms, "dtype": "u8+f32", "per_launch": per,
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                         "traffic": None, "kernel": kernel, "note": note}}


def bench_codec(torch, q, args):
    """Encode, render and servo over one span of the AdamW sweep's size (init / resume / every 100th step)."""
    import numpy as np
    from cudalm_c_amd.binding import SPAN_DTYPE
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev); g.manual_seed(0)
    nq = (args.adamw_weights // 128) * 128
    ng = nq // 128
    P = 0.02 * torch.randn(nq, device=dev, generator=g)
    d = torch.zeros(nq // 2, dtype=torch.int8, device=dev); r = torch.zeros(nq, dtype=torch.int8, device=dev)
    s = torch.zeros(ng, device=dev)
    tab = np.zeros(1, dtype=SPAN_DTYPE)
    tab[0] = (0, 0, 0, nq, 0, ng, 0.0, 0)
    sp = torch.from_numpy(tab.view(np.uint8)).to(dev)
    stream = torch.cuda.current_stream().cuda_stream
    te = timed(torch, lambda: q.encode(P, d, r, s, sp, 1, 128, 7, 1, ng, stream), args.steps, args.warmup)
    tr = timed(torch, lambda: q.render(P, d, s, sp, 1, 128, 1, 0, ng, stream), args.steps, args.warmup)
    # servo thresholds that leave the scales alone (the usual case) and ones that rescale every group
    ts0 = timed(torch, lambda: q.servo(d, r, s, sp, 1, 128, 7, 2.0, -1.0, 1, ng, stream), args.steps, args.warmup)
    state = {"k": 0}

    def servo_all():
        state["k"] ^= 1          # up, down, up, ...: the scales stay in range over any number of calls
        q.servo(d, r, s, sp, 1, 128, 7, (-1.0 if state["k"] else 2.0), (-1.0 if state["k"] else 2.0), 1, ng, stream)
    ts1 = timed(torch, servo_all, args.steps, args.warmup)
    gb = 4.0 / 128
    return _stream_result(
        "encode / render / servo over %d weights, group 128, 4-bit packed" % nq, "k_qlmx_encode, k_qlmx_render, k_qlmx_servo",
        [("encode", nq * (4 + 0.5 + 1 + gb), te), ("render", nq * (0.5 + gb + 4), tr),
         ("servo, no group rescaled", nq * (0.5 + gb), ts0), ("servo, every group rescaled", nq * (2 * 0.5 + 2 * 1 + 2 * gb), ts1)],
        "bytes per weight: encode 4 read + 1.5 written, render 0.5 + 4, servo 0.5 read (+ 1 read + 1.5 written where a group is rescaled)")


def bench_glue(torch, q, args, E=32, D=768, F=2048, tokens=8192, topk=2):
    """The MoE glue kernels at the training layer's shape, each timed on its own."""
    from cudalm_c_amd.binding import ACT_BF16
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev); g.manual_seed(0)
    N, K = tokens, topk
    stream = torch.cuda.current_stream().cuda_stream
    rt = torch.randn(N * E, device=dev, generator=g)
    rprobs = torch.empty(N * E, device=dev); assign = torch.empty(K * N, dtype=torch.int32, device=dev); gate = torch.empty(K * N, device=dev)
    perm = torch.empty(K * N, dtype=torch.int32, device=dev); off = torch.empty(K * (E + 1), dtype=torch.int32, device=dev)
    ws = torch.empty(q.moe_perm_workspace(N, E, K), dtype=torch.uint8, device=dev)
    x = torch.randn(N * D, device=dev, generator=g)
    Xp = torch.empty(N * D, dtype=torch.bfloat16, device=dev)
    gp = torch.randn(N * F, device=dev, generator=g); up = torch.randn(N * F, device=dev, generator=g)
    act = torch.empty(N * F, dtype=torch.bfloat16, device=dev)
    dact = torch.randn(N * F, device=dev, generator=g)
    dg = torch.empty(N * F, dtype=torch.bfloat16, device=dev); du = torch.empty(N * F, dtype=torch.bfloat16, device=dev)
    yp = torch.randn(N * D, device=dev, generator=g); out = torch.zeros(N * D, device=dev)
    dout = torch.randn(N * D, device=dev, generator=g); dgate = torch.empty(N, device=dev)
    dyp = torch.empty(N * D, dtype=torch.bfloat16, device=dev); dx = torch.zeros(N * D, device=dev)
    q.router_topk(rt, rprobs, assign, gate, N, E, K, None, 0, stream)
    q.moe_perm(assign, N, E, K, perm, off, ws, stream)
    T = lambda fn: timed(torch, fn, args.steps, args.warmup)
    ent = [
        ("router_topk", N * E * 8 + K * N * 8, T(lambda: q.router_topk(rt, rprobs, assign, gate, N, E, K, None, 0, stream))),
        ("moe_perm (both passes)", K * N * 8, T(lambda: q.moe_perm(assign, N, E, K, perm, off, ws, stream))),
        ("gather -> bf16 (one pass)", N * D * 6 + N * 4, T(lambda: q.moe_gather(x, perm, Xp, N, D, ACT_BF16, stream))),
        ("swiglu -> bf16 (one pass)", N * F * 10, T(lambda: q.swiglu(gp, up, act, N * F, ACT_BF16, stream))),
        ("scatter_gate (one pass)", N * D * 12 + N * 8, T(lambda: q.moe_scatter_gate(yp, perm, gate, out, N, D, stream))),
        ("dgate -> bf16 (one pass)", N * D * 10 + N * 12, T(lambda: q.moe_dgate(dout, yp, perm, gate, dgate, dyp, N, D, ACT_BF16, stream))),
        ("swiglu_bwd -> bf16 (one pass)", N * F * 16, T(lambda: q.swiglu_bwd(gp, up, dact, dg, du, N * F, ACT_BF16, stream))),
        ("scatter_add (one pass)", N * D * 12 + N * 4, T(lambda: q.moe_scatter_add(yp, perm, dx, N, D, stream))),
    ]
    return _stream_result("MoE glue at E=%d top-%d D=%d F=%d, %d tokens (per pass of %d rows)" % (E, K, D, F, N, N),
                          "qlmx_glue.hip kernels", ent,
                          "bytes: every operand read once and every output written once (scatter kernels read-modify-write their destination)")


def bench_copy(torch, q, args):
    """Plain 1 GiB device copy: the known-size kernel that calibrates the FETCH_SIZE / WRITE_SIZE counters."""
    n = 2 ** 28
    a = torch.randn(n, device="cuda:0"); b = torch.empty_like(a)
    tm = timed(torch, lambda: b.copy_(a), args.steps, args.warmup)
    gbs = 2 * n * 4 / (tm["event_ms_avg"] * 1e-3) / 1e9
    return {"workload": "calibration: torch copy of 1 GiB (1 GiB read + 1 GiB written per launch)", "metric": "copy GB/s", "value": gbs,
            "unit": "GB/s", "ms_per_step": tm["wall_ms"], "dtype": "f32",
            "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS, "traffic": None,
                         "kernel": "at::native elementwise copy"}}


def cpu_gemm(args):
    """Reference CPU expert GEMMs (cpu_rt.h packed SGEMM through g_ab / g_abt_b / g_atb on a rendered fp32
    view) on a bounded sample: one expert's forward, input-gradient and weight-gradient GEMM at the layer's
    D=768, F=2048 with 2048 rows, repeated for about 10 s."""
    import numpy as np
    from oracle.binding import Oracle, Ref, have_ref
    orc = Oracle()
    threads = min(16, os.cpu_count() or 1)
    kind = "reference" if have_ref() else "port"
    lib = Ref(threads=threads) if kind == "reference" else orc
    orc.set_threads(threads)
    M, D, F = 2048, 768, 2048
    X = orc.normal(M * D, 0, 1); W = orc.normal(D * F, 0, 2, 0.02); dY = orc.normal(M * F, 0, 3)
    Y = np.zeros(M * F, np.float32); dX = np.zeros(M * D, np.float32); G = np.zeros(D * F, np.float32)
    lib.gemm_nn(X, W, Y, M, D, F)
    reps, t_used = 0, 0.0
    while t_used < 12.0 and reps < 5000:
        t0 = time.perf_counter()
        lib.gemm_nn(X, W, Y, M, D, F)
        lib.gemm_tn(dY, W, dX, M, F, D, 0.0)
        lib.gemm_nt(X, dY, G, M, D, F)
        t_used += time.perf_counter() - t0
        reps += 1
    tf = 3 * 2.0 * M * D * F * reps / t_used / 1e12
    return {"value": tf, "unit": "TFLOP/s", "cores": threads, "cpu": cpu_model(), "kind": kind,
            "sample": "one expert, %d rows, D=%d F=%d: fwd + dgrad + wgrad fp32 SGEMM on the rendered view, %d repetitions (%s)"
                      % (M, D, F, reps, "cpu_rt.h sg_core via g_ab/g_abt_b/g_atb" if kind == "reference" else "oracle/qlm_oracle.c")}


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_decode(args, E=32, D=768, F=2048, topk=2, T=16, layers=2):
    """Reference CPU path of the decode shape on a bounded sample: the expert part of moe_forward for T=16 tokens top-2
    (cudalm.cu:4193-4228: per expert hit mg_ab on w1 and w3, flush, SwiGLU, mg_ab on w2, flush; with <= 4 rows per
    expert the reference SGEMM takes its small-R path, cpu_rt.h:233-258) over `layers` distinct layers of rendered
    fp32 weights, cycled for about 10 s. The rate is quoted in the GPU leg's unit -- bytes of PACKED digits and scales
    of the distinct experts hit per second -- although the CPU path reads the 8x larger fp32 view."""
    import numpy as np
    from oracle.binding import Oracle, Ref, have_ref
    orc = Oracle()
    threads = min(16, os.cpu_count() or 1)
    kind = "reference" if have_ref() else "port"
    lib = Ref(threads=threads) if kind == "reference" else orc
    orc.set_threads(threads)
    per_expert = 3 * D * F // 2 + 3 * D * F // 128 * 4
    rng = np.random.default_rng(0)
    W = [[orc.normal(E * D * F, 0, 40 + 3 * l + j, 0.02) for j in range(3)] for l in range(layers)]
    x = orc.normal(T * D, 0, 50)
    plans, hits = [], 0
    for l in range(layers):
        logits = rng.standard_normal((T, E))
        top = np.argsort(-logits, axis=1)[:, :topk]
        plan = []
        for e in np.unique(top):
            toks = np.concatenate([np.nonzero(top[:, k] == e)[0] for k in range(topk)])
            plan.append((int(e), np.ascontiguousarray(x.reshape(T, D)[toks].reshape(-1)), len(toks)))
        hits += len(plan)
        plans.append(plan)
    grouped = kind == "reference"

    def layer(l):
        bufs = []
        for e, xe, m in plans[l]:
            gp = np.zeros(m * F, np.float32); up = np.zeros(m * F, np.float32)
            w1 = W[l][0][e * D * F:(e + 1) * D * F]; w3 = W[l][1][e * D * F:(e + 1) * D * F]
            if grouped:
                lib.gemm_nn(xe, w1, gp, m, D, F, grouped=True); lib.gemm_nn(xe, w3, up, m, D, F, grouped=True)
            else:
                lib.gemm_nn(xe, w1, gp, m, D, F); lib.gemm_nn(xe, w3, up, m, D, F)
            bufs.append((e, m, gp, up))
        if grouped:
            lib.mg_flush()
        outs = []
        for e, m, gp, up in bufs:
            ap = np.zeros(m * F, np.float32); yp = np.zeros(m * D, np.float32)
            lib.swiglu(gp, up, ap)
            w2 = W[l][2][e * D * F:(e + 1) * D * F]
            if grouped:
                lib.gemm_nn(ap, w2, yp, m, F, D, grouped=True)
            else:
                lib.gemm_nn(ap, w2, yp, m, F, D)
            outs.append(yp)
        if grouped:
            lib.mg_flush()
        return outs

    layer(0)
    reps, t_used = 0, 0.0
    while t_used < 10.0 and reps < 100000:
        t0 = time.perf_counter()
        for l in range(layers):
            layer(l)
        t_used += time.perf_counter() - t0
        reps += 1
    gbs = hits * per_expert * reps / t_used / 1e9
    return {"value": gbs, "unit": "GB/s", "cores": threads, "cpu": cpu_model(), "kind": kind,
            "sample": "expert part of moe_forward, T=%d top-%d over %d layers (E=%d D=%d F=%d, %d expert hits), %d repetitions; bytes counted as "
                      "packed digits + scales of the experts hit (the GPU leg's unit; the CPU path reads the fp32 view, 8x that); %s"
                      % (T, topk, layers, E, D, F, hits, reps, "cudalm.cu mg_ab + mg_flush -> cpu_rt.h small-R SGEMM, cpu_kern.h swiglu" if grouped else "oracle/qlm_oracle.c"),
            "ms_per_layer": t_used / reps / layers * 1e3}


# HBM bytes from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by the 1 GiB copy calibration); the runs,
# counter values and scale factors are in profiles/*.txt. adamw: per launch. train: per step, i.e. summed over
# the step's 4 launches (1035.9 MiB read + 1086.2 MiB written). c5: per step over the 32 GEMM launches of the 8
# layers (104.4 GiB read + 49.0 GiB written). decode: per launch = per layer at T=16 (64.1 MiB read + 5.1 MiB
# written). layer: per step of the merged layer, all its kernels (2442.1 MiB read + 1393.2 MiB written). train and c5
# are those of the default --bwd pair. The figures are constants of the code state they
# were measured at; that state is named in the JSON line so that a reader can tell a stale one.
PROFILED_TRAFFIC = {"adamw": 1.405e9, "train": 2.225e9, "layer": 4.022e9, "c5": 1.648e11, "decode": 7.39e7}
PROFILED_AT = "git bd3f2f6 (train, layer, c5), ef06021 (decode), 497f628 (adamw)"


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
    want = ["train", "layer", "decode", "adamw", "c5"] if args.workload == "all" else [args.workload]
    runners = {"adamw": bench_adamw, "train": bench_train, "decode": bench_decode, "copy": bench_copy, "codec": bench_codec, "glue": bench_glue, "c5": bench_c5, "layer": bench_layer,
               "train5": lambda t, qq, a: bench_train(t, qq, a, E=64, D=2048, F=1408, tokens=32768, topk=4, label="C5 train layer (one of 8)")}
    results = {}
    for w in want:
        if w in runners:
            results[w] = runners[w](torch, q, args)
    first = next(results[w] for w in ["train", "train5", "c5", "layer", "decode", "adamw", "codec", "glue", "copy"] if w in results)
    line = {
        "metric": "QLM expert dequant-GEMM TFLOP/s & GB/s (% roofline); int-AdamW GB/s",
        "value": first["value"], "unit": first["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": first["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": first["dtype"], "data": "synthetic", "settle_ms": SETTLE_MS,
        "config": {"workload": first["workload"]},
        "roofline": first["roofline"],
        "workloads": results,
        "device": q.call("qlmx_device_name").decode(),
    }
    for w in results:
        if results[w]["roofline"].get("traffic") is None and PROFILED_TRAFFIC.get(w) and not (w == "adamw" and args.render_p) \
                and not (w in ("train", "c5") and (args.bwd != "pair" or args.fwd_math != "f16")):
            results[w]["roofline"]["traffic"] = PROFILED_TRAFFIC[w]
            results[w]["roofline"]["traffic_source"] = "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, summaries in profiles/, measured at " + PROFILED_AT
    if not args.no_cpu:
        if "adamw" in results:
            results["adamw"]["cpu_baseline"] = cpu_adamw(args)
        if "decode" in results:
            results["decode"]["cpu_baseline"] = cpu_decode(args)
        if "train" in results:
            line["cpu_baseline"] = cpu_gemm(args)
        elif "adamw" in results:
            line["cpu_baseline"] = results["adamw"]["cpu_baseline"]
        elif "decode" in results:
            line["cpu_baseline"] = results["decode"]["cpu_baseline"]
    print(json.dumps(line))


if __name__ == "__main__":
    main()
