"""Writes the golden vectors under tests/golden/ from the reference's own CPU backend.

Runs only where oracle/_ref/libcudalm_ref.so exists (a container that mounts the reference and has
run `make -C oracle`). Every expected output below is produced by the reference's compiled code
(qlm.cuh / cpu_kern.h / cpu_rt.h through oracle/ref_shim.cpp); inputs come from the repository's
deterministic generator and are stored beside the outputs, so the fixtures are self-contained data.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle.binding import Oracle, Ref, make_spans  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))
gen = Oracle()      # used ONLY as the input generator here
ref = Ref()

f32 = np.float32


def save(name, **arrs):
    path = os.path.join(OUT, name + ".npz")
    np.savez_compressed(path, **arrs)
    print("%-28s %7.1f KB" % (name + ".npz", os.path.getsize(path) / 1024))


# ---------------------------------------------------------------- hash / stochastic rounding
def golden_hash():
    xs = np.array([0, 1, 2, 0xFFFFFFFF, 0x100000000, 0xFFFFFFFFFFFFFFFF, 0x9E3779B97F4A7C15,
                   0x0123456789ABCDEF] + [int(gen.uniform(1, 7, k, 0, 1)[0] * 2**24) * 0x10000000001 + k
                                          for k in range(56)], dtype=np.uint64)
    hs = np.array([ref.qhashu(int(x)) for x in xs], dtype=np.uint32)
    v = gen.uniform(512, 7, 100, -9.0, 9.0)
    v[:16] = [0.0, -0.0, 0.5, -0.5, 1.0, -1.0, 7.999999, -7.999999, 0.25, -0.25, 3.0, -3.0,
              1e-7, -1e-7, 63.5, -63.5]
    i = (gen.uniform(512, 7, 101, 0, 1) * 2**24).astype(np.uint64) * np.uint64(977) + np.uint64(3)
    i[:4] = [0, 1, 2**32 - 1, 2**40 + 12345]
    t = (gen.uniform(512, 7, 102, 0, 1) * 5000).astype(np.uint64) + np.uint64(1)
    t[4:8] += np.uint64(0x5EED)
    t[8:12] += np.uint64(0xBEEF)
    q = np.array([ref.qsri(float(a), int(b), int(c)) for a, b, c in zip(v, i, t)], dtype=np.int32)
    save("hash", x=xs, h=hs, v=v, i=i, t=t, q=q)


# ---------------------------------------------------------------- nibble packing
def golden_nibble():
    nq = 37
    vals = gen.int8(nq, 7, 200, -7, 7)
    d = np.zeros(int(ref.qd_bytes(nq, 1)), dtype=np.int8)
    for k in range(nq):
        ref.qd_set(d, k, int(vals[k]), 1)
    back = np.array([ref.qd_get(d, k, 1) for k in range(nq)], dtype=np.int8)
    allbytes = np.arange(256, dtype=np.uint8).view(np.int8)
    lo = np.array([ref.qd_get(allbytes, 2 * k, 1) for k in range(256)], dtype=np.int8)
    hi = np.array([ref.qd_get(allbytes, 2 * k + 1, 1) for k in range(256)], dtype=np.int8)
    save("nibble", vals=vals, packed=d, back=back, lo=lo, hi=hi,
         nbytes=np.array([ref.qd_bytes(n, 1) for n in range(9)], dtype=np.uint64))


# ---------------------------------------------------------------- encode / render / step / servo
CFGS = [
    # name       group dmax packed adam lrmode v4 sizes
    ("g128_adam_rel", 128, 7, 1, 1, 0, 0, [128 * 4 + 38, 600, 128 * 2 + 1]),
    ("g128_adam_abs", 128, 7, 1, 1, 1, 0, [128 * 3, 128 * 2]),
    ("g128_lion",     128, 7, 1, 0, 0, 0, [128 * 3, 128 + 2]),
    ("g64_d3_v4",      64, 3, 1, 1, 0, 1, [64 * 5, 64 * 2 + 10]),
    ("g256_int8",     256, 127, 0, 1, 0, 0, [256 * 2 + 5, 300]),
    ("g96_block",      96, 7, 1, 1, 0, 0, [96 * 4, 96 + 50]),
    ("g32_ternary",    32, 1, 1, 1, 0, 0, [32 * 9, 70]),
]


def golden_qlm():
    for (name, group, dmax, packed, adam, lrmode, v4, sizes) in CFGS:
        tab, nq, ng = make_spans(sizes, group)
        # gradients live at a different offset than the weights in the second span
        if len(sizes) > 1:
            tab[1]["gof"] = tab[1]["pof"] + 16
        npar = nq + 16
        P0 = gen.normal(npar, 0, 300, 0.02)
        P0[5:9] = 0.0
        if ng > 2:                       # an all-zero group: scale floor 1e-8
            P0[int(tab[0]["pof"]) + group: int(tab[0]["pof"]) + 2 * group] = 0.0
        out = {"sizes": np.array(sizes), "cfg": np.array([group, dmax, packed, adam, lrmode, v4]), "P0": P0}
        P = P0.copy()
        d = np.zeros(int(ref.qd_bytes(nq, packed)), np.int8)
        r = np.zeros(nq, np.int8)
        s = np.zeros(ng, f32)
        ref.encode(P, d, r, s, tab, group, dmax, packed, ng)
        gen.span_sref(tab, s)            # host arithmetic of qlm.cuh:527-536 (double mean)
        ref.render(P, d, s, tab, group, packed, 0, ng)
        out.update(enc_d=d.copy(), enc_r=r.copy(), enc_s=s.copy(), enc_P=P.copy(), tab=tab.copy())
        m8 = np.zeros(nq, np.int8)
        v8 = np.zeros(nq, np.uint8)
        m8s = np.zeros(ng, f32)
        v8s = np.zeros(ng, f32)
        stat = np.zeros(4, np.int64)
        lr, b1, b2, wd = 3e-4, 0.9, 0.95, 0.1
        gsp = np.array([0.37], f32)
        for t in range(1, 5):
            G = gen.normal(npar, 0, 310 + t, 1e-3 if t != 3 else 0.3)
            # t==2: a large learning rate forces multi-carries; t==3 uses the device clip scalar
            lr_t = lr if t != 2 else 0.05
            bc1 = f32(1) - f32(b1) ** f32(t)
            bc2 = f32(1) - f32(b2) ** f32(t)
            inv_bc1 = float(f32(1) / bc1)
            inv_sqrt_bc2 = float(f32(1) / np.sqrt(bc2))
            if t == 2:
                r[: min(nq, 8)] = [64, 64, -64, -64, 63, -63, 0, 1][: min(nq, 8)]
                out["t2_r_in"] = r.copy()
            ref.step(P, G, d, r, s, m8, m8s, v8 if adam else None, v8s if adam else None, tab, group, dmax,
                     lr_t, b1, b2, wd, 1.0 if t != 3 else 0.0, gsp if t == 3 else None,
                     inv_bc1, inv_sqrt_bc2, lrmode, t, adam, stat, packed, 0, ng, v4)
            out.update({"G%d" % t: G, "P%d" % t: P.copy(), "d%d" % t: d.copy(), "r%d" % t: r.copy(),
                        "m8_%d" % t: m8.copy(), "v8_%d" % t: v8.copy(), "m8s_%d" % t: m8s.copy(),
                        "v8s_%d" % t: v8s.copy(), "hp%d" % t: np.array([lr_t, b1, b2, wd, inv_bc1, inv_sqrt_bc2], f32)})
        out["stat"] = stat.copy()
        # a sub-range step (fused per-layer update): only groups [1, 1+ng2)
        ng2 = max(1, ng // 2)
        G = gen.normal(npar, 0, 330, 1e-3)
        ref.step(P, G, d, r, s, m8, m8s, v8 if adam else None, v8s if adam else None, tab, group, dmax,
                 lr, b1, b2, wd, 1.0, None, 1.5, 1.25, lrmode, 5, adam, None, packed, 1, ng2, v4)
        out.update(G5=G, P5=P.copy(), d5=d.copy(), r5=r.copy(), m8_5=m8.copy(), v8_5=v8.copy(),
                   m8s_5=m8s.copy(), v8s_5=v8s.copy(), sub=np.array([1, ng2]))
        # servo: force one group to rail (grow), one to have no railed digit (shrink), rest idle
        dd = gen.unpack(d, nq, packed).astype(np.int64)
        g_grow, g_shrink = 0, min(1, ng - 1)
        q0 = int(tab[0]["qi0"])
        dd[q0 + g_grow * group: q0 + g_grow * group + group // 2] = dmax
        if ng > 1:
            sl = slice(q0 + g_shrink * group, q0 + g_shrink * group + group)
            dd[sl] = np.clip(dd[sl], -(dmax - 1) if dmax > 1 else 0, (dmax - 1) if dmax > 1 else 0)
        for k in range(nq):
            ref.qd_set(d, k, int(dd[k]), packed)
        fstar = 1.5 / group if dmax > 1 else 0.60
        out.update(sv_d_in=d.copy(), sv_r_in=r.copy(), sv_s_in=s.copy(), sv_f=np.array([fstar * 1.5, fstar * 0.5], f32))
        ref.servo(d, r, s, tab, group, dmax, fstar * 1.5, fstar * 0.5, packed, ng)
        out.update(sv_d=d.copy(), sv_r=r.copy(), sv_s=s.copy())
        save("qlm_" + name, **out)


# ---------------------------------------------------------------- GEMM wrappers + MoE glue
def golden_gemm():
    M, K, N = 67, 53, 91            # the reference selftest's shape (cudalm.cu:9919-9946)
    A = gen.normal(M * K, 0, 400)
    B = gen.normal(K * N, 0, 401)
    Bt = gen.normal(N * K, 0, 402)
    B2 = gen.normal(M * N, 0, 403)
    C0 = gen.normal(M * N, 0, 404)
    W0 = gen.normal(K * N, 0, 405)
    nn = np.zeros(M * N, f32)
    ref.gemm_nn(A, B, nn, M, K, N)
    tn0 = C0.copy()
    ref.gemm_tn(A, Bt, tn0, M, K, N, 0.0)
    tn1 = C0.copy()
    ref.gemm_tn(A, Bt, tn1, M, K, N, 1.0)
    nt = W0.copy()
    ref.gemm_nt(A, B2, nt, M, K, N)
    # grouped queue semantics: two problems then one flush
    g0 = np.zeros(M * N, f32)
    g1 = np.zeros(5 * N, f32)
    ref.gemm_nn(A, B, g0, M, K, N, grouped=True)
    ref.gemm_nn(A[: 5 * K], B, g1, 5, K, N, grouped=True)
    ref.mg_flush()
    save("gemm", dims=np.array([M, K, N]), A=A, B=B, Bt=Bt, B2=B2, C0=C0, W0=W0, nn=nn, tn0=tn0, tn1=tn1,
         nt=nt, g0=g0, g1=g1)


def golden_router():
    out = {}
    for tag, (N, E, K) in {"a": (96, 32, 2), "b": (40, 8, 4), "c": (33, 64, 4)}.items():
        rt = gen.normal(N * E, 0, 500 + ord(tag), 1.0)
        rt[:E] = 0.25                      # exact ties: lowest index must win, K times
        rt[E: 2 * E] = np.repeat(gen.normal(E // 2, 0, 600, 1.0), 2)   # pairwise ties
        pr = np.zeros(N * E, f32)
        asn = np.zeros(K * N, np.int32)
        gate = np.zeros(K * N, f32)
        ref.router_topk(rt, pr, asn, gate, N, E, K)
        out.update({"dims_" + tag: np.array([N, E, K]), "rt_" + tag: rt, "pr_" + tag: pr,
                    "asn_" + tag: asn, "gate_" + tag: gate})
    N, E, K = 96, 32, 2
    bias = gen.normal(K * E, 0, 700, 0.02)
    pr = np.zeros(N * E, f32)
    asn = np.zeros(K * N, np.int32)
    gate = np.zeros(K * N, f32)
    ref.router_topk(out["rt_a"], pr, asn, gate, N, E, K, bias, E)
    out.update(bias=bias, asn_bias=asn, gate_bias=gate)
    save("router", **out)


def golden_glue():
    N, D = 50, 24
    src = gen.normal(N * D, 0, 800)
    perm = np.argsort(gen.uniform(N, 0, 801), kind="stable").astype(np.int32)
    gate = gen.uniform(N, 0, 802, 0.1, 0.6)
    Xp = np.zeros(N * D, f32)
    ref.gather(src, perm, Xp, N, D)
    out0 = gen.normal(N * D, 0, 803)
    sg = out0.copy()
    ref.scatter_gate(Xp, perm, gate, sg, N, D)
    sa = out0.copy()
    ref.scatter_add(Xp, perm, sa, N, D)
    dout = gen.normal(N * D, 0, 804)
    dgate = np.zeros(N, f32)
    dyp = np.zeros(N * D, f32)
    ref.moe_dgate(dout, Xp, perm, gate, dgate, dyp, N, D)
    n = 1003
    G = gen.normal(n, 0, 805, 2.0)
    U = gen.normal(n, 0, 806)
    dA = gen.normal(n, 0, 807)
    O = np.zeros(n, f32)
    ref.swiglu(G, U, O)
    dg = np.zeros(n, f32)
    du = np.zeros(n, f32)
    ref.swiglu_bwd(G, U, dA, dg, du)
    save("glue", dims=np.array([N, D]), src=src, perm=perm, gate=gate, Xp=Xp, out0=out0, sg=sg, sa=sa,
         dout=dout, dgate=dgate, dyp=dyp, G=G, U=U, dA=dA, O=O, dg=dg, du=du)


def golden_step_touched():
    """k_ng_q4_step (cpu_kern.h:620-648): two steps over a list of touched groups of one packed span of
    128*10 + 64 weights (the last group is a short tail), compact gradients, the second step with a
    device clip scalar and a large learning rate (carries)."""
    group, dmax = 128, 7
    nt = 128 * 10 + 64
    ng = 11
    d = gen.digits(nt, 0, 950)
    r = gen.int8(nt, 0, 951, -64, 64)
    m8 = gen.int8(nt, 0, 952, -127, 127)
    v8 = gen.u8(nt, 0, 953, 0, 255)
    s = (0.02 * 3 / 7) * gen.uniform(ng, 0, 954, 0.5, 1.5)
    m8s = (3e-3 / 127) * gen.uniform(ng, 0, 955, 0.5, 1.5)
    v8s = (3e-3 / 255) * gen.uniform(ng, 0, 956, 0.5, 1.5)
    sref = float(np.mean(s.astype(np.float64)))
    P = np.zeros(nt, f32)
    out = {"dims": np.array([nt, group, dmax]), "sref": np.array([sref], f32),
           "d0": d.copy(), "r0": r.copy(), "m8_0": m8.copy(), "v8_0": v8.copy(), "s": s.copy(),
           "m8s_0": m8s.copy(), "v8s_0": v8s.copy()}
    b1, b2, wd = 0.9, 0.95, 0.1
    for t, touched, lr, gs in [(1, [0, 3, 7, 10], 3e-4, None), (2, [10, 2, 3], 0.05, np.array([0.37], f32))]:
        touched = np.array(touched, np.int32)
        Gc = gen.normal(touched.size * group, 0, 960 + t, 1e-3 if t == 1 else 0.2)
        bc1 = f32(1) - f32(b1) ** f32(t); bc2 = f32(1) - f32(b2) ** f32(t)
        inv_bc1 = float(f32(1) / bc1); inv_sqrt_bc2 = float(f32(1) / np.sqrt(bc2))
        ref.step_touched(P, Gc, d, r, s, m8, m8s, v8, v8s, touched, group, dmax, lr, b1, b2, wd, sref,
                         inv_bc1, inv_sqrt_bc2, t, nt, gs)
        out.update({"touched%d" % t: touched, "Gc%d" % t: Gc, "hp%d" % t: np.array([lr, b1, b2, wd, inv_bc1, inv_sqrt_bc2], f32),
                    "P%d" % t: P.copy(), "d%d" % t: d.copy(), "r%d" % t: r.copy(), "m8_%d" % t: m8.copy(),
                    "v8_%d" % t: v8.copy(), "m8s_%d" % t: m8s.copy(), "v8s_%d" % t: v8s.copy()})
    out["gs2"] = np.array([0.37], f32)
    save("step_touched", **out)


def golden_gnorm():
    """k_sqsum and k_gnorm (cpu_kern.h:533-546): the 64 partial sums of squares of three gradient
    vectors (one shorter than 64, one not a multiple of 64, one large enough for a norm above 1) and
    the clip multiplier / norm pairs with and without side slices."""
    out = {}
    for k, (n, scale) in enumerate([(50, 1e-3), (1000 * 3 + 7, 1e-2), (1 << 18, 3e-3)]):
        G = gen.normal(n, 0, 970 + k, scale)
        out["n%d" % k] = np.array([n]); out["seed%d" % k] = np.array([970 + k]); out["scale%d" % k] = np.array([scale], np.float64)
        out["part%d" % k] = ref.sqsum(G)
    side = np.concatenate([out["part2"], out["part1"], out["part0"]])
    for cs in (0, 1):
        out["gs_side%d" % cs] = ref.gnorm(side, 2, cs)
    out["gs_small"] = ref.gnorm(out["part0"], 0, 0)
    bad = side.copy(); bad[70] = np.inf
    out["gs_inf"] = ref.gnorm(bad, 2, 0)
    save("gnorm", **out)


def golden_q4n():
    """q4n wire format (cudalm.cu:638-656): groups on the 4-bit grid (rendered QLM view), groups off
    the grid (stored raw), an all-zero group, a one-hot group and a short tail."""
    group = 128
    n = 128 * 7 + 50
    tab, nq, ng = make_spans([128 * 8], group)
    P0 = gen.normal(128 * 8, 0, 900, 0.02)
    d = np.zeros(nq // 2, np.int8); r = np.zeros(nq, np.int8); s = np.zeros(ng, f32)
    ref.encode(P0, d, r, s, tab, group, 7, 1, ng)
    ref.render(P0, d, s, tab, group, 1, 0, ng)            # P0 = s * digit: on the grid
    P = P0[:n].copy()
    P[128:256] = gen.normal(128, 0, 901, 0.02)            # off the grid -> raw
    P[256:384] = 0.0                                      # all zero -> scale 0
    P[384:512] = 0.0; P[400] = -0.0371                    # one value -> scale = |v| / 7 .. / 1 candidates
    P[512:640] *= f32(0.5)                                # still on a grid (power of two)
    buf = ref.q4n_quantize(P, group)
    ok, back = ref.q4n_dequantize(buf, n, group)
    assert ok == 1
    buf64 = ref.q4n_quantize(P[:300], 64)
    save("q4n", dims=np.array([n, group]), P=P, buf=buf, back=back, buf64=buf64)


def golden_optq():
    """.opt.q checkpoints written by the reference's qlm_save (qlm.cuh:702-738): Integer AdamW state and
    integer Lion state (no v8 / v8s sections), two spans around float parameters (compact bf16 moments),
    with the SREF and PGN1 trailers. The fixture holds every input array and the file's bytes."""
    import tempfile
    group = 128
    for tag, adam in (("adam", 1), ("lion", 0)):
        sizes = [128 * 3, 128 * 2]
        tab, nq, ng = make_spans(sizes, group, pofs=[7, 7 + sizes[0] + 4])
        nfloat = 7 + 4 + 2
        seed = 950 + adam
        d = gen.digits(nq, seed, 1); r = gen.int8(nq, seed, 2, -64, 64); m8 = gen.int8(nq, seed, 3, -127, 127)
        v8 = gen.u8(nq, seed, 4, 0, 255)
        s = gen.uniform(ng, seed, 5, 0.5, 1.5) * f32(0.02 * 3 / 7)
        m8s = gen.uniform(ng, seed, 6, 0.5, 1.5) * f32(3e-3 / 127)
        v8s = gen.uniform(ng, seed, 7, 0.5, 1.5) * f32(3e-3 / 255)
        Mc = (gen.normal(nfloat, seed, 8).view(np.uint32) >> 16).astype(np.uint16)
        Vc = (gen.uniform(nfloat, seed, 9).view(np.uint32) >> 16).astype(np.uint16)
        tab["sref"] = [f32(0.0123), f32(0.0077)]
        with tempfile.TemporaryDirectory() as td:
            path = os.path.join(td, "ck.opt.q")
            ok = ref.qlm_save(path, 4321, 2.5, 7, group, adam, 1, tab, nfloat, Mc, Vc, d, r, m8, v8 if adam else None,
                              s, m8s, v8s if adam else None)
            assert ok == 1
            data = np.fromfile(path, dtype=np.uint8)
        save("optq_" + tag, dims=np.array([7, group, adam, 1, 4321, nfloat]), prev_gn=np.array([2.5], f32), tab=tab.view(np.uint8),
             Mc=Mc, Vc=Vc, d=d, r=r, m8=m8, v8=v8, s=s, m8s=m8s, v8s=v8s, optq=data)


if __name__ == "__main__":
    golden_optq()
    golden_gnorm()
    golden_q4n()
    golden_step_touched()
    golden_hash()
    golden_nibble()
    golden_qlm()
    golden_gemm()
    golden_router()
    golden_glue()
