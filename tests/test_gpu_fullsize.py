"""GPU checks at BASELINE.json's full sizes. Where the CPU oracle finishes in seconds the comparison
is byte for byte (config 4: the whole 120*2^20-weight Integer AdamW sweep); for the training-size GEMMs
(configs 3 and 5) the MFMA kernels are compared against the library's fp32 kernels at full size
(those are themselves pinned to the oracle in test_gpu_gemm.py) and against the oracle on a sampled
subset of experts, and through size-independent properties (linearity in the activations,
wgrad == sum of per-row outer products in any row split)."""
import os
import subprocess

import numpy as np
import pytest

from __graft_entry__ import load_package, PKG_DIR
from oracle.binding import make_spans

pkg = load_package()
f32 = np.float32
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def q():
    return pkg.load()


def dev(a):
    import torch
    if a.dtype.names:
        a = a.view(np.uint8)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_host_mirror_selftest_binary():
    """The C++ host mirror (qlm_gpu_init / qlm_gpu_update / qlm_save / qlm_load / mg_ab + mg_flush)
    run end to end by the compiled selftest, the counterpart of `cudalm selftest`'s QLM section."""
    exe = os.path.join(PKG_DIR, "qlm_selftest")
    assert os.path.exists(exe), "build with python cudalm-c_amd/build.py"
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    print(p.stdout)
    assert p.returncode == 0 and "ALL PASS" in p.stdout, p.stdout


@pytest.mark.parametrize("tag", ["adam", "lion"])
def test_host_mirror_loads_and_rewrites_a_reference_checkpoint(golden, tmp_path, tag):
    """qlm_load of a .opt.q file written by the reference's qlm_save (fixture) into device state, then qlm_save
    from that state: the two files are byte-identical (layout of the fixture: 7 float parameters, span of 384,
    4 floats, span of 256, 2 floats)."""
    g = golden("optq_" + tag)
    src, dst = str(tmp_path / "ref.opt.q"), str(tmp_path / "mine.opt.q")
    g["optq"].tofile(src)
    env = dict(os.environ)
    if tag == "lion":
        env["QLM_OPT"] = "qlion"
    p = subprocess.run([os.path.join(PKG_DIR, "qlm_selftest"), "optq", src, dst, "7", "4", "384", "256"], env=env,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert p.returncode == 0, p.stdout
    assert "iter 4321 prev_gn 2.5" in p.stdout and "nfloat 13" in p.stdout, p.stdout
    assert np.array_equal(np.fromfile(dst, dtype=np.uint8), g["optq"])


def test_host_mirror_init_reference_scales_equal_the_oracle(orc, tmp_path):
    """qlm_gpu_init (qlm.cuh:458-541) on the device against the oracle: group scales bit for bit and every
    span's frozen reference scale (mean of its scales, double sum in group order) bit for bit."""
    sizes = [128 * 300, 128 * 77 + 40, 128 * 1000]
    prefix, gap = 16, 8
    tab, nq, ng = make_spans(sizes, 128, pofs=[prefix, prefix + sizes[0] + gap, prefix + sizes[0] + sizes[1] + 2 * gap])
    np_ = prefix + sum(sizes) + 2 * gap + 2
    P = orc.normal(np_, 77, 1, 0.02)
    src, dst = str(tmp_path / "P.f32"), str(tmp_path / "sref.f32")
    P.tofile(src)
    p = subprocess.run([os.path.join(PKG_DIR, "qlm_selftest"), "sref", src, dst, str(prefix), str(gap)] + [str(n) for n in sizes],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert p.returncode == 0, p.stdout
    assert "4 float gaps holding %d parameters" % (prefix + 2 * gap + 2) in p.stdout, p.stdout
    got = np.fromfile(dst, dtype=f32)
    d = np.zeros((nq + 1) // 2 + 64, np.int8); r = np.zeros(nq, np.int8); s = np.zeros(ng, f32)
    orc.encode(P, d, r, s, tab, 128, 7, 1, ng)
    orc.span_sref(tab, s)
    assert np.array_equal(got[3:].view(np.uint32), s.view(np.uint32))
    assert np.array_equal(got[:3].view(np.uint32), tab["sref"].astype(f32).view(np.uint32))


def test_c4_full_adamw_sweep_bit_exact(q, orc):
    """Config 4: 120*2^20 weights, seeded random integer state, grads ~N(0,1e-3), lr 3e-4,
    betas (0.9, 0.95), wd 0.1, t=1: d, r, m8, v8, m8s, v8s byte-identical to the CPU oracle."""
    import torch
    nq = 120 * 2 ** 20
    group = 128
    tab, _, ng = make_spans([nq], group)
    hd = orc.digits(nq, 0, 20); hr = orc.int8(nq, 0, 21, -64, 64); hm8 = orc.int8(nq, 0, 22, -127, 127)
    hv8 = orc.u8(nq, 0, 23, 0, 255)
    hs = orc.uniform(ng, 0, 24, 0.5, 1.5) * f32(0.02 * 3 / 7)
    hm8s = orc.uniform(ng, 0, 25, 0.5, 1.5) * f32(3e-3 / 127)
    hv8s = orc.uniform(ng, 0, 26, 0.5, 1.5) * f32(3e-3 / 255)
    tab["sref"] = f32(np.mean(hs.astype(np.float64)))
    hG = orc.normal(nq, 0, 27, 1e-3)
    d, r, m8, v8, s, m8s, v8s, G = (dev(x) for x in (hd, hr, hm8, hv8, hs, hm8s, hv8s, hG))
    bc1 = f32(1) - f32(0.9); bc2 = f32(1) - f32(0.95)
    hp = (3e-4, 0.9, 0.95, 0.1, 1.0, None, float(f32(1) / bc1), float(f32(1) / np.sqrt(bc2)), 0, 1, 1, None, 1, 0, ng)
    q.step(None, G, d, r, s, m8, m8s, v8, v8s, dev(tab), 1, group, 7, *hp)
    orc.step(None, hG, hd, hr, hs, hm8, hm8s, hv8, hv8s, tab, group, 7, *hp)
    torch.cuda.synchronize()
    for name, got, want in [("d", d, hd), ("r", r, hr), ("m8", m8, hm8), ("v8", v8, hv8), ("m8s", m8s, hm8s), ("v8s", v8s, hv8s)]:
        g = got.cpu().numpy()
        assert np.array_equal(g.view(np.uint8), want.view(np.uint8)), name
    # the digits stayed inside [-7, 7] and the residuals inside [-64, 64]
    u = d.view(torch.uint8)
    assert int(((u & 15) == 8).sum()) == 0 and int(((u >> 4) == 8).sum()) == 0
    assert int(r.min()) >= -64 and int(r.max()) <= 64


def _packed_random(n, gen):
    import torch
    b = torch.randint(0, 256, (n // 2,), dtype=torch.int16, device="cuda", generator=gen).to(torch.uint8)
    lo = b & 15; hi = b >> 4
    lo = torch.where(lo == 8, torch.zeros_like(lo), lo); hi = torch.where(hi == 8, torch.zeros_like(hi), hi)
    return (lo | (hi << 4)).view(torch.int8)


@pytest.mark.parametrize("E,D,F,rows", [(32, 768, 2048, 16384), (8, 2048, 1408, 16384)])
def test_train_size_mfma_vs_fp32_kernels_and_properties(q, orc, E, D, F, rows):
    """Configs 3 and 5 (one layer's shapes; config 5 on 8 of its 64 experts): Zipf row counts, all three
    orientations at full row count. MFMA vs the fp32 kernels <= 1e-3 relative L2; linearity of the
    forward in the activations; the weight gradient of a row split sums to the unsplit one."""
    import torch
    gen = torch.Generator(device="cuda"); gen.manual_seed(1)
    p = (np.arange(E) + 1.0) ** -1.1
    cnt = np.random.default_rng(0).multinomial(rows, p / p.sum())
    off = np.concatenate([[0], np.cumsum(cnt)]).astype(int)
    nw = E * D * F
    d = _packed_random(nw, gen)
    s = (0.02 * 3 / 7) * (0.5 + torch.rand(nw // 128, device="cuda", generator=gen))
    X = torch.randn(rows * D, device="cuda", generator=gen).to(torch.bfloat16)
    dY = torch.randn(rows * F, device="cuda", generator=gen).to(torch.bfloat16)

    def probs(A, aw, B, bw, C, cw, per_expert=False):
        return q.problems([(A.data_ptr() + int(off[e]) * aw * 2, (B.data_ptr() + int(off[e]) * bw * 2) if B is not None else None,
                            C.data_ptr() + (e * D * F * 4 if per_expert else int(off[e]) * cw * 4),
                            e * D * F, e * D * F // 128, int(cnt[e]), 0.0) for e in range(E)])

    def rel(a, b):
        return float(((a - b).double().norm() / b.double().norm()).item())

    # forward nn: [rows, D] @ W[D, F]
    Y1 = torch.zeros(rows * F, device="cuda"); Y2 = torch.zeros(rows * F, device="cuda")
    q.gemm_nn(d, s, 128, probs(X, D, None, 0, Y1, F), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA)
    q.gemm_nn(d, s, 128, probs(X, D, None, 0, Y2, F), E, D, F, pkg.ACT_BF16, pkg.MATH_F32)
    assert rel(Y1, Y2) < 1e-3
    # linearity: f(-2x) == -2 f(x) up to the matrix core's internal summation rounding
    X2 = (X.float() * -2).to(torch.bfloat16)
    Y3 = torch.zeros(rows * F, device="cuda")
    q.gemm_nn(d, s, 128, probs(X2, D, None, 0, Y3, F), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA)
    assert rel(Y3, -2 * Y1) < 1e-6
    # dgrad tn: [rows, F] @ W[D, F]^T -> [rows, D]
    dX1 = torch.zeros(rows * D, device="cuda"); dX2 = torch.zeros(rows * D, device="cuda")
    q.gemm_tn(d, s, 128, probs(dY, F, None, 0, dX1, D), E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA)
    q.gemm_tn(d, s, 128, probs(dY, F, None, 0, dX2, D), E, F, D, pkg.ACT_BF16, pkg.MATH_F32)
    assert rel(dX1, dX2) < 1e-3
    # the paired input gradient (one continued contraction) against two calls, the second accumulating
    dY2 = torch.randn(rows * F, device="cuda", generator=gen).to(torch.bfloat16)
    dX3 = torch.zeros(rows * D, device="cuda"); dX4 = torch.zeros(rows * D, device="cuda")
    q.gemm_tn_pair(d, s, 128, probs(dY, F, None, 0, dX3, D), probs(dY2, F, None, 0, dX3, D), E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA)
    q.gemm_tn(d, s, 128, probs(dY, F, None, 0, dX4, D), E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA)
    acc = q.problems([(dY2.data_ptr() + int(off[e]) * F * 2, None, dX4.data_ptr() + int(off[e]) * D * 4, e * D * F, e * D * F // 128, int(cnt[e]), 1.0)
                      for e in range(E)])
    q.gemm_tn(d, s, 128, acc, E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA)
    assert rel(dX3, dX4) < 1e-6
    # wgrad nt: G[D, F] += X^T dY per expert
    G1 = torch.zeros(nw, device="cuda"); G2 = torch.zeros(nw, device="cuda")
    q.gemm_nt(probs(X, D, dY, F, G1, 0, True), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA)
    q.gemm_nt(probs(X, D, dY, F, G2, 0, True), E, D, F, pkg.ACT_BF16, pkg.MATH_F32)
    assert rel(G1, G2) < 1e-3
    # splitting every expert's rows in two and accumulating (beta = 1 semantics) gives the same sum
    half = [int(c) // 2 for c in cnt]
    G3 = torch.zeros(nw, device="cuda")
    pa = q.problems([(X.data_ptr() + int(off[e]) * D * 2, dY.data_ptr() + int(off[e]) * F * 2, G3.data_ptr() + e * D * F * 4, 0, 0, half[e], 1.0) for e in range(E)])
    pb = q.problems([(X.data_ptr() + (int(off[e]) + half[e]) * D * 2, dY.data_ptr() + (int(off[e]) + half[e]) * F * 2, G3.data_ptr() + e * D * F * 4, 0, 0, int(cnt[e]) - half[e], 1.0) for e in range(E)])
    q.gemm_nt(pa, E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA)
    q.gemm_nt(pb, E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA)
    assert rel(G3, G1) < 1e-5
    # sampled experts against the CPU oracle (rendered weights, fp32 GEMM)
    torch.cuda.synchronize()
    hs = s.cpu().numpy(); hd = d.cpu().numpy()
    for e in (0, E - 1):
        m = min(int(cnt[e]), 256)
        if m == 0:
            continue
        tab, _, ng = make_spans([D * F], 128)
        P = np.zeros(D * F, f32)
        orc.render(P, hd[e * D * F // 2:(e + 1) * D * F // 2].copy(), hs[e * D * F // 128:(e + 1) * D * F // 128].copy(), tab, 128, 1, 0, ng)
        A = X[int(off[e]) * D:(int(off[e]) + m) * D].float().cpu().numpy()
        want = np.zeros(m * F, f32)
        orc.gemm_nn(A, P, want, m, D, F)
        got = Y1[int(off[e]) * F:(int(off[e]) + m) * F].cpu().numpy()
        assert orc.relerr(got, want) < 1e-3
        B = dY[int(off[e]) * F:(int(off[e]) + m) * F].float().cpu().numpy()
        want = np.zeros(m * D, f32)
        orc.gemm_tn(B, P, want, m, F, D, 0.0)
        got = dX1[int(off[e]) * D:(int(off[e]) + m) * D].cpu().numpy()
        assert orc.relerr(got, want) < 1e-3
    # weight gradients of the most loaded expert (its contraction is the one the launch cuts into slices) and
    # of the least loaded one, over all of their rows, against the oracle
    for e in (int(np.argmax(cnt)), int(np.argmin(np.where(cnt > 0, cnt, 1 << 30)))):
        m = int(cnt[e])
        A = X[int(off[e]) * D:(int(off[e]) + m) * D].float().cpu().numpy()
        B = dY[int(off[e]) * F:(int(off[e]) + m) * F].float().cpu().numpy()
        want = np.zeros(D * F, f32)
        orc.gemm_nt(A, B, want, m, D, F)
        assert orc.relerr(G1[e * D * F:(e + 1) * D * F].cpu().numpy(), want) < 1e-3, (e, m)


@pytest.mark.parametrize("opt,lrmode,clip", [("adam", "rel", None), ("qlion", "rel", None), ("adam", "abs", 0.37)])
def test_host_mirror_update_driver_equals_the_oracle(orc, tmp_path, opt, lrmode, clip):
    """qlm_gpu_init -> five qlm_gpu_update calls through libqlmx_host (cudalm.cu:6082-6103) with QLM_SERVO=2, so the
    servo runs after steps 2 and 4 and the steps behind it work on rescaled groups; d, r, s, m8, v8, m8s, v8s, the
    frozen reference scales and the fp32 view P byte for byte against the oracle's encode / step / servo called in
    the reference's order. QLM_FSTAR=0.02 puts groups with one railed digit under the lower threshold (they shrink)
    and groups with four or more over the upper one (they grow; some groups are built with six weights at the
    group maximum), so every branch of the servo is taken. The last span ends in a short group."""
    group, dmax, steps, fstar = 128, 7, 5, 0.02
    sizes = [128 * 40, 128 * 24, 128 * 9 + 56]
    prefix, gap = 16, 8
    tab, nq, ng = make_spans(sizes, group, pofs=[prefix, prefix + sizes[0] + gap, prefix + sizes[0] + sizes[1] + 2 * gap])
    np_ = prefix + sum(sizes) + 2 * gap + 2
    P = orc.normal(np_, 5, 1, 0.02)
    for si in range(3):                       # every third group: six weights at +- the group's largest magnitude
        pof = int(tab["pof"][si])
        for g in range(0, int(tab["ngrp"][si]) - 1, 3):
            seg = P[pof + g * group: pof + (g + 1) * group]
            seg[5:11] = np.abs(seg).max() * np.array([1, -1, 1, 1, -1, 1], f32)
    G = np.concatenate([orc.normal(np_, 5, 10 + t, 2e-2) for t in range(steps)])
    src, gsrc, dst = str(tmp_path / "P.f32"), str(tmp_path / "G.f32"), str(tmp_path / "state.bin")
    P.tofile(src); G.tofile(gsrc)
    env = dict(os.environ, QLM_SERVO="2", QLM_FSTAR=str(fstar), QLM_LRMODE=lrmode, QLM_TEST_STEPS=str(steps), QLM_TEST_GRADS=gsrc)
    if opt == "qlion":
        env["QLM_OPT"] = "qlion"
    if clip is not None:
        env["QLM_TEST_CLIP"] = repr(clip)
    p = subprocess.run([os.path.join(PKG_DIR, "qlm_selftest"), "update", src, dst, str(prefix), str(gap)] + [str(n) for n in sizes],
                       env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert p.returncode == 0, p.stdout
    adam = opt != "qlion"
    assert "update: %d steps, 2 servo passes, adam %d lrmode %d" % (steps, adam, lrmode == "abs") in p.stdout, p.stdout

    hP = P.copy()
    hd = np.zeros((nq + 1) // 2, np.int8); hr = np.zeros(nq, np.int8); hs = np.zeros(ng, f32)
    hm8 = np.zeros(nq, np.int8); hv8 = np.zeros(nq, np.uint8); hm8s = np.zeros(ng, f32); hv8s = np.zeros(ng, f32)
    orc.encode(hP, hd, hr, hs, tab, group, dmax, 1, ng)
    orc.span_sref(tab, hs)
    orc.render(hP, hd, hs, tab, group, 1, 0, ng)
    b1, b2 = f32(0.9), f32(0.95)
    import ctypes
    powf = ctypes.CDLL("libm.so.6").powf
    powf.restype = ctypes.c_float; powf.argtypes = [ctypes.c_float, ctypes.c_float]
    f_hi, f_lo = float(f32(fstar) * f32(1.5)), float(f32(fstar) * f32(0.5))
    gsp = None if clip is None else np.array([clip, 0], f32)
    rescaled = 0
    for t in range(1, steps + 1):
        bc1 = f32(1) - f32(powf(b1, f32(t))); bc2 = f32(1) - f32(powf(b2, f32(t)))      # the C library's powf, as the driver's caller
        orc.step(hP, G[(t - 1) * np_: t * np_], hd, hr, hs, hm8, hm8s, hv8, hv8s, tab, group, dmax, 3e-4, 0.9, 0.95, 0.1, 1.0, gsp,
                 float(f32(1) / bc1), float(f32(1) / np.sqrt(bc2)), int(lrmode == "abs"), t, int(adam), None, 1, 0, ng)
        if t % 2 == 0:
            before = hs.copy()
            orc.servo(hd, hr, hs, tab, group, dmax, f_hi, f_lo, 1, ng)
            grew, shrank = int((hs > before).sum()), int((hs < before).sum())
            assert grew > 0 and shrank > 0 and grew + shrank < ng, (t, grew, shrank, ng)
            rescaled += grew + shrank
    got = np.fromfile(dst, dtype=np.uint8)
    want = [hd, hr, hm8] + ([hv8] if adam else []) + [hs, hm8s] + ([hv8s] if adam else []) + [tab["sref"].astype(f32), hP]
    names = ["d", "r", "m8"] + (["v8"] if adam else []) + ["s", "m8s"] + (["v8s"] if adam else []) + ["sref", "P"]
    at = 0
    for name, w in zip(names, want):
        wb = np.ascontiguousarray(w).view(np.uint8).ravel()
        assert np.array_equal(got[at: at + wb.size], wb), "%s differs after %d steps (%d groups rescaled on the way)" % (name, steps, rescaled)
        at += wb.size
    assert at == got.size


@pytest.mark.parametrize("prof,debug", [(3, 0), (1, 0), (0, 1)])
def test_host_mirror_check_points_time_their_labels(orc, tmp_path, prof, debug):
    """kchk / prof_report (cudalm.cu:787-855) at the optimizer driver's check points (cudalm.cu:6089, 6101): with
    CUDALM_PROF=3 an event per label and the GPU time between them, with CUDALM_PROF=1 a wait per label and wall time,
    with CUDALM_DEBUG=1 the slowest label; four steps with a servo pass after every second one give four `qlm step`
    and two `qlm servo` entries."""
    sizes = [128 * 12]
    np_ = 4 + sizes[0] + 2
    src, gsrc, dst = str(tmp_path / "P.f32"), str(tmp_path / "G.f32"), str(tmp_path / "state.bin")
    orc.normal(np_, 7, 1, 0.02).tofile(src)
    np.concatenate([orc.normal(np_, 7, 10 + t, 2e-2) for t in range(4)]).tofile(gsrc)
    env = dict(os.environ, QLM_SERVO="2", QLM_TEST_STEPS="4", QLM_TEST_GRADS=gsrc, CUDALM_PROF=str(prof), CUDALM_DEBUG=str(debug))
    p = subprocess.run([os.path.join(PKG_DIR, "qlm_selftest"), "update", src, dst, "4", "0"] + [str(n) for n in sizes],
                       env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert p.returncode == 0, p.stdout
    if prof:
        assert "[prof]" in p.stdout, p.stdout
        step = [l for l in p.stdout.splitlines() if l.strip().startswith("qlm step")][0]
        servo = [l for l in p.stdout.splitlines() if l.strip().startswith("qlm servo")][0]
        # the first mark of the event mode only starts the clock: three of the four steps are intervals
        assert (" x3 " in step + " " or " x4" in step) and " x2" in servo, p.stdout
        if prof >= 3:                                   # GPU time to a microsecond; the waiting mode prints tenths of a millisecond
            assert float(step.split()[2]) > 0.0 and float(servo.split()[2]) > 0.0 and "drained" in step, p.stdout
        else:
            assert float(step.split()[2]) >= float(servo.split()[2]) >= 0.0, p.stdout
    if debug:
        assert "slowest label: qlm " in p.stdout, p.stdout


def test_label_timing_through_the_c_abi(q):
    """qlmx_prof_mark / qlmx_prof_report: a long fill and a short one behind their marks; the long one's label takes
    more GPU time, counts add up, the report is sorted, qlmx_prof_reset forgets."""
    import torch
    cur = torch.cuda.current_stream().cuda_stream
    big = torch.empty(1 << 28, dtype=torch.uint8, device="cuda"); small = torch.empty(1 << 12, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    q.call("qlmx_prof_reset")
    q.prof_mark("start", cur)
    for rep in range(5):
        q.call("qlmx_memset", big, rep, big.numel(), cur); q.prof_mark("big fill", cur)
        q.call("qlmx_memset", small, rep, small.numel(), cur); q.prof_mark("small fill", cur)
    text, n = q.prof_report()
    assert n == 3, text
    lines = [l.split() for l in text.splitlines()[1:]]
    got = {" ".join(l[:-6]): (float(l[-6]), int(l[-3][1:]), int(l[-1])) for l in lines}    # name, ms, "ms", share, xN, "drained", count
    assert got["big fill"][1] == 5 and got["small fill"][1] == 5 and got["start"][1] == 0, text
    assert got["big fill"][0] > 5 * got["small fill"][0] > 0.0, text
    assert lines[0][0] == "big", text                       # largest total first
    q.call("qlmx_prof_reset")
    text, n = q.prof_report()
    assert n == 0, text
