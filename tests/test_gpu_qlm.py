"""GPU parity for the quantized weight format and the integer optimizer: every byte of d, r, m8,
v8, the scales and the rendered view must equal the golden vectors (written by the reference's CPU
backend) and the CPU oracle on the same seeded inputs. All calls go through the C ABI."""
import numpy as np
import pytest

from __graft_entry__ import load_package
from oracle.binding import make_spans

pkg = load_package()
f32 = np.float32
pytestmark = pytest.mark.gpu

QLM_CASES = ["g128_adam_rel", "g128_adam_abs", "g128_lion", "g64_d3_v4", "g256_int8", "g96_block", "g32_ternary"]


@pytest.fixture(scope="module")
def q():
    return pkg.load()


def dev(a):
    import torch
    if a.dtype.names:
        a = a.view(np.uint8)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


def beq(t, ref):
    got = host(t) if hasattr(t, "cpu") else t
    return np.array_equal(np.ascontiguousarray(got).view(np.uint8), np.ascontiguousarray(ref).view(np.uint8))


@pytest.mark.parametrize("name", QLM_CASES)
def test_golden_encode_render_step_servo(q, golden, name):
    import torch
    g = golden("qlm_" + name)
    group, dmax, packed, adam, lrmode, v4 = (int(x) for x in g["cfg"])
    tab0, nq, ng = make_spans([int(x) for x in g["sizes"]], group)
    tab0["gof"] = g["tab"]["gof"]
    nsp = len(tab0)
    P = dev(g["P0"])
    d = torch.zeros(len(g["enc_d"]), dtype=torch.int8, device="cuda")
    r = torch.zeros(nq, dtype=torch.int8, device="cuda")
    s = torch.zeros(ng, dtype=torch.float32, device="cuda")
    sp = dev(tab0)
    q.encode(P, d, r, s, sp, nsp, group, dmax, packed, ng)
    assert beq(d, g["enc_d"]) and beq(r, g["enc_r"]) and beq(s, g["enc_s"])
    sp = dev(g["tab"])
    q.render(P, d, s, sp, nsp, group, packed, 0, ng)
    assert beq(P, g["enc_P"])
    m8 = torch.zeros(nq, dtype=torch.int8, device="cuda"); v8 = torch.zeros(nq, dtype=torch.uint8, device="cuda")
    m8s = torch.zeros(ng, device="cuda"); v8s = torch.zeros(ng, device="cuda")
    stat = torch.zeros(4, dtype=torch.int64, device="cuda")
    gsp = dev(np.array([0.37], f32))
    for t in range(1, 5):
        hp = g["hp%d" % t]
        if t == 2:
            r = dev(g["t2_r_in"])
        q.step(P, dev(g["G%d" % t]), d, r, s, m8, m8s, v8 if adam else None, v8s if adam else None, sp, nsp, group,
               dmax, float(hp[0]), float(hp[1]), float(hp[2]), float(hp[3]), 1.0 if t != 3 else 0.0,
               gsp if t == 3 else None, float(hp[4]), float(hp[5]), lrmode, t, adam, stat, packed, 0, ng, v4)
        for buf, key in [(P, "P%d"), (d, "d%d"), (r, "r%d"), (m8, "m8_%d"), (m8s, "m8s_%d")]:
            assert beq(buf, g[key % t]), (name, t, key)
        if adam:
            assert beq(v8, g["v8_%d" % t]) and beq(v8s, g["v8s_%d" % t]), (name, t)
    assert np.array_equal(host(stat), g["stat"])
    gi_base, ng2 = (int(x) for x in g["sub"])
    q.step(P, dev(g["G5"]), d, r, s, m8, m8s, v8 if adam else None, v8s if adam else None, sp, nsp, group, dmax,
           3e-4, 0.9, 0.95, 0.1, 1.0, None, 1.5, 1.25, lrmode, 5, adam, None, packed, gi_base, ng2, v4)
    for buf, key in [(P, "P5"), (d, "d5"), (r, "r5"), (m8, "m8_5"), (m8s, "m8s_5")]:
        assert beq(buf, g[key]), (name, "sub", key)
    d2, r2, s2 = dev(g["sv_d_in"]), dev(g["sv_r_in"]), dev(g["sv_s_in"])
    q.servo(d2, r2, s2, sp, nsp, group, dmax, float(g["sv_f"][0]), float(g["sv_f"][1]), packed, ng)
    assert beq(d2, g["sv_d"]) and beq(r2, g["sv_r"]) and beq(s2, g["sv_s"])


def test_servo_vs_oracle_seeded(q, orc):
    """Servo over 1M weights in two spans (the second ends in a short group): thresholds chosen so that
    groups go up, down and stay; digits, residuals and scales byte-identical to the CPU oracle."""
    group, dmax = 128, 7
    tab, nq, ng = make_spans([128 * 5000, 128 * 3000 + 40], group)
    hd = orc.digits(nq, 3, 1); hr = orc.int8(nq, 3, 2, -64, 64)
    hs = orc.uniform(ng, 3, 3, 0.5, 1.5) * f32(0.02 * 3 / 7)
    # uniform digits rail 2/15 of the elements on average: thresholds either side of that
    f_hi, f_lo = 0.15, 0.11
    d, r, s = dev(hd), dev(hr), dev(hs)
    q.servo(d, r, s, dev(tab), len(tab), group, dmax, f_hi, f_lo, 1, ng)
    s0 = hs.copy()
    orc.servo(hd, hr, hs, tab, group, dmax, f_hi, f_lo, 1, ng)
    assert beq(d, hd) and beq(r, hr) and beq(s, hs)
    up, down = int((hs > s0).sum()), int((hs < s0).sum())
    assert up > 100 and down > 100 and ng - up - down > 100


@pytest.mark.parametrize("nopview", [False, True])
def test_step_vs_oracle_seeded_2m(q, orc, nopview):
    """Three consecutive steps over 2M weights in two spans (one with a short tail group and a
    shifted gradient offset), random integer state: byte-identical to the CPU oracle. With P=NULL
    the integer state must be the same as with the view rendered."""
    import torch
    group, dmax = 128, 7
    tab, nq, ng = make_spans([128 * 9000, 128 * 7000 + 66], group)
    tab[1]["gof"] = tab[1]["pof"] + 8
    tab["sref"] = [0.0086, 0.0091]
    npar = nq + 8
    hd = orc.digits(nq, 1, 20); hr = orc.int8(nq, 1, 21, -64, 64); hm8 = orc.int8(nq, 1, 22, -127, 127)
    hv8 = orc.u8(nq, 1, 23, 0, 255)
    hs = orc.uniform(ng, 1, 24, 0.5, 1.5) * f32(0.02 * 3 / 7)
    hm8s = orc.uniform(ng, 1, 25, 0.5, 1.5) * f32(3e-3 / 127); hv8s = orc.uniform(ng, 1, 26, 0.5, 1.5) * f32(3e-3 / 255)
    hP = np.zeros(npar, f32)
    d, r, m8, v8, s, m8s, v8s = (dev(x) for x in (hd, hr, hm8, hv8, hs, hm8s, hv8s))
    P = None if nopview else dev(hP)
    sp = dev(tab)
    stat = torch.zeros(4, dtype=torch.int64, device="cuda"); hstat = np.zeros(4, np.int64)
    for t in range(1, 4):
        hG = orc.normal(npar, 1, 30 + t, 1e-3)
        bc1 = f32(1) - f32(0.9) ** f32(t); bc2 = f32(1) - f32(0.95) ** f32(t)
        hp = (3e-4, 0.9, 0.95, 0.1, 1.0, None, float(f32(1) / bc1), float(f32(1) / np.sqrt(bc2)), 0, t, 1)
        q.step(P, dev(hG), d, r, s, m8, m8s, v8, v8s, sp, 2, group, dmax, *hp, stat, 1, 0, ng)
        orc.step(hP, hG, hd, hr, hs, hm8, hm8s, hv8, hv8s, tab, group, dmax, *hp, hstat, 1, 0, ng)
    for got, want, nm in [(d, hd, "d"), (r, hr, "r"), (m8, hm8, "m8"), (v8, hv8, "v8"), (m8s, hm8s, "m8s"), (v8s, hv8s, "v8s")]:
        assert beq(got, want), nm
    if not nopview:
        assert beq(P, hP)
    assert np.array_equal(host(stat), hstat)


def test_encode_render_vs_oracle_and_invariants(q, orc):
    """4M weights: bytes equal the oracle's; rendered error <= 0.51 step; <= 15 levels per group
    (cudalm.cu:10494-10523); render(encode(render(x))) is a fixed point."""
    import torch
    group, dmax = 128, 7
    tab, nq, ng = make_spans([128 * 32768], group)
    hP0 = orc.normal(nq, 2, 1, 0.02)
    hP = hP0.copy(); hd = np.zeros(nq // 2, np.int8); hr = np.zeros(nq, np.int8); hs = np.zeros(ng, f32)
    orc.encode(hP, hd, hr, hs, tab, group, dmax, 1, ng)
    orc.render(hP, hd, hs, tab, group, 1, 0, ng)
    P = dev(hP0); d = torch.zeros(nq // 2, dtype=torch.int8, device="cuda")
    r = torch.zeros(nq, dtype=torch.int8, device="cuda"); s = torch.zeros(ng, device="cuda")
    sp = dev(tab)
    q.encode(P, d, r, s, sp, 1, group, dmax, 1, ng)
    q.render(P, d, s, sp, 1, group, 1, 0, ng)
    assert beq(d, hd) and beq(r, hr) and beq(s, hs) and beq(P, hP)
    err = (P.view(ng, group) - dev(hP0).view(ng, group)).abs() / s[:, None]
    assert float(err.max()) <= 0.51
    d2 = torch.zeros_like(d); r2 = torch.zeros_like(r); s2 = torch.zeros_like(s); P2 = P.clone()
    q.encode(P2, d2, r2, s2, sp, 1, group, dmax, 1, ng)
    q.render(P2, d2, s2, sp, 1, group, 1, 0, ng)
    assert float((P2 - P).abs().max()) <= float(s.max()) * 1e-6 and int(r2.abs().max()) <= 1


def test_step_touched_vs_reference_fixture(q, golden):
    """k_ng_q4_step (cudalm.cu:4472): list-driven step, bytes and bits against the reference's output."""
    import torch
    g = golden("step_touched")
    nt, group, dmax = (int(v) for v in g["dims"])
    d, r, m8, v8 = dev(g["d0"]), dev(g["r0"]), dev(g["m8_0"]), dev(g["v8_0"])
    s, m8s, v8s = dev(g["s"]), dev(g["m8s_0"]), dev(g["v8s_0"])
    P = torch.zeros(nt, device="cuda")
    gs2 = dev(g["gs2"])
    for t in (1, 2):
        lr, b1, b2, wd, ib1, ib2 = (float(v) for v in g["hp%d" % t])
        touched = dev(g["touched%d" % t])
        q.step_touched(P, dev(g["Gc%d" % t]), d, r, s, m8, m8s, v8, v8s, touched, touched.numel(), group, dmax,
                       lr, b1, b2, wd, float(g["sref"][0]), ib1, ib2, t, nt, gs2 if t == 2 else None)
        torch.cuda.synchronize()
        for name, got in (("d", d), ("r", r), ("m8_", m8), ("v8_", v8), ("m8s_", m8s), ("v8s_", v8s), ("P", P)):
            assert beq(got, g["%s%d" % (name, t)]), (name, t)


@pytest.mark.parametrize("v4", [0, 1])
def test_step_touched_vs_oracle_sparse_table(q, orc, v4):
    """A 4 M-weight table of which 3000 random groups are touched (plus the short tail group)."""
    import torch
    group, dmax = 128, 7
    nt = 128 * 32768 + 96
    ng = (nt + group - 1) // group
    d, r = orc.digits(nt, 6, 1), orc.int8(nt, 6, 2, -64, 64)
    m8, v8 = orc.int8(nt, 6, 3, -127, 127), orc.u8(nt, 6, 4, 0, 255)
    s = (0.02 * 3 / 7) * orc.uniform(ng, 6, 5, 0.5, 1.5)
    m8s = (3e-3 / 127) * orc.uniform(ng, 6, 6, 0.5, 1.5)
    v8s = (3e-3 / 255) * orc.uniform(ng, 6, 7, 0.5, 1.5)
    if v4:
        v8s = np.sqrt(v8s).astype(f32)
    rng = np.random.default_rng(6)
    touched = np.concatenate([rng.choice(ng - 1, 3000, replace=False), [ng - 1]]).astype(np.int32)
    Gc = orc.normal(touched.size * group, 6, 8, 1e-3)
    gs = np.array([0.81], f32)
    sref = float(np.mean(s.astype(np.float64)))
    dd, dr, dm8, dv8, dm8s, dv8s = dev(d), dev(r), dev(m8), dev(v8), dev(m8s), dev(v8s)
    P = torch.zeros(nt, device="cuda")
    q.step_touched(P, dev(Gc), dd, dr, dev(s), dm8, dm8s, dv8, dv8s, dev(touched), touched.size, group, dmax,
                   3e-4, 0.9, 0.95, 0.1, sref, 10.0, 4.47, 7, nt, dev(gs), v4)
    torch.cuda.synchronize()
    Ph = np.zeros(nt, f32)
    orc.step_touched(Ph, Gc, d, r, s, m8, m8s, v8, v8s, touched, group, dmax, 3e-4, 0.9, 0.95, 0.1, sref, 10.0, 4.47,
                     7, nt, gs, v4)
    for got, want in ((dd, d), (dr, r), (dm8, m8), (dv8, v8), (dm8s, m8s), (dv8s, v8s), (P, Ph)):
        assert beq(got, want)


def test_sqsum_gnorm_and_clipped_step(q, orc, golden):
    """k_sqsum / k_gnorm (cudalm.cu:2794-2816 with the CPU kernels' definition, cpu_kern.h:533-546): the 64
    partial sums against the reference fixture and the oracle (the double additions run in another
    order on the GPU: at most one float ulp), the clip pair from the same partials bit for bit, and a step
    that reads its clip multiplier from the device equal to the oracle's step with that multiplier."""
    import torch
    g = golden("gnorm")
    parts = []
    for k in range(3):
        G = orc.normal(int(g["n%d" % k][0]), 0, int(g["seed%d" % k][0]), float(g["scale%d" % k][0]))
        part = torch.zeros(64, device="cuda")
        q.sqsum(dev(G), G.size, part)
        got = host(part)
        ulps = np.abs(got.view(np.int32).astype(np.int64) - g["part%d" % k].view(np.int32).astype(np.int64)).max()
        assert ulps <= 1, (k, ulps)
        parts.append(got)
    side = np.concatenate([parts[2], parts[1], parts[0]])
    gs = torch.zeros(2, device="cuda")
    for cs in (0, 1):
        q.gnorm(dev(side), 2, cs, gs)
        assert np.array_equal(host(gs).view(np.uint32), orc.gnorm(side, 2, cs).view(np.uint32))
    bad = side.copy(); bad[70] = np.inf
    q.gnorm(dev(bad), 2, 0, gs)
    assert np.isnan(host(gs)[1]) and host(gs)[0] == 1.0
    # a step clipped through the device scalar
    group, dmax = 128, 7
    tab, nq, ng = make_spans([128 * 300 + 40], group)
    tab["sref"] = [0.0088]
    hd = orc.digits(nq, 5, 20); hr = orc.int8(nq, 5, 21, -64, 64); hm8 = orc.int8(nq, 5, 22, -127, 127); hv8 = orc.u8(nq, 5, 23, 0, 255)
    hs = orc.uniform(ng, 5, 24, 0.5, 1.5) * f32(0.02 * 3 / 7)
    hm8s = orc.uniform(ng, 5, 25, 0.5, 1.5) * f32(3e-3 / 127); hv8s = orc.uniform(ng, 5, 26, 0.5, 1.5) * f32(3e-3 / 255)
    hG = orc.normal(nq, 5, 27, 0.05)                                   # norm well above 1
    d, r, m8, v8, s, m8s, v8s, G = (dev(x) for x in (hd, hr, hm8, hv8, hs, hm8s, hv8s, hG))
    part = torch.zeros(64, device="cuda")
    q.sqsum(G, nq, part); q.gnorm(part, 0, 0, gs)
    hgs = host(gs)
    assert hgs[1] > 1.0 and hgs[0] == f32(1.0) / hgs[1]
    hp = lambda gsp: (3e-4, 0.9, 0.95, 0.1, 1.0, gsp, 10.0, 4.4721, 0, 1, 1, None, 1, 0, ng)
    q.step(None, G, d, r, s, m8, m8s, v8, v8s, dev(tab), 1, group, dmax, *hp(gs))
    orc.step(None, hG, hd, hr, hs, hm8, hm8s, hv8, hv8s, tab, group, dmax, *hp(hgs[:1].copy()))
    for got, want, nm in [(d, hd, "d"), (r, hr, "r"), (m8, hm8, "m8"), (v8, hv8, "v8"), (m8s, hm8s, "m8s"), (v8s, hv8s, "v8s")]:
        assert beq(got, want), nm


def test_short_sqrt_form_equals_sqrtf_on_every_float_it_serves(q):
    """The step's square root of the second moment is v_sqrt_f32 plus the two neighbour tests of the compiler's own
    sqrtf expansion, without that expansion's subnormal rescaling; it is used for arguments >= 2^-96. Exhaustive:
    all 1,879,048,193 bit patterns from 2^-96 to +infinity give the bits sqrtf gives."""
    import torch
    bad = torch.zeros(1, dtype=torch.int64, device="cuda")
    first, last = 0x0F800000, 0x7F800000
    q.call("qlmx_test_sqrt_form", first, last - first + 1, bad, None)
    torch.cuda.synchronize()
    assert int(bad.item()) == 0


def test_step_zero_and_tiny_second_moments_take_the_general_square_root(q, orc):
    """Groups whose gradient and second moment are exactly zero, or so small that the new second moment is a
    subnormal number, sit below the short form's bound; whole wavefronts then take sqrtf. Bytes equal the oracle."""
    import torch
    group, dmax = 128, 7
    tab, nq, ng = make_spans([128 * 64], group)
    tab["sref"] = [0.0086]
    hd = orc.digits(nq, 9, 20); hr = orc.int8(nq, 9, 21, -64, 64); hm8 = orc.int8(nq, 9, 22, -127, 127)
    hv8 = orc.u8(nq, 9, 23, 0, 255)
    hs = orc.uniform(ng, 9, 24, 0.5, 1.5) * f32(0.02 * 3 / 7)
    hm8s = orc.uniform(ng, 9, 25, 0.5, 1.5) * f32(3e-3 / 127); hv8s = orc.uniform(ng, 9, 26, 0.5, 1.5) * f32(3e-3 / 255)
    hG = orc.normal(nq, 9, 27, 1e-3)
    hG[:128 * 8] = 0.0; hv8[:128 * 8] = 0                      # exact zeros: vv = 0
    hG[128 * 8:128 * 16] *= f32(1e-22); hv8[128 * 8:128 * 16] = 0    # gr^2 * 0.05 ~ 1e-51: subnormal / underflowing
    hG[128 * 16:128 * 17] *= f32(1e-18); hv8s[16] = f32(1e-20)       # tiny but mixed with a live v8
    hv8[128 * 20 + 5] = 0; hG[128 * 20 + 5] = 0.0                    # one zero element in an ordinary group
    d, r, m8, v8, s, m8s, v8s, G = (dev(x) for x in (hd, hr, hm8, hv8, hs, hm8s, hv8s, hG))
    for t in (1, 2):
        hp = (3e-4, 0.9, 0.95, 0.1, 1.0, None, 10.0, 4.4721, 0, t, 1, None, 1, 0, ng)
        q.step(None, G, d, r, s, m8, m8s, v8, v8s, dev(tab), 1, group, dmax, *hp)
        orc.step(None, hG, hd, hr, hs, hm8, hm8s, hv8, hv8s, tab, group, dmax, *hp)
    for got, want, nm in [(d, hd, "d"), (r, hr, "r"), (m8, hm8, "m8"), (v8, hv8, "v8"), (m8s, hm8s, "m8s"), (v8s, hv8s, "v8s")]:
        assert beq(got, want), nm


def test_step_short_division_equals_the_full_one(q):
    """The step's mid-range division (no scaling, no special-case fix-up) gives the bits of `/` on 2^33 pseudo-random
    operand pairs with magnitudes in [2^-40, 2^40], and an exact zero for a zero dividend."""
    import torch
    bad = torch.zeros(1, dtype=torch.int64, device="cuda")
    q.call("qlmx_test_div_form", 12345, 1 << 33, bad, None)
    torch.cuda.synchronize()
    assert int(bad.item()) == 0


@pytest.mark.parametrize("v4,render,inv_sqrt_bc2", [(0, False, 4.4721), (1, True, 4.4721), (0, True, 2000.0)])
def test_step_operands_at_the_edges_of_the_mid_range_forms(q, orc, v4, render, inv_sqrt_bc2):
    """Groups built to sit on either side of every guard of the step's mid-range forms (whole wavefronts of four groups
    each, and single elements inside ordinary groups): first moments that are exactly zero, tiny (below 2^-40 after
    the bias correction) and huge, gradients that put the second moment's root above 2^25, a stored second-moment
    scale above 2^20, a group whose largest first moment is below 2^-32, and -- third case -- an inverse bias
    correction outside the range the host admits. Two steps; every byte equals the oracle, with and without the
    fp32 view and in the fourth-root form."""
    import torch
    group, dmax = 128, 7
    tab, nq, ng = make_spans([128 * 96], group)
    tab["sref"] = [0.0086]
    hd = orc.digits(nq, 11, 20); hr = orc.int8(nq, 11, 21, -64, 64); hm8 = orc.int8(nq, 11, 22, -127, 127)
    hv8 = orc.u8(nq, 11, 23, 1, 255)
    hs = orc.uniform(ng, 11, 24, 0.5, 1.5) * f32(0.02 * 3 / 7)
    hm8s = orc.uniform(ng, 11, 25, 0.5, 1.5) * f32(3e-3 / 127); hv8s = orc.uniform(ng, 11, 26, 0.5, 1.5) * f32(3e-3 / 255)
    hG = orc.normal(nq, 11, 27, 1e-3)
    g = lambda a, b: slice(128 * a, 128 * b)
    hG[g(0, 4)] = 0.0; hm8[g(0, 4)] = 0                             # first moment exactly zero, second moment live
    hG[g(8, 12)] *= f32(1e-12); hm8[g(8, 12)] = 0                   # |m| ~ 1e-16: below 2^-40
    hG[g(16, 20)] *= f32(1e9)                                        # sqrt(v) ~ 2e5, m ~ 1e5: inside
    hG[g(24, 28)] *= f32(1e13)                                       # sqrt(v) ~ 2e9 > 2^25, m ~ 1e9
    hG[g(32, 36)] *= f32(1e17)                                       # m * inv_bc1 > 2^40
    hv8s[40:44] = f32(3e6)                                           # eps = stored scale > 2^20
    hG[g(48, 52)] *= f32(1e-8); hm8[g(48, 52)] = 0; hv8[g(48, 52)] = 200    # largest |m| of a lane below 2^-32
    hG[128 * 60 + 7] = 0.0; hm8[128 * 60 + 7] = 0                    # single zero first moment in an ordinary group
    hG[128 * 64 + 9] = f32(1e-15); hm8[128 * 64 + 9] = 0             # single tiny one
    hG[128 * 68 + 3] = f32(5e7)                                      # single huge one
    hm8[g(72, 76)] = 127; hG[g(72, 76)] = f32(2e-3)                  # every quotient of the requantisation at the rail
    P = torch.zeros(nq, device="cuda") if render else None
    hP = np.zeros(nq, f32) if render else None
    d, r, m8, v8, s, m8s, v8s, G = (dev(x) for x in (hd, hr, hm8, hv8, hs, hm8s, hv8s, hG))
    for t in (1, 2):
        hp = (3e-4, 0.9, 0.95, 0.1, 1.0, None, 10.0, inv_sqrt_bc2, 0, t, 1, None, 1, 0, ng)
        q.step(P, G, d, r, s, m8, m8s, v8, v8s, dev(tab), 1, group, dmax, *hp, v4)
        orc.step(hP, hG, hd, hr, hs, hm8, hm8s, hv8, hv8s, tab, group, dmax, *hp, v4)
    pairs = [(d, hd, "d"), (r, hr, "r"), (m8, hm8, "m8"), (v8, hv8, "v8"), (m8s, hm8s, "m8s"), (v8s, hv8s, "v8s")]
    if render:
        pairs.append((P, hP, "P"))
    for got, want, nm in pairs:
        assert beq(got, want), nm


@pytest.mark.parametrize("v4,render", [(0, False), (1, True)])
def test_step_eight_groups_per_wavefront_equals_one_per_row(q, orc, v4, render):
    """The training step's kernel (eight groups per wavefront, 16 weights per lane) against the general one (a group
    per row of 16 lanes) and the oracle: two spans, the first with a short last group in the middle of a wavefront, a
    shifted gradient offset on the second, a group count that is no multiple of 8, and a sub-range launch that starts
    inside a wavefront's worth of groups; three steps, every byte."""
    import torch
    group, dmax = 128, 7
    tab, nq, ng = make_spans([128 * 203 + 40, 128 * 118], group)
    tab[1]["gof"] = tab[1]["pof"] + 8
    tab["sref"] = [0.0086, 0.0091]
    npar = nq + 8
    st0 = dict(hd=orc.digits(nq, 31, 20), hr=orc.int8(nq, 31, 21, -64, 64), hm8=orc.int8(nq, 31, 22, -127, 127), hv8=orc.u8(nq, 31, 23, 1, 255),
               hs=orc.uniform(ng, 31, 24, 0.5, 1.5) * f32(0.02 * 3 / 7), hm8s=orc.uniform(ng, 31, 25, 0.5, 1.5) * f32(3e-3 / 127),
               hv8s=orc.uniform(ng, 31, 26, 0.5, 1.5) * f32(3e-3 / 255))
    grads = [orc.normal(npar, 31, 30 + t, 1e-3) for t in range(1, 4)]
    ranges = [(0, ng), (5, ng - 11), (0, ng)]                 # the second step over a sub-range
    results = []
    for wide in (1, 0):
        q.call("qlmx_test_step_wide", wide)
        try:
            d, r, m8, v8, s, m8s, v8s = (dev(st0[k].copy()) for k in ("hd", "hr", "hm8", "hv8", "hs", "hm8s", "hv8s"))
            P = torch.zeros(npar, device="cuda") if render else None
            for t in range(1, 4):
                bc1 = f32(1) - f32(0.9) ** f32(t); bc2 = f32(1) - f32(0.95) ** f32(t)
                hp = (3e-4, 0.9, 0.95, 0.1, 1.0, None, float(f32(1) / bc1), float(f32(1) / np.sqrt(bc2)), 0, t, 1, None, 1) + ranges[t - 1]
                q.step(P, dev(grads[t - 1]), d, r, s, m8, m8s, v8, v8s, dev(tab), 2, group, dmax, *hp, v4)
            results.append([host(x) for x in (d, r, m8, v8, m8s, v8s)] + ([host(P)] if render else []))
        finally:
            q.call("qlmx_test_step_wide", 1)
    h = {k: v.copy() for k, v in st0.items()}
    hP = np.zeros(npar, f32) if render else None
    for t in range(1, 4):
        bc1 = f32(1) - f32(0.9) ** f32(t); bc2 = f32(1) - f32(0.95) ** f32(t)
        hp = (3e-4, 0.9, 0.95, 0.1, 1.0, None, float(f32(1) / bc1), float(f32(1) / np.sqrt(bc2)), 0, t, 1, None, 1) + ranges[t - 1]
        orc.step(hP, grads[t - 1], h["hd"], h["hr"], h["hs"], h["hm8"], h["hm8s"], h["hv8"], h["hv8s"], tab, group, dmax, *hp, v4)
    want = [h["hd"], h["hr"], h["hm8"], h["hv8"], h["hm8s"], h["hv8s"]] + ([hP] if render else [])
    for i, nm in enumerate(["d", "r", "m8", "v8", "m8s", "v8s"] + (["P"] if render else [])):
        assert np.array_equal(results[0][i].view(np.uint8), results[1][i].view(np.uint8)), nm
        assert np.array_equal(results[0][i].view(np.uint8), np.asarray(want[i]).view(np.uint8)), nm


def test_argument_errors(q):
    import torch
    x = torch.zeros(256, device="cuda")
    with pytest.raises(pkg.QlmxError, match="group"):
        q.render(x, x, x, x, 1, 1000, 1, 0, 1)
    with pytest.raises(pkg.QlmxError, match="packed"):
        q.encode(x, x, x, x, x, 1, 128, 127, 1, 1)
    with pytest.raises(pkg.QlmxError, match="NULL"):
        q.servo(None, x, x, x, 1, 128, 7, 0.1, 0.01, 1, 1)
