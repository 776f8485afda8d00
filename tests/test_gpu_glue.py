"""GPU parity of the MoE glue (router, grouping permutation, gather / scatter, gate gradient, SwiGLU)
and of a whole expert-FFN layer -- forward and backward -- put together from the library's entry
points, against the CPU oracle (orc_moe_forward / orc_moe_backward follow cudalm.cu:4193-4228 and
4299-4371) and the fixtures written by the compiled reference.

Bars: indices (assign, perm, off), gate probabilities and every pure data move are bit-exact; SwiGLU
and the dot product of the gate gradient follow the oracle to 1e-6 relative L2; layer outputs to 1e-5
with the fp32 GEMMs. With the bf16 MFMA GEMMs each GEMM meets 1e-3 on equal inputs (tested with the
GEMMs); the whole layer, whose GEMM inputs are then stored as bf16, meets 1e-3 against the oracle's layer
with the same five buffers rounded to bf16, and 4e-3 against the all-fp32 layer."""
import numpy as np
import pytest

from __graft_entry__ import load_package
from oracle.binding import make_spans

pkg = load_package()
f32 = np.float32
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def q():
    return pkg.load()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def zeros(n, dtype=None):
    import torch
    return torch.zeros(n, dtype=dtype or torch.float32, device="cuda")


def bf16_to_f32(t):
    """int16 tensor of bf16 bit patterns -> fp32 numpy"""
    import torch
    return (t.to(torch.int32) << 16).view(torch.float32).cpu().numpy()


# ------------------------------------------------------------------ router
@pytest.mark.parametrize("tag", ["a", "b", "c"])
def test_router_vs_reference_fixture(q, golden, tag):
    import torch
    g = golden("router")
    N, E, K = (int(v) for v in g["dims_" + tag])
    pr, asn, gate = zeros(N * E), zeros(K * N, torch.int32), zeros(K * N)
    q.router_topk(dev(g["rt_" + tag]), pr, asn, gate, N, E, K)
    torch.cuda.synchronize()
    assert np.array_equal(asn.cpu().numpy(), g["asn_" + tag])
    assert np.array_equal(gate.cpu().numpy().view(np.uint32), g["gate_" + tag].view(np.uint32))
    assert np.array_equal(pr.cpu().numpy().view(np.uint32), g["pr_" + tag].view(np.uint32))


def test_router_bias_vs_reference_fixture(q, golden):
    import torch
    g = golden("router")
    N, E, K = (int(v) for v in g["dims_a"])
    pr, asn, gate = zeros(N * E), zeros(K * N, torch.int32), zeros(K * N)
    q.router_topk(dev(g["rt_a"]), pr, asn, gate, N, E, K, dev(g["bias"]), E)
    torch.cuda.synchronize()
    assert np.array_equal(asn.cpu().numpy(), g["asn_bias"])
    assert np.array_equal(gate.cpu().numpy().view(np.uint32), g["gate_bias"].view(np.uint32))


def test_router_training_size_vs_oracle(q, orc):
    """8192 tokens x 32 experts, logits quantised to 1/8 so that many exact ties occur."""
    import torch
    N, E, K = 8192, 32, 2
    rt = np.round(orc.normal(N * E, 3, 1, 2.0) * 8).astype(f32) / 8
    want_pr = np.zeros(N * E, f32); want_asn = np.zeros(K * N, np.int32); want_gate = np.zeros(K * N, f32)
    orc.router_topk(rt, want_pr, want_asn, want_gate, N, E, K)
    pr, asn, gate = zeros(N * E), zeros(K * N, torch.int32), zeros(K * N)
    q.router_topk(dev(rt), pr, asn, gate, N, E, K)
    torch.cuda.synchronize()
    assert np.array_equal(asn.cpu().numpy(), want_asn)
    assert np.array_equal(gate.cpu().numpy().view(np.uint32), want_gate.view(np.uint32))
    assert np.array_equal(pr.cpu().numpy().view(np.uint32), want_pr.view(np.uint32))


@pytest.mark.parametrize("N,E,K,with_bias", [(1000, 64, 4, False), (77, 5, 2, True), (130, 96, 8, False), (65, 97, 3, True),
                                              (300, 7, 7, False), (1, 32, 2, False), (515, 32, 8, True), (200, 16, 3, False), (129, 8, 8, True)])
def test_router_shapes_vs_oracle(q, orc, N, E, K, with_bias):
    """Expert counts served by the register kernel (8, 16, 32, 64), by the LDS-staged one and beyond its
    limit, odd counts, token counts off the workgroup size, K up to its maximum, per-pass bias:
    bit-identical to the CPU oracle."""
    import torch
    rt = np.round(orc.normal(N * E, 5, N + E, 2.0) * 16).astype(f32) / 16
    bias = (orc.normal(K * E, 5, 7, 0.01) if with_bias else None)
    want_pr = np.zeros(N * E, f32); want_asn = np.zeros(K * N, np.int32); want_gate = np.zeros(K * N, f32)
    orc.router_topk(rt, want_pr, want_asn, want_gate, N, E, K, bias, E if with_bias else 0)
    pr, asn, gate = zeros(N * E), zeros(K * N, torch.int32), zeros(K * N)
    q.router_topk(dev(rt), pr, asn, gate, N, E, K, dev(bias) if with_bias else None, E if with_bias else 0)
    torch.cuda.synchronize()
    assert np.array_equal(asn.cpu().numpy(), want_asn)
    assert np.array_equal(gate.cpu().numpy().view(np.uint32), want_gate.view(np.uint32))
    assert np.array_equal(pr.cpu().numpy().view(np.uint32), want_pr.view(np.uint32))


def test_router_limits(q):
    z = zeros(64)
    with pytest.raises(pkg.QlmxError, match="K"):
        q.router_topk(z, z, z, z, 4, 4, 9)


# ------------------------------------------------------------------ permutation
def gpu_perm(q, asn, N, E, K):
    import torch
    ws = torch.zeros(q.moe_perm_workspace(N, E, K), dtype=torch.uint8, device="cuda")
    perm, off = zeros(K * N, torch.int32), zeros(K * (E + 1), torch.int32)
    q.moe_perm(dev(asn), N, E, K, perm, off, ws)
    q.moe_perm_status(ws, N, E, K)
    return perm.cpu().numpy(), off.cpu().numpy(), ws


@pytest.mark.parametrize("N,E,K", [(1, 1, 1), (50, 3, 2), (256, 8, 1), (257, 8, 3), (1000, 64, 4), (8192, 32, 2), (5000, 300, 2), (40000, 70, 2)])
def test_perm_vs_oracle(q, orc, N, E, K):
    rng = np.random.default_rng(N * 31 + E)
    p = (np.arange(E) + 1.0) ** -1.1; p /= p.sum()
    asn = rng.choice(E, size=K * N, p=p).astype(np.int32)
    if E > 2:
        asn[asn == 1] = 0                                # an expert nobody picks
    perm, off, _ = gpu_perm(q, asn, N, E, K)
    for k in range(K):
        wp = np.zeros(N, np.int32); wo = np.zeros(E + 1, np.int32)
        assert orc.moe_perm(asn[k * N:(k + 1) * N], N, E, wp, wo) == 0
        assert np.array_equal(off[k * (E + 1):(k + 1) * (E + 1)], wo)
        assert np.array_equal(perm[k * N:(k + 1) * N], wp)


def test_perm_workspace_reused(q, orc):
    """The same workspace serves one call after another (its counters are cleared by each call)."""
    import torch
    N, E, K = 3000, 16, 2
    ws = torch.zeros(q.moe_perm_workspace(N, E, K), dtype=torch.uint8, device="cuda")
    for seed in (1, 2, 3):
        asn = np.random.default_rng(seed).integers(0, E, K * N).astype(np.int32)
        perm, off = zeros(K * N, torch.int32), zeros(K * (E + 1), torch.int32)
        q.moe_perm(dev(asn), N, E, K, perm, off, ws)
        q.moe_perm_status(ws, N, E, K)
        for k in range(K):
            wp = np.zeros(N, np.int32); wo = np.zeros(E + 1, np.int32)
            assert orc.moe_perm(asn[k * N:(k + 1) * N], N, E, wp, wo) == 0
            assert np.array_equal(off.cpu().numpy()[k * (E + 1):(k + 1) * (E + 1)], wo)
            assert np.array_equal(perm.cpu().numpy()[k * N:(k + 1) * N], wp)


def test_perm_reports_bad_expert(q):
    asn = np.array([0, 1, 9, 2], np.int32)
    with pytest.raises(pkg.QlmxError, match="out of range"):
        gpu_perm(q, asn, 4, 4, 1)


# ------------------------------------------------------------------ row movers, dgate, swiglu
def test_glue_vs_reference_fixture(q, golden):
    import torch
    g = golden("glue")
    N, D = (int(v) for v in g["dims"])
    perm, gate = dev(g["perm"]), dev(g["gate"])
    Xp = zeros(N * D)
    q.moe_gather(dev(g["src"]), perm, Xp, N, D)
    sg = dev(g["out0"].copy()); q.moe_scatter_gate(Xp, perm, gate, sg, N, D)
    sa = dev(g["out0"].copy()); q.moe_scatter_add(Xp, perm, sa, N, D)
    dgate, dyp = zeros(N), zeros(N * D)
    q.moe_dgate(dev(g["dout"]), Xp, perm, gate, dgate, dyp, N, D)
    n = (g["G"].size // 4) * 4
    O, dg, du = zeros(n), zeros(n), zeros(n)
    G, U, dA = dev(g["G"][:n]), dev(g["U"][:n]), dev(g["dA"][:n])
    q.swiglu(G, U, O, n)
    q.swiglu_bwd(G, U, dA, dg, du, n)
    torch.cuda.synchronize()
    bits = lambda a: np.ascontiguousarray(a).view(np.uint32)
    assert np.array_equal(bits(Xp.cpu().numpy()), bits(g["Xp"]))
    assert np.array_equal(bits(sg.cpu().numpy()), bits(g["sg"]))
    assert np.array_equal(bits(sa.cpu().numpy()), bits(g["sa"]))
    assert np.array_equal(bits(dyp.cpu().numpy()), bits(g["dyp"]))
    rel = lambda a, b: float(np.linalg.norm(a.astype(np.float64) - b) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))
    assert rel(dgate.cpu().numpy(), g["dgate"]) < 1e-6
    # the reference's CPU sigmoid uses explicit FMA intrinsics (cpu_kern.h:37-50): tolerance, not bits
    assert rel(O.cpu().numpy(), g["O"][:n]) < 1e-6
    assert rel(dg.cpu().numpy(), g["dg"][:n]) < 1e-6
    assert rel(du.cpu().numpy(), g["du"][:n]) < 1e-6


def test_glue_negative_perm_and_bf16_outputs(q, orc):
    import torch
    N, D = 37, 64
    src = orc.normal(N * D, 2, 1)
    perm = np.arange(N, dtype=np.int32)[::-1].copy(); perm[5] = -1; perm[20] = -1
    want = np.zeros(N * D, f32); orc.gather(src, perm, want, N, D)
    Xp = zeros(N * D); q.moe_gather(dev(src), dev(perm), Xp, N, D)
    Xb = zeros(N * D, torch.int16); q.moe_gather(dev(src), dev(perm), Xb, N, D, pkg.ACT_BF16)
    torch.cuda.synchronize()
    assert np.array_equal(Xp.cpu().numpy(), want)
    assert np.array_equal(bf16_to_f32(Xb), orc.bf16_round(want))
    n = 4096
    G, U = orc.normal(n, 2, 2, 2.0), orc.normal(n, 2, 3)
    wantO = np.zeros(n, f32); orc.swiglu(G, U, wantO)
    Ob = zeros(n, torch.int16); q.swiglu(dev(G), dev(U), Ob, n, pkg.ACT_BF16)
    Of = zeros(n); q.swiglu(dev(G), dev(U), Of, n)
    torch.cuda.synchronize()
    assert np.array_equal(Of.cpu().numpy().view(np.uint32), wantO.view(np.uint32))      # same operations as the oracle
    assert np.array_equal(bf16_to_f32(Ob), orc.bf16_round(wantO))


# ------------------------------------------------------------------ a whole layer from the entry points
def encode_layer(orc, seed, E, D, F, group=128):
    n = E * D * F
    tab, nq, ng = make_spans([n, n, n], group)
    P = np.concatenate([orc.normal(n, seed, 1, 0.02), orc.normal(n, seed, 2, 0.02), orc.normal(n, seed, 3, 0.02)])
    d = np.zeros(nq // 2, np.int8); r = np.zeros(nq, np.int8); s = np.zeros(ng, f32)
    orc.encode(P, d, r, s, tab, group, 7, 1, ng)
    orc.render(P, d, s, tab, group, 1, 0, ng)
    return d, s, P, n


class GpuLayer:
    """moe_forward / moe_backward (cudalm.cu:4193-4228, 4299-4371, stash off) on the library's entry
    points; the only host step is reading the expert row counts to size the grouped GEMM calls, which
    the reference does as well (cudalm.cu:3576-3602)."""

    def __init__(self, q, dd, ds, n, N, D, F, E, K, math, group=128):
        import torch
        self.q, self.dd, self.ds, self.n, self.N, self.D, self.F, self.E, self.K, self.math, self.group = q, dd, ds, n, N, D, F, E, K, math, group
        self.act = pkg.ACT_BF16 if math == pkg.MATH_MFMA else pkg.ACT_F32
        self.esz = 2 if math == pkg.MATH_MFMA else 4
        adt = torch.int16 if math == pkg.MATH_MFMA else torch.float32
        self.ws = torch.zeros(q.moe_perm_workspace(N, E, K), dtype=torch.uint8, device="cuda")
        self.perm, self.off = zeros(K * N, torch.int32), zeros(K * (E + 1), torch.int32)
        self.Xp, self.ap = zeros(N * D, adt), zeros(N * F, adt)
        self.gp, self.up, self.yp = zeros(N * F), zeros(N * F), zeros(N * D)
        self.dyp, self.dgp, self.dup = zeros(N * D, adt), zeros(N * F, adt), zeros(N * F, adt)
        self.dap, self.dXp = zeros(N * F), zeros(N * D)

    def group_tokens(self, assign):
        q = self.q
        q.moe_perm(assign, self.N, self.E, self.K, self.perm, self.off, self.ws)
        q.moe_perm_status(self.ws, self.N, self.E, self.K)
        self.offh = self.off.cpu().numpy().reshape(self.K, self.E + 1)

    def probs(self, k, A, a_cols, a_esz, C, c_cols, wbase, B=None, b_cols=0, b_esz=0, beta=0.0, out_expert=False):
        off = self.offh[k]; DF = self.D * self.F
        items = []
        for e in range(self.E):
            ne = int(off[e + 1] - off[e])
            a = A.data_ptr() + int(off[e]) * a_cols * a_esz
            b = None if B is None else B.data_ptr() + int(off[e]) * b_cols * b_esz
            c = C.data_ptr() + (e * DF * 4 if out_expert else int(off[e]) * c_cols * 4)
            wq = wbase + e * DF
            items.append((a, b, c, wq, wq // self.group, ne, beta))
        return self.q.problems(items)

    def experts_fwd(self, k):
        q, D, F, E, n = self.q, self.D, self.F, self.E, self.n
        q.gemm_nn(self.dd, self.ds, self.group, self.probs(k, self.Xp, D, self.esz, self.gp, F, 0), E, D, F, self.act, self.math)
        q.gemm_nn(self.dd, self.ds, self.group, self.probs(k, self.Xp, D, self.esz, self.up, F, n), E, D, F, self.act, self.math)
        q.swiglu(self.gp, self.up, self.ap, self.N * F, self.act)
        q.gemm_nn(self.dd, self.ds, self.group, self.probs(k, self.ap, F, self.esz, self.yp, D, 2 * n), E, F, D, self.act, self.math)

    def forward(self, x, assign, gate, out):
        q, N, D = self.q, self.N, self.D
        self.group_tokens(assign)
        for k in range(self.K):
            prm = self.perm[k * N:(k + 1) * N]
            q.moe_gather(x, prm, self.Xp, N, D, self.act)
            self.experts_fwd(k)
            q.moe_scatter_gate(self.yp, prm, gate[k * N:(k + 1) * N], out, N, D)

    def backward(self, x, gate, dout, dx, dgate, Gw1, Gw3, Gw2):
        q, N, D, F, E, n = self.q, self.N, self.D, self.F, self.E, self.n
        dx.zero_()
        for k in range(self.K):
            prm = self.perm[k * N:(k + 1) * N]
            q.moe_gather(x, prm, self.Xp, N, D, self.act)
            self.experts_fwd(k)
            q.moe_dgate(dout, self.yp, prm, gate[k * N:(k + 1) * N], dgate[k * N:(k + 1) * N], self.dyp, N, D, self.act)
            q.gemm_nt(self.probs(k, self.ap, F, self.esz, Gw2, 0, 0, B=self.dyp, b_cols=D, b_esz=self.esz, beta=1.0, out_expert=True), E, F, D, self.act, self.math)
            q.gemm_tn(self.dd, self.ds, self.group, self.probs(k, self.dyp, D, self.esz, self.dap, F, 2 * n), E, D, F, self.act, self.math)
            q.swiglu_bwd(self.gp, self.up, self.dap, self.dgp, self.dup, N * F, self.act)
            q.gemm_nt(self.probs(k, self.Xp, D, self.esz, Gw1, 0, 0, B=self.dgp, b_cols=F, b_esz=self.esz, beta=1.0, out_expert=True), E, D, F, self.act, self.math)
            q.gemm_nt(self.probs(k, self.Xp, D, self.esz, Gw3, 0, 0, B=self.dup, b_cols=F, b_esz=self.esz, beta=1.0, out_expert=True), E, D, F, self.act, self.math)
            q.gemm_tn(self.dd, self.ds, self.group, self.probs(k, self.dgp, F, self.esz, self.dXp, D, 0), E, F, D, self.act, self.math)
            q.gemm_tn(self.dd, self.ds, self.group, self.probs(k, self.dup, F, self.esz, self.dXp, D, n, beta=1.0), E, F, D, self.act, self.math)
            q.moe_scatter_add(self.dXp, prm, dx, N, D)


class GpuLayerFused:
    """The same layer from the fused entry points, bf16 activations: fp16 forward GEMMs with gather and SwiGLU folded
    in, gated scatter behind w2, SwiGLU gradient behind the down projection's input gradient, scatter-add behind the
    paired input gradient. merged = False: pass after pass, as moe_forward / moe_backward loop (cudalm.cu:4193-4228,
    4299-4371). merged = True: all K passes as one expert-grouped list of K*N rows (cudalm.cu:3532-3561, 4048-4110),
    every GEMM once per layer, the passes' contributions combined per token in pass order."""

    def __init__(self, q, dd, ds, n, N, D, F, E, K, merged, group=128):
        import torch
        self.q, self.dd, self.ds, self.n, self.N, self.D, self.F, self.E, self.K, self.merged, self.group = q, dd, ds, n, N, D, F, E, K, merged, group
        R = K * N if merged else N                                   # rows of the grouped buffers
        self.R, self.P = R, (1 if merged else K)                     # and how many grouped lists there are
        self.ws = torch.zeros(q.moe_perm_workspace(R, E, self.P), dtype=torch.uint8, device="cuda")
        self.perm, self.off = zeros(K * N, torch.int32), zeros(self.P * (E + 1), torch.int32)
        self.tok, self.inv = zeros(K * N, torch.int32), zeros(K * N, torch.int32)
        i16 = torch.int16
        self.xb, self.Xp, self.ap = zeros(N * D, i16), zeros(R * D, i16), zeros(R * F, i16)
        self.gp, self.up, self.yp = zeros(R * F), zeros(R * F), zeros(R * D)
        self.dyp, self.dgp, self.dup = zeros(R * D, i16), zeros(R * F, i16), zeros(R * F, i16)
        self.dXp = zeros(R * D)
        self.ident = dev(np.arange(N, dtype=np.int32))

    def group_tokens(self, assign):
        q = self.q
        q.moe_perm(assign, self.R, self.E, self.P, self.perm, self.off, self.ws)
        q.moe_perm_status(self.ws, self.R, self.E, self.P)
        self.offh = self.off.cpu().numpy().reshape(self.P, self.E + 1)
        if self.merged:
            q.moe_merge_rows(self.perm, self.N, self.K, self.tok, self.inv)
        else:
            self.tok = self.perm                                     # a pass's entries are the tokens themselves

    def probs(self, k, A, a_cols, C, c_cols, wbase, B=None, b_cols=0, beta=0.0, out_expert=False, idx_a=False, idx_c=False):
        off = self.offh[k]; DF = self.D * self.F
        items = []
        for e in range(self.E):
            ne, o = int(off[e + 1] - off[e]), int(off[e])
            a = self.tok.data_ptr() + (k * self.R + o) * 4 if idx_a else A.data_ptr() + o * a_cols * 2
            b = None if B is None else B.data_ptr() + o * b_cols * 2
            if idx_c:        c = self.tok.data_ptr() + (k * self.R + o) * 4
            elif C is None:  c = None
            else:            c = C.data_ptr() + (e * DF * 4 if out_expert else o * c_cols * 4)
            wq = wbase + e * DF
            items.append((a, b, c, wq, wq // self.group, ne, beta))
        return self.q.problems(items)

    def forward(self, x, assign, gate, out):
        q, N, D, F, E, K, n, R = self.q, self.N, self.D, self.F, self.E, self.K, self.n, self.R
        self.group_tokens(assign)
        q.moe_gather(x, self.ident, self.xb, N, D, pkg.ACT_BF16)                       # the token matrix as bf16, once
        for k in range(self.P):
            q.gemm_nn_gather_swiglu(self.dd, self.ds, self.group, self.probs(k, None, 0, None, 0, 0, idx_a=True),
                                    self.probs(k, self.Xp, D, None, 0, n, B=self.ap, b_cols=F), E, D, F, self.xb)
            if self.merged:
                q.gemm_nn(self.dd, self.ds, self.group, self.probs(k, self.ap, F, self.yp, D, 2 * n), E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA_F16)
                q.moe_combine(self.yp, self.inv, gate, out, N, K, D)
            else:
                q.gemm_nn_scatter(self.dd, self.ds, self.group, self.probs(k, self.ap, F, None, 0, 2 * n, idx_c=True), E, F, D, out, gate[k * N:(k + 1) * N])

    def backward(self, x, gate, dout, dx, dgate, Gw1, Gw3, Gw2):
        q, N, D, F, E, K, n, R = self.q, self.N, self.D, self.F, self.E, self.K, self.n, self.R
        dx.zero_()
        for k in range(self.P):
            tok = self.tok[k * R:(k + 1) * R]
            q.moe_gather(x, tok, self.Xp, R, D, pkg.ACT_BF16)                          # the weight gradient reads the grouped rows
            q.gemm_nn_swiglu(self.dd, self.ds, self.group, self.probs(k, self.Xp, D, self.gp, F, 0),
                             self.probs(k, self.Xp, D, self.up, F, n, B=self.ap, b_cols=F), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA_F16)
            q.gemm_nn(self.dd, self.ds, self.group, self.probs(k, self.ap, F, self.yp, D, 2 * n), E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA_F16)
            if self.merged: q.moe_dgate_merged(dout, self.yp, self.perm, gate, dgate, self.dyp, N, K, D, pkg.ACT_BF16)
            else:           q.moe_dgate(dout, self.yp, tok, gate[k * N:(k + 1) * N], dgate[k * N:(k + 1) * N], self.dyp, N, D, pkg.ACT_BF16)
            q.gemm_nt(self.probs(k, self.ap, F, Gw2, 0, 0, B=self.dyp, b_cols=D, beta=1.0, out_expert=True), E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA)
            q.gemm_tn_swiglu_bwd(self.dd, self.ds, self.group, self.probs(k, self.dyp, D, self.gp, F, 2 * n), E, D, F, self.gp, self.up, self.dgp, self.dup)
            q.gemm_nt(self.probs(k, self.Xp, D, Gw1, 0, 0, B=self.dgp, b_cols=F, beta=1.0, out_expert=True), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA)
            q.gemm_nt(self.probs(k, self.Xp, D, Gw3, 0, 0, B=self.dup, b_cols=F, beta=1.0, out_expert=True), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA)
            if self.merged:
                q.gemm_tn_pair(self.dd, self.ds, self.group, self.probs(k, self.dgp, F, self.dXp, D, 0), self.probs(k, self.dup, F, self.dXp, D, n), E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA)
                q.moe_combine(self.dXp, self.inv, None, dx, N, K, D)
            else:
                q.gemm_tn_pair_scatter(self.dd, self.ds, self.group, self.probs(k, self.dgp, F, None, 0, 0, idx_c=True),
                                       self.probs(k, self.dup, F, None, 0, n, idx_c=True), E, F, D, dx)


def _perm_case(orc, N, E, seed, drop=()):
    """one pass: tokens assigned to experts at random, stable counting sort, a few rows dropped (index -1)"""
    rng = np.random.default_rng(seed)
    asn = rng.integers(0, E, N).astype(np.int32)
    perm = np.argsort(asn, kind="stable").astype(np.int32)
    cnt = np.bincount(asn, minlength=E)
    off = np.concatenate([[0], np.cumsum(cnt)]).astype(int)
    for j in drop:
        perm[j] = -1
    return perm, off


def same_but_for_rounding_flips(got, want):
    """bf16 outputs of a GEMM epilogue whose sigmoid comes from the transcendental unit (within 3e-7 of the SwiGLU
    kernel's) against the kernel's: the fp32 values differ by a unit or two in the last place, so now and then one
    lands on the other side of a bf16 rounding boundary. Observed: 3 to 11 elements in a million differ, each by one
    bf16 step (2^-7 relative at most), 2e-6 to 6e-5 relative L2 overall. Allowed: one in 10,000, one step each."""
    import torch
    a, b = (got.to(torch.int32) << 16).view(torch.float32).double(), (want.to(torch.int32) << 16).view(torch.float32).double()
    assert torch.isfinite(a).all()
    assert float((got != want).float().mean()) < 1e-4
    assert float(((a - b).abs() / b.abs().clamp_min(1e-30)).max()) <= 2.0 ** -7
    assert float((a - b).norm() / b.norm()) < 3e-4


@pytest.mark.parametrize("N,E,D,F", [(700, 5, 256, 384), (1500, 8, 768, 2048)])
def test_fused_row_moves_equal_the_separate_kernels(q, orc, N, E, D, F):
    """qlmx_moe_gemm_nn_gather == gather + GEMM, qlmx_moe_gemm_nn_scatter == GEMM + gated scatter,
    qlmx_moe_gemm_tn_pair_scatter == paired input-gradient GEMM + scatter-add, qlmx_moe_gemm_nn_(gather_)swiglu ==
    GEMMs + SwiGLU, qlmx_moe_gemm_tn_swiglu_bwd == GEMM + SwiGLU gradient. Moves and fp32 outputs bit for bit (the
    same arithmetic); the bf16 outputs of the two SwiGLU epilogues up to rare rounding flips (their sigmoid is the
    hardware's). With dropped rows, empty experts and every last-tile height; the separate path is itself checked
    against the oracle in the layer tests below."""
    import torch
    d, s, P, n = encode_layer(orc, 70 + N, E, D, F)
    dd, ds = dev(d), dev(s)
    perm, off = _perm_case(orc, N, E, N, drop=(3, N // 2, N - 1))
    dperm = dev(perm)
    x = orc.bf16_round(orc.normal(N * D, 71, 1))
    dx = dev(x)
    xb = zeros(N * D, torch.int16)
    q.moe_gather(dx, dev(np.arange(N, dtype=np.int32)), xb, N, D, pkg.ACT_BF16)        # the token matrix as bf16, once
    rows = [int(off[e + 1] - off[e]) for e in range(E)]

    def probs(A, a_esz, a_cols, C, c_cols, wbase, idx_a=False, idx_c=False, beta=0.0):
        items = []
        for e in range(E):
            a = dperm.data_ptr() + int(off[e]) * 4 if idx_a else A.data_ptr() + int(off[e]) * a_cols * a_esz
            c = dperm.data_ptr() + int(off[e]) * 4 if idx_c else (None if C is None else C.data_ptr() + int(off[e]) * c_cols * 4)
            items.append((a, None, c, wbase + e * D * F, (wbase + e * D * F) // 128, rows[e], beta))
        return q.problems(items)

    # (a) gather in front of w1
    Xp = zeros(N * D, torch.int16)
    q.moe_gather(dx, dperm, Xp, N, D, pkg.ACT_BF16)
    g_sep, g_fus = zeros(N * F), zeros(N * F)
    q.gemm_nn(dd, ds, 128, probs(Xp, 2, D, g_sep, F, 0), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA_F16)
    q.gemm_nn_gather(dd, ds, 128, probs(None, 0, 0, g_fus, F, 0, idx_a=True), E, D, F, xb)
    torch.cuda.synchronize()
    assert torch.equal(g_sep, g_fus)
    # (b) gated scatter behind w2
    ap = zeros(N * F, torch.int16)
    q.moe_gather(dev(orc.bf16_round(orc.normal(N * F, 71, 2))), dev(np.arange(N, dtype=np.int32)), ap, N, F, pkg.ACT_BF16)
    gate = dev(orc.uniform(N, 71, 3, 0.1, 0.6))
    res = orc.normal(N * D, 71, 4)
    yp, o_sep, o_fus = zeros(N * D), dev(res), dev(res)
    q.gemm_nn(dd, ds, 128, probs(ap, 2, F, yp, D, 2 * n), E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA_F16)
    q.moe_scatter_gate(yp, dperm, gate, o_sep, N, D)
    q.gemm_nn_scatter(dd, ds, 128, probs(ap, 2, F, None, 0, 2 * n, idx_c=True), E, F, D, o_fus, gate)
    torch.cuda.synchronize()
    assert torch.equal(o_sep, o_fus)
    assert not torch.equal(o_fus, dev(res))
    # (b') the same with subnormal products on subnormal sums: the additions of the fused epilogue are float atomics,
    # and must keep subnormals as the separate kernel's load-add-store does
    tiny = dev((orc.uniform(N, 71, 7, 1.0, 64.0) * np.float32(2.0 ** -140)).astype(f32))
    res_t = (orc.normal(N * D, 71, 8) * np.float32(2.0 ** -135)).astype(f32)
    assert np.count_nonzero(res_t) > N * D // 2 and np.abs(res_t).max() < np.float32(2.0 ** -126)
    t_sep, t_fus = dev(res_t), dev(res_t)
    q.moe_scatter_gate(yp, dperm, tiny, t_sep, N, D)
    q.gemm_nn_scatter(dd, ds, 128, probs(ap, 2, F, None, 0, 2 * n, idx_c=True), E, F, D, t_fus, tiny)
    torch.cuda.synchronize()
    assert torch.equal(t_sep.view(torch.int32), t_fus.view(torch.int32))
    assert not torch.equal(t_fus.view(torch.int32), dev(res_t).view(torch.int32))
    assert float(t_fus.abs().max()) < 2.0 ** -120
    # (c) scatter-add behind the paired input gradient
    dgp, dup = zeros(N * F, torch.int16), zeros(N * F, torch.int16)
    ident = dev(np.arange(N, dtype=np.int32))
    q.moe_gather(dev(orc.bf16_round(orc.normal(N * F, 71, 5))), ident, dgp, N, F, pkg.ACT_BF16)
    q.moe_gather(dev(orc.bf16_round(orc.normal(N * F, 71, 6))), ident, dup, N, F, pkg.ACT_BF16)
    dXp, x_sep, x_fus = zeros(N * D), dev(res), dev(res)
    q.gemm_tn_pair(dd, ds, 128, probs(dgp, 2, F, dXp, D, 0), probs(dup, 2, F, dXp, D, n), E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA)
    q.moe_scatter_add(dXp, dperm, x_sep, N, D)
    q.gemm_tn_pair_scatter(dd, ds, 128, probs(dgp, 2, F, None, 0, 0, idx_c=True), probs(dup, 2, F, None, 0, n, idx_c=True), E, F, D, x_fus)
    torch.cuda.synchronize()
    assert torch.equal(x_sep, x_fus)
    # (d) gate | up with the SwiGLU in the epilogue, fp16 matrix core: with and without the gather in front, with and
    # without the fp32 outputs; against the two GEMMs + qlmx_swiglu
    u_sep, a_sep = zeros(N * F), zeros(N * F, torch.int16)
    q.gemm_nn(dd, ds, 128, probs(Xp, 2, D, u_sep, F, n), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA_F16)
    q.swiglu(g_sep, u_sep, a_sep, N * F, pkg.ACT_BF16)

    def up_probs(C, act):
        return q.problems([(None, act.data_ptr() + int(off[e]) * F * 2, None if C is None else C.data_ptr() + int(off[e]) * F * 4,
                            n + e * D * F, (n + e * D * F) // 128, rows[e], 0.0) for e in range(E)])
    poison = lambda: torch.full((N * F,), 0x7FC1, dtype=torch.int16, device="cuda")
    live = torch.zeros(N, dtype=torch.bool, device="cuda"); live[:int(off[E])] = True      # rows past the last expert's are nobody's
    live = live.repeat_interleave(F)
    for gather in (False, True):
        for keep in (True, False):
            g2, u2, a2 = zeros(N * F), zeros(N * F), poison()
            gate_p = probs(None, 0, 0, g2 if keep else None, F, 0, idx_a=True) if gather else probs(Xp, 2, D, g2 if keep else None, F, 0)
            if gather: q.gemm_nn_gather_swiglu(dd, ds, 128, gate_p, up_probs(u2 if keep else None, a2), E, D, F, xb)
            else:      q.gemm_nn_swiglu(dd, ds, 128, gate_p, up_probs(u2 if keep else None, a2), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA_F16)
            torch.cuda.synchronize()
            same_but_for_rounding_flips(a2[live], a_sep[live])
            assert torch.equal(a2[~live], poison()[~live])
            if keep:
                assert torch.equal(g2, g_sep) and torch.equal(u2, u_sep)
    # (e) the SwiGLU gradient behind the down projection's input gradient
    dyp = zeros(N * D, torch.int16)
    q.moe_gather(dev(orc.bf16_round(orc.normal(N * D, 71, 9))), ident, dyp, N, D, pkg.ACT_BF16)
    dap = zeros(N * F)
    q.gemm_tn(dd, ds, 128, probs(dyp, 2, D, dap, F, 2 * n), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA)
    dg_sep, du_sep = zeros(N * F, torch.int16), zeros(N * F, torch.int16)
    q.swiglu_bwd(g_sep, u_sep, dap, dg_sep, du_sep, N * F, pkg.ACT_BF16)
    dg_fus, du_fus = poison(), poison()
    q.gemm_tn_swiglu_bwd(dd, ds, 128, probs(dyp, 2, D, g_sep, F, 2 * n), E, D, F, g_sep, u_sep, dg_fus, du_fus)
    torch.cuda.synchronize()
    same_but_for_rounding_flips(dg_fus[live], dg_sep[live]); same_but_for_rounding_flips(du_fus[live], du_sep[live])
    assert torch.equal(dg_fus[~live], poison()[~live]) and torch.equal(du_fus[~live], poison()[~live])


@pytest.mark.parametrize("math,N,E,D,F,K", [("f32", 96, 4, 128, 256, 2), ("f32", 300, 8, 256, 384, 2),
                                            ("mfma", 512, 4, 256, 384, 2), ("mfma", 1024, 8, 768, 2048, 2),
                                            ("fused", 512, 4, 256, 384, 2), ("fused", 1024, 8, 768, 2048, 2),
                                            ("merged", 512, 4, 256, 384, 2), ("merged", 1024, 8, 768, 2048, 2), ("merged", 700, 8, 256, 384, 4)])
def test_layer_forward_backward_vs_oracle(q, orc, math, N, E, D, F, K):
    import torch
    mth = pkg.MATH_MFMA if math == "mfma" else pkg.MATH_F32
    # MFMA layer: the GEMM inputs ap, dyp, dgp, dup are stored as bf16 (as the reference's GPU path stores them,
    # cudalm.cu:4001-4008, 4061-4087). The oracle rounds the same five buffers, so what is compared is the GEMMs'
    # own error: 1e-3 as for every matmul output. Against the all-fp32 layer the storage rounding alone is worth
    # 2^-9/sqrt(3) = 1.1e-3 per rounded operand; that end-to-end distance is checked second, at 4e-3.
    fused = math in ("fused", "merged")                 # the fused entry points, pass by pass or all passes as one list
    variant, math = math, ("mfma" if fused else math)
    tol = 1e-3 if math == "mfma" else 1e-5
    # The fused layers run the forward on the fp16 matrix core: 2e-4 per GEMM on equal inputs (held to 1e-3 with the
    # GEMMs, and below on this layer's own buffers). Between the layer's GEMMs that error meets a bf16 store: a value
    # that is off by eps lands on the other side of a rounding boundary with probability eps / 2^-8 and is then off by
    # a whole bf16 step, sqrt(2e-4 * 2^-8) = 9e-4 in relative L2 -- against an oracle that rounds the exact values the
    # whole layer therefore shows 0.9e-3 to 1.1e-3 (observed), of which the GEMMs' own share is the 2e-4.
    # (1.11e-3 is the largest figure of the five fused cases below; every GEMM's own share is asserted further down.)
    if fused: tol = 1.2e-3
    d, s, P, n = encode_layer(orc, 40 + N, E, D, F)
    x = orc.normal(N * D, 41, 1)
    dout = orc.normal(N * D, 41, 2)
    if math == "mfma":                                   # bf16 activations, as the training config feeds them
        x = orc.bf16_round(x); dout = orc.bf16_round(dout)
    rt = orc.normal(N * E, 41, 3)
    pr = np.zeros(N * E, f32); asn = np.zeros(K * N, np.int32); gate = np.zeros(K * N, f32)
    orc.router_topk(rt, pr, asn, gate, N, E, K)
    # oracle
    w_out = np.zeros(N * D, f32)
    def oracle_layer(bf16_inter):
        o = np.zeros(N * D, f32)
        rc, ws = orc.moe_forward(x, P[:n], P[n:2 * n], P[2 * n:], asn, gate, o, N, D, F, E, K, bf16_inter=bf16_inter)
        assert rc == 0
        dx_, dg_ = np.zeros(N * D, f32), np.zeros(K * N, f32)
        Gs = [np.zeros(n, f32) for _ in range(3)]
        orc.moe_backward(ws, x, P[:n], P[n:2 * n], P[2 * n:], gate, dout, dx_, dg_, Gs[0], Gs[1], Gs[2])
        orc.moe_ws_free(ws)
        return o, dx_, dg_, Gs
    w_out, w_dx, w_dgate, w_G = oracle_layer(math == "mfma")
    # library: router and grouping on the device too
    dpr, dasn, dgt = zeros(N * E), zeros(K * N, torch.int32), zeros(K * N)
    q.router_topk(dev(rt), dpr, dasn, dgt, N, E, K)
    L = GpuLayerFused(q, dev(d), dev(s), n, N, D, F, E, K, variant == "merged") if fused else GpuLayer(q, dev(d), dev(s), n, N, D, F, E, K, mth)
    out = zeros(N * D)
    dx_ = dev(x); ddout = dev(dout)
    L.forward(dx_, dasn, dgt, out)
    dx, dgate = zeros(N * D), zeros(K * N)
    G = [zeros(n) for _ in range(3)]
    L.backward(dx_, dgt, ddout, dx, dgate, G[0], G[1], G[2])
    torch.cuda.synchronize()
    assert np.array_equal(dasn.cpu().numpy(), asn)
    got = {"out": out, "dx": dx, "dgate": dgate, "G_w1": G[0], "G_w3": G[1], "G_w2": G[2]}
    want = {"out": w_out, "dx": w_dx, "dgate": w_dgate, "G_w1": w_G[0], "G_w3": w_G[1], "G_w2": w_G[2]}
    errs = {k: orc.relerr(got[k].cpu().numpy(), want[k]) for k in got}
    print("layer %s N=%d E=%d D=%d F=%d relative L2 per output:" % (variant, N, E, D, F), {k: "%.2e" % v for k, v in errs.items()})
    assert max(errs.values()) < tol, errs
    if variant == "merged":
        # a row's products do not depend on where the row sits, and the combine adds the passes in their order: what is
        # summed per token equals the pass-by-pass path bit for bit (the weight gradients sum their rows in another order)
        L2 = GpuLayerFused(q, dev(d), dev(s), n, N, D, F, E, K, False)
        out2, dx2, dgate2 = zeros(N * D), zeros(N * D), zeros(K * N)
        G2 = [zeros(n) for _ in range(3)]
        L2.forward(dx_, dasn, dgt, out2)
        L2.backward(dx_, dgt, ddout, dx2, dgate2, G2[0], G2[1], G2[2])
        torch.cuda.synchronize()
        assert torch.equal(out, out2) and torch.equal(dx, dx2) and torch.equal(dgate, dgate2)
        for a, b in zip(G, G2):
            assert orc.relerr(a.cpu().numpy(), b.cpu().numpy()) < 1e-5
    if math == "mfma":
        # Every matmul of the layer against the oracle ON THE LAYER'S OWN INPUTS, for the expert with the most rows and
        # the one with the fewest: the 1e-3 bar of a matmul output, one GEMM at a time. After the backward pass the
        # grouped buffers hold the rows of the last list that ran (all K*N rows when merged, the last pass otherwise); a
        # pass-by-pass layer sums its weight gradients over the passes, so there the three weight-gradient GEMMs are
        # run once more on the last pass's buffers into gradients of their own.
        k = L.offh.shape[0] - 1
        Gs = G
        if variant != "merged":
            Gs = [zeros(n) for _ in range(3)]
            if fused:
                pr = lambda A, a_cols, Gm, B, b_cols: L.probs(k, A, a_cols, Gm, 0, 0, B=B, b_cols=b_cols, beta=1.0, out_expert=True)
            else:
                pr = lambda A, a_cols, Gm, B, b_cols: L.probs(k, A, a_cols, 2, Gm, 0, 0, B=B, b_cols=b_cols, b_esz=2, beta=1.0, out_expert=True)
            q.gemm_nt(pr(L.ap, F, Gs[2], L.dyp, D), E, F, D, pkg.ACT_BF16, pkg.MATH_MFMA)
            q.gemm_nt(pr(L.Xp, D, Gs[0], L.dgp, F), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA)
            q.gemm_nt(pr(L.Xp, D, Gs[1], L.dup, F), E, D, F, pkg.ACT_BF16, pkg.MATH_MFMA)
            torch.cuda.synchronize()
        cnt = np.diff(L.offh[k]); DF = D * F
        for e in sorted({int(np.argmax(cnt)), int(np.argmin(np.where(cnt > 0, cnt, cnt.max() + 1)))}):
            o, ne = int(L.offh[k][e]), int(cnt[e])
            rows = lambda t, cols, bf: (bf16_to_f32(t[o * cols:(o + ne) * cols]) if bf else t[o * cols:(o + ne) * cols].cpu().numpy())
            Xp_e, ap_e, dyp_e, dgp_e, dup_e = rows(L.Xp, D, 1), rows(L.ap, F, 1), rows(L.dyp, D, 1), rows(L.dgp, F, 1), rows(L.dup, F, 1)
            w1, w3, w2 = P[e * DF:(e + 1) * DF], P[n + e * DF:n + (e + 1) * DF], P[2 * n + e * DF:2 * n + (e + 1) * DF]
            stage = {}
            c = np.zeros(ne * F, f32); orc.gemm_nn(Xp_e, w1, c, ne, D, F); stage["gp"] = orc.relerr(rows(L.gp, F, 0), c)
            c = np.zeros(ne * F, f32); orc.gemm_nn(Xp_e, w3, c, ne, D, F); stage["up"] = orc.relerr(rows(L.up, F, 0), c)
            c = np.zeros(ne * D, f32); orc.gemm_nn(ap_e, w2, c, ne, F, D); stage["yp"] = orc.relerr(rows(L.yp, D, 0), c)
            if not fused:                                              # the fused layer never stores d(act)
                c = np.zeros(ne * F, f32); orc.gemm_tn(dyp_e, w2, c, ne, D, F, 0.0); stage["dap"] = orc.relerr(rows(L.dap, F, 0), c)
            if variant != "fused":                                     # ... and its pass-by-pass form scatters dXp from the accumulators
                c = np.zeros(ne * D, f32); orc.gemm_tn(dgp_e, w1, c, ne, F, D, 0.0); orc.gemm_tn(dup_e, w3, c, ne, F, D, 1.0)
                stage["dXp"] = orc.relerr(rows(L.dXp, D, 0), c)
            c = np.zeros(DF, f32); orc.gemm_nt(ap_e, dyp_e, c, ne, F, D); stage["G_w2"] = orc.relerr(Gs[2][e * DF:(e + 1) * DF].cpu().numpy(), c)
            c = np.zeros(DF, f32); orc.gemm_nt(Xp_e, dgp_e, c, ne, D, F); stage["G_w1"] = orc.relerr(Gs[0][e * DF:(e + 1) * DF].cpu().numpy(), c)
            c = np.zeros(DF, f32); orc.gemm_nt(Xp_e, dup_e, c, ne, D, F); stage["G_w3"] = orc.relerr(Gs[1][e * DF:(e + 1) * DF].cpu().numpy(), c)
            print("    expert %d (%d rows), each matmul on the layer's own inputs:" % (e, ne), {k_: "%.2e" % v for k_, v in stage.items()})
            assert max(stage.values()) < 1e-3, (e, stage)
        f_out, f_dx, f_dgate, f_G = oracle_layer(False)             # the CPU build's all-fp32 layer, end to end
        want = {"out": f_out, "dx": f_dx, "dgate": f_dgate, "G_w1": f_G[0], "G_w3": f_G[1], "G_w2": f_G[2]}
        e2e = {k: orc.relerr(got[k].cpu().numpy(), want[k]) for k in got}
        print("    against the all-fp32 layer:", {k: "%.2e" % v for k, v in e2e.items()})
        assert max(e2e.values()) < 4e-3, e2e
