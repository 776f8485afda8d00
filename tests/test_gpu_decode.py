"""GPU parity of the decode-shaped (few-token) expert path: the streaming GEMV behind
qlmx_moe_gemm_nn and the fused qlmx_moe_decode_forward, against the CPU oracle's rendered-weights
fp32 layer (moe_forward call order, cudalm.cu:4193-4228). Tolerance 1e-3 relative L2 as stated for
matmul outputs. The fused layer has two multiply loops and every layer test runs with both: the default
fp32 one differs from the oracle in summation order and the libm exp only (observed 4e-7, held to 2e-5),
the other (qlmx_decode_math(1)) takes its inputs as fp16 pairs (11 significant bits; observed 2.4e-4 ..
4.9e-4 on a layer's output, held to 7e-4 here). Routing indices come from the oracle's router and are consumed as
given."""
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


@pytest.fixture(params=[0, 1], ids=["fp32", "fp16-inputs"])
def tol(request, q):
    """Selects the decode layer's multiply loop for one test and returns the bound its output is held to."""
    q.call("qlmx_decode_math", request.param)
    yield 7e-4 if request.param else 2e-5
    q.call("qlmx_decode_math", 0)


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def encode_layer(orc, seed, E, D, F, group=128):
    """w1 | w3 | w2 back to back in one digit array (three consecutive spans)."""
    n = E * D * F
    tab, nq, ng = make_spans([n, n, n], group)
    P = orc.normal(nq, seed, 1, 0.02)
    d = np.zeros(nq // 2, np.int8); r = np.zeros(nq, np.int8); s = np.zeros(ng, f32)
    orc.encode(P, d, r, s, tab, group, 7, 1, ng)
    orc.render(P, d, s, tab, group, 1, 0, ng)
    return d, s, P, n


@pytest.mark.parametrize("K,N", [(768, 2048), (2048, 768), (512, 1536)])
def test_gemv_small_rows_vs_oracle(q, orc, K, N):
    """qlmx_moe_gemm_nn with 1..4 rows per expert takes the streaming path; an empty expert is skipped."""
    import torch
    E = 5
    rows = [1, 4, 0, 2, 3]
    n = E * K * N
    tab, nq, ng = make_spans([n], 128)
    P = orc.normal(n, 3, 1, 0.02)
    d = np.zeros(n // 2, np.int8); r = np.zeros(n, np.int8); s = np.zeros(ng, f32)
    orc.encode(P, d, r, s, tab, 128, 7, 1, ng)
    orc.render(P, d, s, tab, 128, 1, 0, ng)
    off = np.concatenate([[0], np.cumsum(rows)])
    A = orc.normal(int(off[-1]) * K, 3, 2)
    dA, dC, dd, ds = dev(A), torch.full((int(off[-1]) * N,), 7.0, device="cuda"), dev(d), dev(s)
    items = [(dA.data_ptr() + int(off[e]) * K * 4, None, dC.data_ptr() + int(off[e]) * N * 4, e * K * N, e * K * N // 128, rows[e], 0.0)
             for e in range(E)]
    q.gemm_nn(dd, ds, 128, q.problems(items), E, K, N, pkg.ACT_F32, pkg.MATH_F32)
    torch.cuda.synchronize()
    want = np.zeros(int(off[-1]) * N, f32)
    for e in range(E):
        if rows[e]:
            orc.gemm_nn(A[off[e] * K:], P[e * K * N:(e + 1) * K * N], want[off[e] * N:off[e + 1] * N], rows[e], K, N)
    err = orc.relerr(dC.cpu().numpy(), want)
    assert err < 1e-5, err
    # a second call reuses the tickets and scratch: same answer
    dC.fill_(0)
    q.gemm_nn(dd, ds, 128, q.problems(items), E, K, N, pkg.ACT_F32, pkg.MATH_F32)
    torch.cuda.synchronize()
    assert orc.relerr(dC.cpu().numpy(), want) < 1e-5
    # forty calls without a synchronisation between them go twice round the ring of problem tables,
    # each call with its own output (and a different problem order): every one must come out right
    outs = [torch.zeros(int(off[-1]) * N, device="cuda") for _ in range(40)]
    for it, o in enumerate(outs):
        its = [(dA.data_ptr() + int(off[e]) * K * 4, None, o.data_ptr() + int(off[e]) * N * 4, e * K * N, e * K * N // 128, rows[e], 0.0)
               for e in range(E)]
        if it & 1:
            its.reverse()
        q.gemm_nn(dd, ds, 128, q.problems(its), E, K, N, pkg.ACT_F32, pkg.MATH_F32)
    torch.cuda.synchronize()
    for o in outs:
        assert orc.relerr(o.cpu().numpy(), want) < 1e-5


@pytest.mark.parametrize("T,E,D,F,K", [(1, 32, 768, 2048, 2), (4, 32, 768, 2048, 2), (16, 32, 768, 2048, 2), (4, 8, 768, 2048, 2), (16, 8, 768, 2048, 2),
                                       (16, 4, 256, 384, 4), (5, 3, 128, 256, 1), (7, 6, 1024, 640, 3), (3, 4, 2048, 256, 2)])
def test_decode_forward_vs_oracle_layer(q, orc, tol, T, E, D, F, K):
    import torch
    d, s, P, n = encode_layer(orc, 11 + T, E, D, F)
    x = orc.normal(T * D, 11, 2)
    rt = orc.normal(T * E, 11, 3)
    pr = np.zeros(T * E, f32); asn = np.zeros(K * T, np.int32); gate = np.zeros(K * T, f32)
    orc.router_topk(rt, pr, asn, gate, T, E, K)
    res = orc.normal(T * D, 11, 4)                      # residual the layer accumulates into
    want = res.copy()
    rc, ws = orc.moe_forward(x, P[:n], P[n:2 * n], P[2 * n:], asn, gate, want, T, D, F, E, K)
    orc.moe_ws_free(ws)
    assert rc == 0
    out = dev(res)
    dd, ds = dev(d), dev(s)
    q.decode_forward(dev(x), dev(asn), dev(gate), out, dd, ds, 128, 0, n, 2 * n, T, K, E, D, F)
    torch.cuda.synchronize()
    err = orc.relerr(out.cpu().numpy() - res, want - res)
    assert err < 1e-3, err
    assert err < tol, err
    # run-to-run determinism: slice order, not arrival order, fixes the sums
    out2 = dev(res)
    q.decode_forward(dev(x), dev(asn), dev(gate), out2, dd, ds, 128, 0, n, 2 * n, T, K, E, D, F)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


@pytest.mark.parametrize("T", [2, 3, 5, 6, 7, 9, 11, 13, 24, 32])
def test_decode_token_counts_cover_leftover_groups(q, orc, tol, T):
    """Token counts whose numbers of problems leave every remainder modulo the 8 XCDs (the groups left over after
    a full round are cut into pieces over the XCDs), up to the 64 (pass, token) pairs a call may carry."""
    import torch
    E, D, F, K = 16, 256, 512, 2
    d, s, P, n = encode_layer(orc, 70 + T, E, D, F)
    x = orc.normal(T * D, 70 + T, 2)
    rt = orc.normal(T * E, 70 + T, 3)
    pr = np.zeros(T * E, f32); asn = np.zeros(K * T, np.int32); gate = np.zeros(K * T, f32)
    orc.router_topk(rt, pr, asn, gate, T, E, K)
    want = np.zeros(T * D, f32)
    rc, ws = orc.moe_forward(x, P[:n], P[n:2 * n], P[2 * n:], asn, gate, want, T, D, F, E, K)
    orc.moe_ws_free(ws)
    assert rc == 0
    out = torch.zeros(T * D, device="cuda")
    q.decode_forward(dev(x), dev(asn), dev(gate), out, dev(d), dev(s), 128, 0, n, 2 * n, T, K, E, D, F)
    torch.cuda.synchronize()
    assert orc.relerr(out.cpu().numpy(), want) < tol


def test_decode_all_tokens_one_expert(q, orc, tol):
    """Collision case: 16 tokens on the same two experts -> problems are cut into row pairs."""
    import torch
    T, E, D, F, K = 16, 4, 256, 512, 2
    d, s, P, n = encode_layer(orc, 5, E, D, F)
    x = orc.normal(T * D, 5, 2)
    asn = np.concatenate([np.full(T, 2), np.full(T, 0)]).astype(np.int32)
    gate = orc.uniform(K * T, 5, 3, 0.1, 0.6)
    want = np.zeros(T * D, f32)
    rc, ws = orc.moe_forward(x, P[:n], P[n:2 * n], P[2 * n:], asn, gate, want, T, D, F, E, K)
    orc.moe_ws_free(ws)
    out = torch.zeros(T * D, device="cuda")
    q.decode_forward(dev(x), dev(asn), dev(gate), out, dev(d), dev(s), 128, 0, n, 2 * n, T, K, E, D, F)
    torch.cuda.synchronize()
    assert orc.relerr(out.cpu().numpy(), want) < tol


def test_decode_group_256_and_rejected_groups(q, orc, tol):
    """Scale groups of 256 (one per task row) go through the same kernel; 64 and 96 are refused."""
    import torch
    T, E, D, F, K = 4, 4, 512, 768, 2
    d, s, P, n = encode_layer(orc, 21, E, D, F, group=256)
    x = orc.normal(T * D, 21, 2)
    rt = orc.normal(T * E, 21, 3)
    pr = np.zeros(T * E, f32); asn = np.zeros(K * T, np.int32); gate = np.zeros(K * T, f32)
    orc.router_topk(rt, pr, asn, gate, T, E, K)
    want = np.zeros(T * D, f32)
    rc, ws = orc.moe_forward(x, P[:n], P[n:2 * n], P[2 * n:], asn, gate, want, T, D, F, E, K)
    orc.moe_ws_free(ws)
    out = torch.zeros(T * D, device="cuda")
    q.decode_forward(dev(x), dev(asn), dev(gate), out, dev(d), dev(s), 256, 0, n, 2 * n, T, K, E, D, F)
    torch.cuda.synchronize()
    assert orc.relerr(out.cpu().numpy(), want) < tol
    for g in (64, 96):
        with pytest.raises(pkg.QlmxError, match="group"):
            q.decode_forward(dev(x), dev(asn), dev(gate), out, dev(d), dev(s), g, 0, n, 2 * n, T, K, E, D, F)


def test_decode_invalid_expert_is_skipped(q, orc, tol):
    """A pair with an out-of-range expert adds nothing; the other pairs are unaffected."""
    import torch
    T, E, D, F, K = 3, 4, 256, 512, 2
    d, s, P, n = encode_layer(orc, 9, E, D, F)
    x = orc.normal(T * D, 9, 2)
    asn = np.array([1, 3, 0, 2, 1, 3], np.int32)          # [k][t]
    gate = orc.uniform(K * T, 9, 3, 0.1, 0.6)
    bad = asn.copy(); bad[4] = 7                          # pass 1, token 1 -> expert 7 of 4
    gate_ref = gate.copy(); gate_ref[4] = 0.0             # the reference result with that pair's weight zeroed
    want = np.zeros(T * D, f32)
    rc, ws = orc.moe_forward(x, P[:n], P[n:2 * n], P[2 * n:], asn, gate_ref, want, T, D, F, E, K)
    orc.moe_ws_free(ws)
    out = torch.zeros(T * D, device="cuda")
    q.decode_forward(dev(x), dev(bad), dev(gate), out, dev(d), dev(s), 128, 0, n, 2 * n, T, K, E, D, F)
    torch.cuda.synchronize()
    assert orc.relerr(out.cpu().numpy(), want) < tol
    allbad = np.full(K * T, -1, np.int32)
    out.zero_()
    q.decode_forward(dev(x), dev(allbad), dev(gate), out, dev(d), dev(s), 128, 0, n, 2 * n, T, K, E, D, F)
    torch.cuda.synchronize()
    assert float(out.abs().max()) == 0.0


def test_decode_repeated_calls_alternating_shapes(q, orc, tol):
    """The hand-over words carry the call's epoch: stale partial sums of earlier calls, of other
    shapes and token counts, must never be taken for current ones."""
    import torch
    cases = []
    for (T, E, D, F, K, seed) in [(16, 8, 256, 512, 2, 31), (1, 8, 256, 512, 2, 32), (5, 4, 512, 256, 3, 33)]:
        d, s, P, n = encode_layer(orc, seed, E, D, F)
        x = orc.normal(T * D, seed, 2)
        rt = orc.normal(T * E, seed, 3)
        pr = np.zeros(T * E, f32); asn = np.zeros(K * T, np.int32); gate = np.zeros(K * T, f32)
        orc.router_topk(rt, pr, asn, gate, T, E, K)
        want = np.zeros(T * D, f32)
        rc, ws = orc.moe_forward(x, P[:n], P[n:2 * n], P[2 * n:], asn, gate, want, T, D, F, E, K)
        orc.moe_ws_free(ws)
        cases.append((T, E, D, F, K, n, dev(x), dev(asn), dev(gate), dev(d), dev(s), want))
    outs = []
    for rep in range(12):
        T, E, D, F, K, n, x, asn, gate, d, s, want = cases[rep % 3]
        out = torch.zeros(T * D, device="cuda")
        q.decode_forward(x, asn, gate, out, d, s, 128, 0, n, 2 * n, T, K, E, D, F)
        outs.append((out, want))
    torch.cuda.synchronize()
    for out, want in outs:
        assert orc.relerr(out.cpu().numpy(), want) < tol


def test_decode_wait_timeout_is_reported_once(q, orc, tol):
    """The waits between the three task lists are bounded. Forced from the host (qlmx_test_force_wait_timeout: for
    one launch every wait looks, for one poll, for a tag nobody writes) all of them give up, the kernel still ends
    normally, the NEXT call returns QLMX_E_HIP once, and the call after that is correct again."""
    import torch
    T, E, D, F, K = 8, 8, 256, 512, 2
    d, s, P, n = encode_layer(orc, 51, E, D, F)
    x = orc.normal(T * D, 51, 2)
    rt = orc.normal(T * E, 51, 3)
    pr = np.zeros(T * E, f32); asn = np.zeros(K * T, np.int32); gate = np.zeros(K * T, f32)
    orc.router_topk(rt, pr, asn, gate, T, E, K)
    want = np.zeros(T * D, f32)
    rc, ws = orc.moe_forward(x, P[:n], P[n:2 * n], P[2 * n:], asn, gate, want, T, D, F, E, K)
    orc.moe_ws_free(ws)
    args = (dev(x), dev(asn), dev(gate))
    dd, ds = dev(d), dev(s)
    out = torch.zeros(T * D, device="cuda")
    q.call("qlmx_test_force_wait_timeout", 1)
    q.decode_forward(*args, out, dd, ds, 128, 0, n, 2 * n, T, K, E, D, F)      # gives up everywhere, ends normally
    torch.cuda.synchronize()
    with pytest.raises(pkg.QlmxError, match="gave up waiting"):
        q.decode_forward(*args, out, dd, ds, 128, 0, n, 2 * n, T, K, E, D, F)
    out.zero_()
    q.decode_forward(*args, out, dd, ds, 128, 0, n, 2 * n, T, K, E, D, F)
    torch.cuda.synchronize()
    assert orc.relerr(out.cpu().numpy(), want) < tol


def test_decode_limits(q):
    import torch
    z = torch.zeros(65536, device="cuda")
    zi = torch.zeros(256, dtype=torch.int32, device="cuda")
    with pytest.raises(pkg.QlmxError, match="pairs"):
        q.decode_forward(z, zi, z, z, z, z, 128, 0, 0, 0, 64, 2, 4, 128, 128)
    with pytest.raises(pkg.QlmxError, match="multiples of 32"):
        q.decode_forward(z, zi, z, z, z, z, 128, 0, 0, 0, 2, 2, 4, 100, 128)
