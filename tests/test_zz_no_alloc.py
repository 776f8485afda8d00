"""GPU test of qlmx_moe_decode_forward_noalloc, the decode layer over a fixed device array for callers
that cannot allocate: through the C ABI, bit-for-bit against qlmx_moe_decode_forward (the same kernel
over the library's grow-only workspace) and within 1e-3 relative L2 (observed ~1e-6) of the CPU oracle's
layer, on two calls in a row of which the second has a smaller input, then under a HIP graph whose
replays must each equal the eager result. Collected last (file name) so that a failure here hides no
other test."""
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


def layer(orc, seed, E, D, F, group=128):
    n = E * D * F
    tab, nq, ng = make_spans([n, n, n], group)
    P = orc.normal(nq, seed, 1, 0.02)
    d = np.zeros(nq // 2, np.int8); r = np.zeros(nq, np.int8); s = np.zeros(ng, f32)
    orc.encode(P, d, r, s, tab, group, 7, 1, ng)
    orc.render(P, d, s, tab, group, 1, 0, ng)
    return d, s, P, n


def case(orc, seed, T, E, D, F, K):
    x = orc.normal(T * D, seed, 2)
    rt = orc.normal(T * E, seed, 3)
    pr = np.zeros(T * E, f32); asn = np.zeros(K * T, np.int32); gate = np.zeros(K * T, f32)
    orc.router_topk(rt, pr, asn, gate, T, E, K)
    res = orc.normal(T * D, seed, 4)
    return x, asn, gate, res


def test_noalloc_equals_allocating_entry_two_calls(q, orc):
    import torch
    E, D, F, K = 8, 768, 2048, 2
    d, s, P, n = layer(orc, 21, E, D, F)
    dd, ds = dev(d), dev(s)
    for seed, T in ((31, 16), (32, 3)):                      # the second call is smaller and reuses the array as the first left it
        x, asn, gate, res = case(orc, seed, T, E, D, F, K)
        dx, da, dg = dev(x), dev(asn), dev(gate)
        ref_out, out = dev(res), dev(res)
        q.decode_forward(dx, da, dg, ref_out, dd, ds, 128, 0, n, 2 * n, T, K, E, D, F)
        q.decode_forward_noalloc(dx, da, dg, out, dd, ds, 128, 0, n, 2 * n, T, K, E, D, F)
        torch.cuda.synchronize()
        assert torch.equal(out, ref_out), "T=%d: outputs of the two entry points differ" % T
        want = res.copy()
        rc, ws = orc.moe_forward(x, P[:n], P[n:2 * n], P[2 * n:], asn, gate, want, T, D, F, E, K)
        orc.moe_ws_free(ws)
        assert rc == 0
        err = orc.relerr(out.cpu().numpy() - res, want - res)
        assert err < 1e-3 and err < 2e-5, err                # fp32 math: tolerance 1e-3 relative L2, observed ~1e-6


def test_noalloc_rejects_shapes_beyond_the_array(q):
    import torch
    # 64 pairs at D = F = 8192: far more partial sums than the array holds -> QLMX_E_LIMIT (-4) before any launch
    z = torch.zeros(8, device="cuda")
    zi = torch.zeros(64, dtype=torch.int32, device="cuda")
    with pytest.raises(pkg.QlmxError) as ei:
        q.decode_forward_noalloc(z, zi, z, z, z.view(torch.int8), z, 128, 0, 0, 0, 32, 2, 4, 8192, 8192)
    assert "error -4" in str(ei.value) and "fixed scratch" in str(ei.value)


def test_noalloc_in_a_graph_every_replay_equals_eager(q, orc):
    """Three layers with different problem counts recorded once and replayed with new inputs: the tag of the
    hand-over words is a device word that each launch moves on, so a replay must not see an earlier
    replay's partial sums as current. Eager work and synchronisations sit between the replays."""
    import torch
    E, D, F, K = 8, 256, 512, 2
    layers = [layer(orc, 40 + l, E, D, F) for l in range(3)]
    Ts = 8
    dws = [(dev(d), dev(s)) for d, s, _, _ in layers]
    n = layers[0][3]
    # layer l sees a different number of distinct experts: restrict the routed experts per layer
    asns, gates = [], []
    for l in range(3):
        rt = orc.normal(Ts * E, 50 + l, 3)
        rt.reshape(Ts, E)[:, (2 + 3 * l):] -= 30.0          # layer 0: experts 0-1, layer 1: 0-4, layer 2: all
        pr = np.zeros(Ts * E, f32); a = np.zeros(K * Ts, np.int32); g = np.zeros(K * Ts, f32)
        orc.router_topk(rt, pr, a, g, Ts, E, K)
        asns.append(dev(a)); gates.append(dev(g))
    x = torch.zeros(Ts * D, device="cuda")
    out = torch.zeros(Ts * D, device="cuda")
    side = torch.cuda.Stream()

    def run(stream):
        for l in range(3):
            q.decode_forward_noalloc(x, asns[l], gates[l], out, dws[l][0], dws[l][1], 128, 0, n, 2 * n, Ts, K, E, D, F, stream)

    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(side.cuda_stream); side.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr, stream=side):
            run(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for rep in range(5):
        xv = dev(orc.normal(Ts * D, 60 + rep, 2))
        x.copy_(xv); out.zero_()
        torch.cuda.synchronize()
        gr.replay()
        torch.cuda.synchronize()
        got = out.clone()
        out.zero_()
        run(torch.cuda.current_stream().cuda_stream)          # eager, same inputs
        torch.cuda.synchronize()
        assert torch.equal(got, out), "replay %d differs from the eager result" % rep
