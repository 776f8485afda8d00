"""ctypes bindings for the two CPU checkers. TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this module;
the shipped library never does. `Oracle` wraps oracle/libqlm_oracle.so (the repo's C restatement),
`Ref` wraps oracle/_ref/libcudalm_ref.so (the reference's own CPU backend, present only where it
was built from the reference sources). Both take numpy arrays and mutate them in place, exactly
like the C functions.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "libqlm_oracle.so")
REF_SO = os.path.join(HERE, "_ref", "libcudalm_ref.so")

SPAN_DTYPE = np.dtype(
    [("pof", "<u8"), ("gof", "<u8"), ("qi0", "<u8"), ("n", "<u8"),
     ("gi0", "<i4"), ("ngrp", "<i4"), ("sref", "<f4"), ("_pad", "<i4")], align=False)
assert SPAN_DTYPE.itemsize == 48

c_f = C.c_float
c_i = C.c_int
c_u64 = C.c_ulonglong
c_vp = C.c_void_p
c_sz = C.c_size_t


def _p(a):
    """numpy array (or None) -> void*"""
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "array must be C-contiguous"
    return a.ctypes.data_as(c_vp)


def make_spans(sizes, group, pofs=None, gofs=None):
    """Span table for tensors of the given element counts laid out back to back
    (qlm.cuh:448-455). Returns (table, nq, ngrp)."""
    tab = np.zeros(len(sizes), dtype=SPAN_DTYPE)
    nq = 0
    ngrp = 0
    pof = 0
    for i, n in enumerate(sizes):
        tab[i]["pof"] = pofs[i] if pofs is not None else pof
        tab[i]["gof"] = gofs[i] if gofs is not None else tab[i]["pof"]
        tab[i]["qi0"] = nq
        tab[i]["n"] = n
        tab[i]["gi0"] = ngrp
        tab[i]["ngrp"] = (n + group - 1) // group
        tab[i]["sref"] = 1.0
        nq += n
        ngrp += int(tab[i]["ngrp"])
        pof += n
    return tab, nq, ngrp


class _Lib:
    def __init__(self, path):
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        self.lib = C.CDLL(path)

    def _sig(self, name, restype, argtypes):
        f = getattr(self.lib, name)
        f.restype = restype
        f.argtypes = argtypes
        return f


_STEP_ARGS = [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i,
              c_f, c_f, c_f, c_f, c_f, c_vp, c_f, c_f, c_i, c_u64, c_i, c_vp, c_i, c_i, c_i]


class Oracle(_Lib):
    def __init__(self, path=ORACLE_SO):
        super().__init__(path)
        s = self._sig
        self.qhashu = s("orc_qhashu", C.c_uint32, [c_u64])
        self.qsri = s("orc_qsri", c_i, [c_f, c_u64, c_u64])
        self.qclmp = s("orc_qclmp", c_i, [c_i, c_i, c_i])
        self._qd_get = s("orc_qd_get", c_i, [c_vp, c_u64, c_i])
        self._qd_set = s("orc_qd_set", None, [c_vp, c_u64, c_i, c_i])
        self.qd_bytes = s("orc_qd_bytes", c_u64, [c_u64, c_i])
        self._span_sref = s("orc_span_sref", None, [c_vp, c_i, c_vp])
        self._encode = s("orc_encode", None, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i])
        self._render = s("orc_render", None, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i])
        self._step = s("orc_step", None, _STEP_ARGS + [c_i])
        self._servo = s("orc_servo", None, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_f, c_f, c_i, c_i])
        self._gemm_nn = s("orc_gemm_nn", None, [c_vp, c_vp, c_vp, c_i, c_i, c_i])
        self._gemm_tn = s("orc_gemm_tn", None, [c_vp, c_vp, c_vp, c_i, c_i, c_i, c_f])
        self._gemm_nt = s("orc_gemm_nt", None, [c_vp, c_vp, c_vp, c_i, c_i, c_i])
        self._gemm_nn64 = s("orc_gemm_nn_f64", None, [c_vp, c_vp, c_vp, c_i, c_i, c_i])
        self._gemm_tn64 = s("orc_gemm_tn_f64", None, [c_vp, c_vp, c_vp, c_i, c_i, c_i])
        self._gemm_nt64 = s("orc_gemm_nt_f64", None, [c_vp, c_vp, c_vp, c_i, c_i, c_i])
        self._relerr = s("orc_relerr", C.c_double, [c_vp, c_vp, c_sz])
        self.fexp = s("orc_fexp", c_f, [c_f])
        self._router = s("orc_router_topk", None, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_vp, c_i])
        self._perm = s("orc_moe_perm", c_i, [c_vp, c_i, c_i, c_vp, c_vp])
        self._gather = s("orc_gather", None, [c_vp, c_vp, c_vp, c_i, c_i])
        self._scatter_gate = s("orc_scatter_gate", None, [c_vp, c_vp, c_vp, c_vp, c_i, c_i])
        self._scatter_add = s("orc_scatter_add", None, [c_vp, c_vp, c_vp, c_i, c_i])
        self._dgate = s("orc_moe_dgate", None, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i])
        self._swiglu = s("orc_swiglu", None, [c_vp, c_vp, c_vp, c_sz])
        self._swiglu_bwd = s("orc_swiglu_bwd", None, [c_vp, c_vp, c_vp, c_vp, c_vp, c_sz])
        self._recip = s("orc_recip_div_mismatches", c_sz, [C.c_uint64, c_sz])
        self._sqsum = s("orc_sqsum", None, [c_vp, C.c_uint64, c_vp])
        self._gnorm = s("orc_gnorm", None, [c_vp, c_i, c_i, c_vp])
        self._step_touched = s("orc_step_touched", None, [c_vp] * 10 + [c_i, c_i, c_i, c_f, c_f, c_f, c_f, c_f, c_f, c_f,
                                                                       C.c_uint64, C.c_uint64, c_vp, c_i])
        self._q4n_q = s("orc_q4n_quantize", c_sz, [c_vp, c_sz, c_i, c_vp, c_sz, c_vp])
        self._q4n_d = s("orc_q4n_dequantize", c_i, [c_vp, c_sz, c_vp, c_sz, c_i])
        self._ws_new = s("orc_moe_ws_new", c_vp, [c_i, c_i, c_i, c_i, c_i])
        self._ws_free = s("orc_moe_ws_free", None, [c_vp])
        self._ws_bf16 = s("orc_moe_ws_bf16", None, [c_vp, c_i])
        self._moe_fwd = s("orc_moe_forward", c_i, [c_vp] * 8)
        self._moe_bwd = s("orc_moe_backward", None, [c_vp] * 12)
        self._fill_normal = s("orc_fill_normal", None, [c_vp, c_sz, c_u64, c_u64, c_f])
        self._fill_uniform = s("orc_fill_uniform", None, [c_vp, c_sz, c_u64, c_u64, c_f, c_f])
        self._fill_int8 = s("orc_fill_int8", None, [c_vp, c_sz, c_u64, c_u64, c_i, c_i])
        self._fill_u8 = s("orc_fill_u8", None, [c_vp, c_sz, c_u64, c_u64, c_i, c_i])
        self._fill_digits = s("orc_fill_digits", None, [c_vp, c_sz, c_u64, c_u64, c_i, c_i])
        self._bf16_n = s("orc_bf16_round_n", None, [c_vp, c_sz])
        self.set_threads = s("orc_set_threads", None, [c_i])
        self.get_threads = s("orc_get_threads", c_i, [])

    # ---- helpers ----
    def qd_get(self, d, i, packed):
        return self._qd_get(_p(d), i, packed)

    def qd_set(self, d, i, v, packed):
        self._qd_set(_p(d), i, v, packed)

    def unpack(self, d, nq, packed=1):
        """all digits as an int8 vector (numpy, vectorised statement of qd_get)"""
        if not packed:
            return d[:nq].astype(np.int8).copy()
        b = d.view(np.uint8)
        lo = (b & 15).astype(np.int16)
        hi = (b >> 4).astype(np.int16)
        out = np.empty(b.size * 2, dtype=np.int16)
        out[0::2] = lo
        out[1::2] = hi
        out = np.where(out >= 8, out - 16, out).astype(np.int8)
        return out[:nq]

    def span_sref(self, tab, s):
        self._span_sref(_p(tab), len(tab), _p(s))

    def encode(self, P, d, r, s, tab, group, dmax, packed, ngrp):
        self._encode(_p(P), _p(d), _p(r), _p(s), _p(tab), len(tab), group, dmax, packed, ngrp)

    def render(self, P, d, s, tab, group, packed, gi_base, ng):
        self._render(_p(P), _p(d), _p(s), _p(tab), len(tab), group, packed, gi_base, ng)

    def step(self, P, G, d, r, s, m8, m8s, v8, v8s, tab, group, dmax, lr, b1, b2, wd, gscale, gsp,
             inv_bc1, inv_sqrt_bc2, lrmode, t, adam, stat, packed, gi_base, ng, v4=0):
        self._step(_p(P), _p(G), _p(d), _p(r), _p(s), _p(m8), _p(m8s), _p(v8), _p(v8s), _p(tab), len(tab),
                   group, dmax, lr, b1, b2, wd, gscale, _p(gsp), inv_bc1, inv_sqrt_bc2, lrmode, t, adam,
                   _p(stat), packed, gi_base, ng, v4)

    def servo(self, d, r, s, tab, group, dmax, f_hi, f_lo, packed, ngrp):
        self._servo(_p(d), _p(r), _p(s), _p(tab), len(tab), group, dmax, f_hi, f_lo, packed, ngrp)

    def step_slice(self, G, d, r, s, m8, m8s, v8, v8s, qi0, gi0, sref, group, dmax, lr, b1, b2, wd, gscale,
                   inv_bc1, inv_sqrt_bc2, lrmode, t, adam, v4=0):
        """The step over a cut-out piece of a much larger packed state: the arrays hold only elements
        qi0 .. qi0+r.size (groups gi0 ..) of the whole, and the arithmetic (hash keys are functions of the
        global element index) is that of the whole sweep. Groups are independent, so this equals the same
        groups of a step over everything. The pointers handed to the C function are moved back by the
        piece's offset; only the piece is ever touched."""
        n = r.size
        assert n % group == 0 and qi0 % 2 == 0 and d.size * 2 == n and G.size == n and s.size * group == n
        tab = np.zeros(1, dtype=SPAN_DTYPE)
        tab[0] = (0, 0, qi0, n, gi0, n // group, sref, 0)
        for a in (G, d, r, s, m8, m8s, v8, v8s):
            assert a.flags["C_CONTIGUOUS"]

        def back(a, off_bytes):
            return c_vp(a.ctypes.data - off_bytes)
        self._step(None, _p(G), back(d, qi0 // 2), back(r, qi0), back(s, 4 * gi0), back(m8, qi0), back(m8s, 4 * gi0),
                   back(v8, qi0), back(v8s, 4 * gi0), _p(tab), 1, group, dmax, lr, b1, b2, wd, gscale, None,
                   inv_bc1, inv_sqrt_bc2, lrmode, t, adam, None, 1, gi0, n // group, v4)

    def gemm_nn(self, A, B, Cm, M, K, N):
        self._gemm_nn(_p(A), _p(B), _p(Cm), M, K, N)

    def gemm_tn(self, A, B, Cm, M, K, N, beta):
        self._gemm_tn(_p(A), _p(B), _p(Cm), M, K, N, beta)

    def gemm_nt(self, A, B, Cm, M, K, N):
        self._gemm_nt(_p(A), _p(B), _p(Cm), M, K, N)

    def gemm_nn_f64(self, A, B, Cm, M, K, N):
        self._gemm_nn64(_p(A), _p(B), _p(Cm), M, K, N)

    def gemm_tn_f64(self, A, B, Cm, M, K, N):
        self._gemm_tn64(_p(A), _p(B), _p(Cm), M, K, N)

    def gemm_nt_f64(self, A, B, Cm, M, K, N):
        self._gemm_nt64(_p(A), _p(B), _p(Cm), M, K, N)

    def relerr(self, a, b):
        a = np.ascontiguousarray(a, dtype=np.float32)
        b = np.ascontiguousarray(b, dtype=np.float32)
        assert a.size == b.size
        return self._relerr(_p(a), _p(b), a.size)

    def router_topk(self, rt, rprobs, assign, gate, N, E, K, bias=None, bs=0):
        self._router(_p(rt), _p(rprobs), _p(assign), _p(gate), N, E, K, _p(bias), bs)

    def moe_perm(self, assign, N, E, perm, off):
        return self._perm(_p(assign), N, E, _p(perm), _p(off))

    def gather(self, src, perm, Xp, N, D):
        self._gather(_p(src), _p(perm), _p(Xp), N, D)

    def scatter_gate(self, yp, perm, gate, out, N, D):
        self._scatter_gate(_p(yp), _p(perm), _p(gate), _p(out), N, D)

    def scatter_add(self, dXp, perm, dst, N, D):
        self._scatter_add(_p(dXp), _p(perm), _p(dst), N, D)

    def moe_dgate(self, dout, yp, perm, gate, d_gate, dyp, N, D):
        self._dgate(_p(dout), _p(yp), _p(perm), _p(gate), _p(d_gate), _p(dyp), N, D)

    def swiglu(self, G, U, O):
        self._swiglu(_p(G), _p(U), _p(O), G.size)

    def swiglu_bwd(self, Gg, U, dact, dg, du):
        self._swiglu_bwd(_p(Gg), _p(U), _p(dact), _p(dg), _p(du), Gg.size)

    def step_touched(self, P, Gc, d, r, s, m8, m8s, v8, v8s, touched, group, dmax, lr, b1, b2, wd, sref,
                     inv_bc1, inv_sqrt_bc2, t, nt, gs=None, v4=0):
        self._step_touched(_p(P), _p(Gc), _p(d), _p(r), _p(s), _p(m8), _p(m8s), _p(v8), _p(v8s), _p(touched),
                           touched.size, group, dmax, lr, b1, b2, wd, sref, inv_bc1, inv_sqrt_bc2, t, nt,
                           _p(gs) if gs is not None else None, v4)

    def sqsum(self, G):
        part = np.zeros(64, np.float32)
        self._sqsum(_p(G), G.size, _p(part))
        return part

    def gnorm(self, part, nside, clip_side):
        gs = np.zeros(2, np.float32)
        self._gnorm(_p(part), nside, clip_side, _p(gs))
        return gs

    def recip_div_mismatches(self, seed, n):
        return int(self._recip(seed, n))

    def q4n_quantize(self, P, group):
        """returns (bytes as uint8 array, number of raw groups)"""
        cap = 4 * P.size + 4 * ((P.size + group - 1) // group) + 16
        out = np.zeros(cap, np.uint8)
        nraw = C.c_size_t(0)
        n = self._q4n_q(_p(P), P.size, group, _p(out), cap, C.addressof(nraw))
        return out[:n].copy(), int(nraw.value)

    def q4n_dequantize(self, buf, n, group):
        P = np.zeros(n, np.float32)
        ok = self._q4n_d(_p(buf), buf.size, _p(P), n, group)
        return ok, P

    def moe_forward(self, x, w1, w3, w2, assign, gate, out, N, D, F, E, K, bf16_inter=False):
        """returns (rc, ws) -- keep ws for moe_backward, free with moe_ws_free. bf16_inter: the GEMM inputs
        (Xp, ap, dyp, dgp, dup) are stored rounded to bf16 in both directions, as the reference's GPU path does."""
        ws = self._ws_new(N, D, F, E, K)
        self._ws_bf16(ws, 1 if bf16_inter else 0)
        rc = self._moe_fwd(ws, _p(x), _p(w1), _p(w3), _p(w2), _p(assign), _p(gate), _p(out))
        return rc, ws

    def moe_backward(self, ws, x, w1, w3, w2, gate, dout, dx, dgate, Gw1, Gw3, Gw2):
        self._moe_bwd(ws, _p(x), _p(w1), _p(w3), _p(w2), _p(gate), _p(dout), _p(dx), _p(dgate),
                      _p(Gw1), _p(Gw3), _p(Gw2))

    def moe_ws_free(self, ws):
        self._ws_free(ws)

    # ---- deterministic inputs ----
    def normal(self, n, seed, tid, scale=1.0):
        a = np.empty(n, dtype=np.float32)
        self._fill_normal(_p(a), n, seed, tid, scale)
        return a

    def uniform(self, n, seed, tid, lo=0.0, hi=1.0):
        a = np.empty(n, dtype=np.float32)
        self._fill_uniform(_p(a), n, seed, tid, lo, hi)
        return a

    def int8(self, n, seed, tid, lo, hi):
        a = np.empty(n, dtype=np.int8)
        self._fill_int8(_p(a), n, seed, tid, lo, hi)
        return a

    def u8(self, n, seed, tid, lo, hi):
        a = np.empty(n, dtype=np.uint8)
        self._fill_u8(_p(a), n, seed, tid, lo, hi)
        return a

    def digits(self, nq, seed, tid, dmax=7, packed=1):
        a = np.zeros(int(self.qd_bytes(nq, packed)), dtype=np.int8)
        self._fill_digits(_p(a), nq, seed, tid, dmax, packed)
        return a

    def bf16_round(self, a):
        a = np.ascontiguousarray(a, dtype=np.float32).copy()
        self._bf16_n(_p(a), a.size)
        return a


class Ref(_Lib):
    """The reference's own CPU backend (cudalm.cu built with -DCUDALM_CPU)."""

    def __init__(self, path=REF_SO, threads=0):
        super().__init__(path)
        s = self._sig
        s("ref_init", None, [c_i])(threads)
        self.threads = s("ref_threads", c_i, [])
        assert s("ref_sizeof_span", c_i, [])() == SPAN_DTYPE.itemsize
        self.qhashu = s("ref_qhashu", C.c_uint, [c_u64])
        self.qsri = s("ref_qsri", c_i, [c_f, c_u64, c_u64])
        self.qclmp = s("ref_qclmp", c_i, [c_i, c_i, c_i])
        self._qd_get = s("ref_qd_get", c_i, [c_vp, c_u64, c_i])
        self._qd_set = s("ref_qd_set_host", None, [c_vp, c_u64, c_i, c_i])
        self.qd_bytes = s("ref_qd_bytes", c_u64, [c_u64, c_i])
        self.set_qv4 = s("ref_set_qv4", None, [c_i])
        self._encode = s("ref_encode", None, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i])
        self._render = s("ref_render", None, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i])
        self._step = s("ref_step", None, _STEP_ARGS)
        sb = list(_STEP_ARGS)
        del sb[18]  # the block kernel has no gsp
        self._step_block = s("ref_step_block", None, sb)
        self._servo = s("ref_servo", None, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_f, c_f, c_i, c_i])
        g3 = [c_vp, c_vp, c_vp, c_i, c_i, c_i]
        self._g_ab = s("ref_g_ab", None, g3)
        self._g_abt_b = s("ref_g_abt_b", None, g3 + [c_f])
        self._g_atb = s("ref_g_atb", None, g3)
        self._mg_ab = s("ref_mg_ab", None, g3)
        self._mg_abt_b = s("ref_mg_abt_b", None, g3 + [c_f])
        self._mg_atb = s("ref_mg_atb", None, g3)
        self.mg_flush = s("ref_mg_flush", None, [])
        self._router = s("ref_router_topk", None, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_vp, c_i])
        self._gather = s("ref_gather", None, [c_vp, c_vp, c_vp, c_i, c_i])
        self._scatter_gate = s("ref_scatter_gate", None, [c_vp, c_vp, c_vp, c_vp, c_i, c_i])
        self._scatter_add = s("ref_scatter_add", None, [c_vp, c_vp, c_vp, c_i, c_i])
        self._dgate = s("ref_moe_dgate", None, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i])
        self._swiglu = s("ref_swiglu", None, [c_vp, c_vp, c_vp, c_sz])
        self._swiglu_bwd = s("ref_swiglu_bwd", None, [c_vp, c_vp, c_vp, c_vp, c_vp, c_sz])
        self._q4n_q = s("ref_q4n_quantize", c_sz, [c_vp, c_sz, c_i, c_vp, c_sz])
        optq = [c_i, c_i, c_i, c_i, c_vp, c_i, c_u64] + [c_vp] * 9
        self._qlm_save = s("ref_qlm_save", c_i, [C.c_char_p, c_i, c_f] + optq)
        self._qlm_load = s("ref_qlm_load", c_i, [C.c_char_p, c_vp, c_vp] + optq)
        self._ng_step = s("ref_ng_q4_step", None, [c_vp] * 10 + [c_i, c_i, c_i, c_f, c_f, c_f, c_f, c_f, c_f, c_f,
                                                                 C.c_uint64, C.c_uint64, c_vp])
        self._q4n_d = s("ref_q4n_dequantize", c_i, [c_vp, c_sz, c_vp, c_sz, c_i])
        self._relerr = s("ref_relerr", c_f, [c_vp, c_vp, c_sz])
        self._sqsum = s("ref_sqsum", None, [c_vp, C.c_uint64, c_vp])
        self._gnorm = s("ref_gnorm", None, [c_vp, c_i, c_i, c_vp])

    def qd_get(self, d, i, packed):
        return self._qd_get(_p(d), i, packed)

    def qd_set(self, d, i, v, packed):
        self._qd_set(_p(d), i, v, packed)

    def encode(self, P, d, r, s, tab, group, dmax, packed, ngrp):
        self._encode(_p(P), _p(d), _p(r), _p(s), _p(tab), len(tab), group, dmax, packed, ngrp)

    def render(self, P, d, s, tab, group, packed, gi_base, ng):
        self._render(_p(P), _p(d), _p(s), _p(tab), len(tab), group, packed, gi_base, ng)

    def step(self, P, G, d, r, s, m8, m8s, v8, v8s, tab, group, dmax, lr, b1, b2, wd, gscale, gsp,
             inv_bc1, inv_sqrt_bc2, lrmode, t, adam, stat, packed, gi_base, ng, v4=0):
        self.set_qv4(v4)
        self._step(_p(P), _p(G), _p(d), _p(r), _p(s), _p(m8), _p(m8s), _p(v8), _p(v8s), _p(tab), len(tab),
                   group, dmax, lr, b1, b2, wd, gscale, _p(gsp), inv_bc1, inv_sqrt_bc2, lrmode, t, adam,
                   _p(stat), packed, gi_base, ng)
        self.set_qv4(0)

    def step_block(self, P, G, d, r, s, m8, m8s, v8, v8s, tab, group, dmax, lr, b1, b2, wd, gscale,
                   inv_bc1, inv_sqrt_bc2, lrmode, t, adam, stat, packed, gi_base, ng):
        self._step_block(_p(P), _p(G), _p(d), _p(r), _p(s), _p(m8), _p(m8s), _p(v8), _p(v8s), _p(tab),
                         len(tab), group, dmax, lr, b1, b2, wd, gscale, inv_bc1, inv_sqrt_bc2, lrmode, t,
                         adam, _p(stat), packed, gi_base, ng)

    def servo(self, d, r, s, tab, group, dmax, f_hi, f_lo, packed, ngrp):
        self._servo(_p(d), _p(r), _p(s), _p(tab), len(tab), group, dmax, f_hi, f_lo, packed, ngrp)

    def gemm_nn(self, A, B, Cm, M, K, N, grouped=False):
        (self._mg_ab if grouped else self._g_ab)(_p(A), _p(B), _p(Cm), M, K, N)

    def gemm_tn(self, A, B, Cm, M, K, N, beta, grouped=False):
        (self._mg_abt_b if grouped else self._g_abt_b)(_p(A), _p(B), _p(Cm), M, K, N, beta)

    def gemm_nt(self, A, B, Cm, M, K, N, grouped=False):
        (self._mg_atb if grouped else self._g_atb)(_p(A), _p(B), _p(Cm), M, K, N)

    def router_topk(self, rt, rprobs, assign, gate, N, E, K, bias=None, bs=0):
        self._router(_p(rt), _p(rprobs), _p(assign), _p(gate), N, E, K, _p(bias), bs)

    def gather(self, src, perm, Xp, N, D):
        self._gather(_p(src), _p(perm), _p(Xp), N, D)

    def scatter_gate(self, yp, perm, gate, out, N, D):
        self._scatter_gate(_p(yp), _p(perm), _p(gate), _p(out), N, D)

    def scatter_add(self, dXp, perm, dst, N, D):
        self._scatter_add(_p(dXp), _p(perm), _p(dst), N, D)

    def moe_dgate(self, dout, yp, perm, gate, d_gate, dyp, N, D):
        self._dgate(_p(dout), _p(yp), _p(perm), _p(gate), _p(d_gate), _p(dyp), N, D)

    def swiglu(self, G, U, O):
        self._swiglu(_p(G), _p(U), _p(O), G.size)

    def swiglu_bwd(self, Gg, U, dact, dg, du):
        self._swiglu_bwd(_p(Gg), _p(U), _p(dact), _p(dg), _p(du), Gg.size)


def _ref_qlm_save(self, path, iter_, prev_gn, dmax, group, adam, packed, tab, nfloat, Mc, Vc, d, r, m8, v8, s, m8s, v8s):
    """the reference's qlm_save (qlm.cuh:702-738) over host arrays; returns its status"""
    return self._qlm_save(path.encode(), iter_, prev_gn, dmax, group, adam, packed, _p(tab), len(tab), nfloat,
                          _p(Mc), _p(Vc), _p(d), _p(r), _p(m8), _p(v8), _p(s), _p(m8s), _p(v8s))


def _ref_qlm_load(self, path, dmax, group, adam, packed, tab, nfloat, Mc, Vc, d, r, m8, v8, s, m8s, v8s, prev_gn=1.0):
    """the reference's qlm_load (qlm.cuh:740-788) into host arrays; returns (status, iter, prev_gn); tab's sref is updated"""
    it = C.c_int(-1); pg = C.c_float(prev_gn)
    ok = self._qlm_load(path.encode(), C.addressof(it), C.addressof(pg), dmax, group, adam, packed, _p(tab), len(tab), nfloat,
                        _p(Mc), _p(Vc), _p(d), _p(r), _p(m8), _p(v8), _p(s), _p(m8s), _p(v8s))
    return ok, it.value, pg.value


def _ref_q4n_quantize(self, P, group):
    cap = 4 * P.size + 4 * ((P.size + group - 1) // group) + 16
    out = np.zeros(cap, np.uint8)
    n = self._q4n_q(_p(P), P.size, group, _p(out), cap)
    return out[:n].copy()


def _ref_q4n_dequantize(self, buf, n, group):
    P = np.zeros(n, np.float32)
    ok = self._q4n_d(_p(buf), buf.size, _p(P), n, group)
    return ok, P


def _ref_step_touched(self, P, Gc, d, r, s, m8, m8s, v8, v8s, touched, group, dmax, lr, b1, b2, wd, sref,
                      inv_bc1, inv_sqrt_bc2, t, nt, gs=None):
    self._ng_step(_p(P), _p(Gc), _p(d), _p(r), _p(s), _p(m8), _p(m8s), _p(v8), _p(v8s), _p(touched),
                  touched.size, group, dmax, lr, b1, b2, wd, sref, inv_bc1, inv_sqrt_bc2, t, nt,
                  _p(gs) if gs is not None else None)


def _ref_sqsum(self, G):
    part = np.zeros(64, np.float32)
    self._sqsum(_p(G), G.size, _p(part))
    return part


def _ref_gnorm(self, part, nside, clip_side):
    gs = np.zeros(2, np.float32)
    self._gnorm(_p(part), nside, clip_side, _p(gs))
    return gs


Ref.qlm_save = _ref_qlm_save
Ref.qlm_load = _ref_qlm_load
Ref.sqsum = _ref_sqsum
Ref.gnorm = _ref_gnorm
Ref.step_touched = _ref_step_touched
Ref.q4n_quantize = _ref_q4n_quantize
Ref.q4n_dequantize = _ref_q4n_dequantize


def have_ref():
    return os.path.exists(REF_SO)
