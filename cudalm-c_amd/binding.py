"""ctypes view of libqlmx.so. Pointers may be given as ints, torch tensors (data_ptr), numpy arrays
(host pointers, only where the C function takes host memory) or None."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

SPAN_DTYPE = np.dtype(
    [("pof", "<u8"), ("gof", "<u8"), ("qi0", "<u8"), ("n", "<u8"),
     ("gi0", "<i4"), ("ngrp", "<i4"), ("sref", "<f4"), ("_pad", "<i4")])

c_f, c_i, c_u64, c_vp, c_sz = C.c_float, C.c_int, C.c_ulonglong, C.c_void_p, C.c_size_t


class QlmxError(RuntimeError):
    pass


class GemmProb(C.Structure):
    """qlmx_gemm_prob of include/qlmx.h"""
    _fields_ = [("A", c_vp), ("B", c_vp), ("C", c_vp), ("wq", c_u64), ("wg", c_u64), ("M", c_i), ("beta", c_f)]


ACT_F32, ACT_BF16 = 0, 1
MATH_F32, MATH_MFMA, MATH_MFMA_F16 = 0, 1, 2


def lib_path():
    """QLMX_LIB names another build of the library (comparing two builds in one harness)"""
    return os.environ.get("QLMX_LIB") or os.path.join(HERE, "libqlmx.so")


def _ptr(x):
    if x is None:
        return None
    if isinstance(x, (int, np.integer)):
        return int(x)
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    if isinstance(x, np.ndarray):
        return x.ctypes.data
    raise TypeError("cannot take a pointer of %r" % type(x))


# name -> (restype, argtypes). Kept in step with include/qlmx.h; tests check every declared symbol.
_STEP = [c_vp] * 10 + [c_i, c_i, c_i, c_f, c_f, c_f, c_f, c_f, c_vp, c_f, c_f, c_i, c_u64, c_i, c_vp, c_i, c_i, c_i, c_i, c_vp]
SIGNATURES = {
    "qlmx_version": (c_i, []),
    "qlmx_init": (c_i, [c_i]),
    "qlmx_last_error": (C.c_char_p, []),
    "qlmx_device_name": (C.c_char_p, []),
    "qlmx_malloc": (c_i, [C.POINTER(c_vp), c_sz]),
    "qlmx_free": (c_i, [c_vp]),
    "qlmx_memcpy_h2d": (c_i, [c_vp, c_vp, c_sz]),
    "qlmx_memcpy_d2h": (c_i, [c_vp, c_vp, c_sz]),
    "qlmx_memcpy_d2d": (c_i, [c_vp, c_vp, c_sz, c_vp]),
    "qlmx_memset": (c_i, [c_vp, c_i, c_sz, c_vp]),
    "qlmx_sync": (c_i, [c_vp]),
    "qlmx_side_fork": (c_i, [c_vp, C.POINTER(c_vp)]),
    "qlmx_side_join": (c_i, [c_vp]),
    "qlmx_pair_begin": (c_i, [c_vp]),
    "qlmx_pair_end": (c_i, [c_vp]),
    "qlmx_prof_mark": (c_i, [C.c_char_p, c_vp]),
    "qlmx_prof_report": (c_i, [C.c_char_p, C.c_size_t, C.POINTER(c_i)]),
    "qlmx_prof_reset": (c_i, []),
    "qlmx_qhashu": (C.c_uint, [c_u64]),
    "qlmx_qsri": (c_i, [c_f, c_u64, c_u64]),
    "qlmx_qclmp": (c_i, [c_i, c_i, c_i]),
    "qlmx_qd_get": (c_i, [c_vp, c_u64, c_i]),
    "qlmx_qd_set_host": (None, [c_vp, c_u64, c_i, c_i]),
    "qlmx_qd_bytes": (c_u64, [c_u64, c_i]),
    "qlmx_encode": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "qlmx_render": (c_i, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "qlmx_step": (c_i, _STEP),
    "qlmx_servo": (c_i, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_f, c_f, c_i, c_i, c_vp]),
    "qlmx_moe_gemm_nn": (c_i, [c_vp, c_vp, c_i, c_vp, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "qlmx_moe_gemm_tn": (c_i, [c_vp, c_vp, c_i, c_vp, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "qlmx_moe_gemm_tn_pair": (c_i, [c_vp, c_vp, c_i, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "qlmx_moe_gemm_nn_swiglu": (c_i, [c_vp, c_vp, c_i, c_vp, c_vp, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "qlmx_moe_gemm_nn_gather": (c_i, [c_vp, c_vp, c_i, c_vp, c_i, c_i, c_i, c_vp, c_vp]),
    "qlmx_moe_gemm_nn_gather_swiglu": (c_i, [c_vp, c_vp, c_i, c_vp, c_vp, c_i, c_i, c_i, c_vp, c_vp]),
    "qlmx_moe_gemm_tn_swiglu_bwd": (c_i, [c_vp, c_vp, c_i, c_vp, c_i, c_i, c_i, c_vp, c_vp, c_vp, c_vp, c_vp]),
    "qlmx_moe_gemm_nn_scatter": (c_i, [c_vp, c_vp, c_i, c_vp, c_i, c_i, c_i, c_vp, c_vp, c_vp]),
    "qlmx_moe_gemm_tn_pair_scatter": (c_i, [c_vp, c_vp, c_i, c_vp, c_vp, c_i, c_i, c_i, c_vp, c_vp]),
    "qlmx_moe_gemm_nt": (c_i, [c_vp, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "qlmx_moe_decode_forward": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_u64, c_u64, c_u64, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "qlmx_moe_decode_forward_noalloc": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_u64, c_u64, c_u64, c_i, c_i, c_i, c_i, c_i, c_vp]),
    "qlmx_decode_status": (c_i, []),
    "qlmx_test_force_wait_timeout": (c_i, [c_i]),
    "qlmx_nt_tile": (c_i, [c_i]),
    "qlmx_decode_math": (c_i, [c_i]),
    "qlmx_test_sqrt_form": (c_i, [C.c_uint, c_u64, c_vp, c_vp]),
    "qlmx_test_div_form": (c_i, [c_u64, c_u64, c_vp, c_vp]),
    "qlmx_test_step_wide": (c_i, [c_i]),
    "qlmx_step_touched": (c_i, [c_vp] * 10 + [c_i, c_i, c_i, c_f, c_f, c_f, c_f, c_f, c_f, c_f, c_u64, c_u64, c_vp, c_i, c_vp]),
    "qlmx_sqsum": (c_i, [c_vp, c_u64, c_vp, c_vp]),
    "qlmx_gnorm": (c_i, [c_vp, c_i, c_i, c_vp, c_vp]),
    "qlmx_router_topk": (c_i, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_vp, c_i, c_vp]),
    "qlmx_moe_perm_workspace": (c_sz, [c_i, c_i, c_i]),
    "qlmx_moe_perm": (c_i, [c_vp, c_i, c_i, c_i, c_vp, c_vp, c_vp, c_vp]),
    "qlmx_moe_perm_status": (c_i, [c_vp, c_i, c_i, c_i, c_vp]),
    "qlmx_moe_gather": (c_i, [c_vp, c_vp, c_vp, c_i, c_i, c_i, c_vp]),
    "qlmx_moe_scatter_gate": (c_i, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_vp]),
    "qlmx_moe_scatter_add": (c_i, [c_vp, c_vp, c_vp, c_i, c_i, c_vp]),
    "qlmx_moe_dgate": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_vp]),
    "qlmx_moe_dgate_merged": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_i, c_vp]),
    "qlmx_moe_merge_rows": (c_i, [c_vp, c_i, c_i, c_vp, c_vp, c_vp]),
    "qlmx_moe_combine": (c_i, [c_vp, c_vp, c_vp, c_vp, c_i, c_i, c_i, c_vp]),
    "qlmx_swiglu": (c_i, [c_vp, c_vp, c_vp, c_sz, c_i, c_vp]),
    "qlmx_swiglu_bwd": (c_i, [c_vp, c_vp, c_vp, c_vp, c_vp, c_sz, c_i, c_vp]),
    "qlmx_q4n_bound": (c_sz, [c_sz, c_i]),
    "qlmx_q4n_quantize": (c_i, [c_vp, c_sz, c_i, c_vp, c_sz, c_vp, c_vp]),
    "qlmx_q4n_dequantize": (c_i, [c_vp, c_sz, c_vp, c_sz, c_i, c_vp]),
}


class Qlmx:
    """Loaded library. `init=True` binds device 0 and raises if that fails."""

    def __init__(self, path=None, init=True, device=0):
        path = path or lib_path()
        if not os.path.exists(path):
            raise QlmxError("libqlmx.so is not built (%s): run `python cudalm-c_amd/build.py`" % path)
        self.lib = C.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            f = getattr(self.lib, name)
            f.restype, f.argtypes = res, args
        if init:
            self.check(self.lib.qlmx_init(device))

    def last_error(self):
        return self.lib.qlmx_last_error().decode()

    def check(self, rc):
        if rc != 0:
            raise QlmxError("libqlmx error %d: %s" % (rc, self.last_error()))

    def call(self, name, *args):
        conv = []
        for a, t in zip(args, SIGNATURES[name][1]):
            conv.append(_ptr(a) if t is c_vp else a)
        rc = getattr(self.lib, name)(*conv)
        if SIGNATURES[name][0] is c_i and name not in ("qlmx_version", "qlmx_qsri", "qlmx_qclmp", "qlmx_qd_get"):
            self.check(rc)
        return rc

    # convenience wrappers with the reference's argument order
    def encode(self, P, d, r, s, sp, nspan, group, dmax, packed, ngrp, stream=None):
        self.call("qlmx_encode", P, d, r, s, sp, nspan, group, dmax, packed, ngrp, stream)

    def render(self, P, d, s, sp, nspan, group, packed, gi_base, ng, stream=None):
        self.call("qlmx_render", P, d, s, sp, nspan, group, packed, gi_base, ng, stream)

    def step(self, P, G, d, r, s, m8, m8s, v8, v8s, sp, nspan, group, dmax, lr, b1, b2, wd, gscale, gsp,
             inv_bc1, inv_sqrt_bc2, lrmode, t, adam, stat, packed, gi_base, ng, v4=0, stream=None):
        self.call("qlmx_step", P, G, d, r, s, m8, m8s, v8, v8s, sp, nspan, group, dmax, lr, b1, b2, wd, gscale,
                  gsp, inv_bc1, inv_sqrt_bc2, lrmode, t, adam, stat, packed, gi_base, ng, v4, stream)

    def servo(self, d, r, s, sp, nspan, group, dmax, f_hi, f_lo, packed, ngrp, stream=None):
        self.call("qlmx_servo", d, r, s, sp, nspan, group, dmax, f_hi, f_lo, packed, ngrp, stream)

    @staticmethod
    def problems(items):
        """items: iterable of dicts/tuples (A, B, C, wq, wg, M, beta) with tensors or ints as pointers"""
        arr = (GemmProb * max(1, len(items)))()
        for i, (A, B, Cc, wq, wg, M, beta) in enumerate(items):
            arr[i].A, arr[i].B, arr[i].C = _ptr(A), _ptr(B), _ptr(Cc)
            arr[i].wq, arr[i].wg, arr[i].M, arr[i].beta = int(wq), int(wg), int(M), float(beta)
        return arr

    def gemm_nn(self, d, s, group, probs, nprob, K, N, act=ACT_F32, math=MATH_F32, stream=None):
        self.call("qlmx_moe_gemm_nn", d, s, group, C.addressof(probs), nprob, K, N, act, math, stream)

    def gemm_tn(self, d, s, group, probs, nprob, K, N, act=ACT_F32, math=MATH_F32, stream=None):
        self.call("qlmx_moe_gemm_tn", d, s, group, C.addressof(probs), nprob, K, N, act, math, stream)

    def gemm_tn_pair(self, d, s, group, first, second, nprob, K, N, act=ACT_F32, math=MATH_F32, stream=None):
        self.call("qlmx_moe_gemm_tn_pair", d, s, group, C.addressof(first), C.addressof(second), nprob, K, N, act, math, stream)

    def gemm_nn_swiglu(self, d, s, group, gate, up, nprob, K, N, act=ACT_F32, math=MATH_F32, stream=None):
        self.call("qlmx_moe_gemm_nn_swiglu", d, s, group, C.addressof(gate), C.addressof(up), nprob, K, N, act, math, stream)

    def gemm_nn_gather(self, d, s, group, probs, nprob, K, N, x_bf16, stream=None):
        self.call("qlmx_moe_gemm_nn_gather", d, s, group, C.addressof(probs), nprob, K, N, x_bf16, stream)

    def gemm_nn_gather_swiglu(self, d, s, group, gate, up, nprob, K, N, x_bf16, stream=None):
        self.call("qlmx_moe_gemm_nn_gather_swiglu", d, s, group, C.addressof(gate), C.addressof(up), nprob, K, N, x_bf16, stream)

    def gemm_tn_swiglu_bwd(self, d, s, group, probs, nprob, K, N, gp, up, dgp, dup, stream=None):
        self.call("qlmx_moe_gemm_tn_swiglu_bwd", d, s, group, C.addressof(probs), nprob, K, N, gp, up, dgp, dup, stream)

    def gemm_nn_scatter(self, d, s, group, probs, nprob, K, N, out, gate, stream=None):
        self.call("qlmx_moe_gemm_nn_scatter", d, s, group, C.addressof(probs), nprob, K, N, out, gate, stream)

    def gemm_tn_pair_scatter(self, d, s, group, first, second, nprob, K, N, dst, stream=None):
        self.call("qlmx_moe_gemm_tn_pair_scatter", d, s, group, C.addressof(first), C.addressof(second), nprob, K, N, dst, stream)

    def gemm_nt(self, probs, nprob, K, N, act=ACT_F32, math=MATH_F32, stream=None):
        self.call("qlmx_moe_gemm_nt", C.addressof(probs), nprob, K, N, act, math, stream)

    def decode_forward(self, x, assign, gate, out, d, s, group, w1q, w3q, w2q, T, K, E, D, F, stream=None):
        self.call("qlmx_moe_decode_forward", x, assign, gate, out, d, s, group, w1q, w3q, w2q, T, K, E, D, F, stream)

    def decode_forward_noalloc(self, x, assign, gate, out, d, s, group, w1q, w3q, w2q, T, K, E, D, F, stream=None):
        self.call("qlmx_moe_decode_forward_noalloc", x, assign, gate, out, d, s, group, w1q, w3q, w2q, T, K, E, D, F, stream)

    def step_touched(self, P, Gc, d, r, s, m8, m8s, v8, v8s, touched, ntouched, group, dmax, lr, b1, b2, wd, sref,
                     inv_bc1, inv_sqrt_bc2, t, nt, gs=None, v4=0, stream=None):
        self.call("qlmx_step_touched", P, Gc, d, r, s, m8, m8s, v8, v8s, touched, ntouched, group, dmax, lr, b1, b2, wd, sref,
                  inv_bc1, inv_sqrt_bc2, t, nt, gs, v4, stream)

    def sqsum(self, G, n, part64, stream=None):
        self.call("qlmx_sqsum", G, n, part64, stream)

    def gnorm(self, part, nside, clip_side, gs, stream=None):
        self.call("qlmx_gnorm", part, nside, clip_side, gs, stream)

    # MoE glue (argument order of the reference kernels)
    def router_topk(self, rt, rprobs, assign, gate, N, E, K, bias=None, bs=0, stream=None):
        self.call("qlmx_router_topk", rt, rprobs, assign, gate, N, E, K, bias, bs, stream)

    def moe_perm_workspace(self, N, E, K):
        return int(self.lib.qlmx_moe_perm_workspace(N, E, K))

    def moe_perm(self, assign, N, E, K, perm, off, workspace, stream=None):
        self.call("qlmx_moe_perm", assign, N, E, K, perm, off, workspace, stream)

    def moe_perm_status(self, workspace, N, E, K, stream=None):
        self.call("qlmx_moe_perm_status", workspace, N, E, K, stream)

    def moe_gather(self, src, perm, Xp, N, D, out_dtype=ACT_F32, stream=None):
        self.call("qlmx_moe_gather", src, perm, Xp, N, D, out_dtype, stream)

    def moe_scatter_gate(self, yp, perm, gate, out, N, D, stream=None):
        self.call("qlmx_moe_scatter_gate", yp, perm, gate, out, N, D, stream)

    def moe_scatter_add(self, dXp, perm, dst, N, D, stream=None):
        self.call("qlmx_moe_scatter_add", dXp, perm, dst, N, D, stream)

    def moe_dgate_merged(self, dout, yp, perm, gate, d_gate, dyp, N, K, D, out_dtype=ACT_F32, stream=None):
        self.call("qlmx_moe_dgate_merged", dout, yp, perm, gate, d_gate, dyp, N, K, D, out_dtype, stream)

    def moe_merge_rows(self, perm, N, K, tok, inv, stream=None):
        self.call("qlmx_moe_merge_rows", perm, N, K, tok, inv, stream)

    def moe_combine(self, y, inv, gate, out, N, K, D, stream=None):
        self.call("qlmx_moe_combine", y, inv, gate, out, N, K, D, stream)

    def moe_dgate(self, dout, yp, perm, gate, d_gate, dyp, N, D, out_dtype=ACT_F32, stream=None):
        self.call("qlmx_moe_dgate", dout, yp, perm, gate, d_gate, dyp, N, D, out_dtype, stream)

    def swiglu(self, G, U, O, n, out_dtype=ACT_F32, stream=None):
        self.call("qlmx_swiglu", G, U, O, n, out_dtype, stream)

    def swiglu_bwd(self, Gg, U, dact, dg, du, n, out_dtype=ACT_F32, stream=None):
        self.call("qlmx_swiglu_bwd", Gg, U, dact, dg, du, n, out_dtype, stream)

    # q4n wire format (host memory, numpy arrays)
    def q4n_quantize(self, P, group):
        """P: fp32 numpy array -> (uint8 numpy array in the wire format, number of raw groups)"""
        import numpy as np
        cap = int(self.lib.qlmx_q4n_bound(P.size, group))
        out = np.zeros(max(cap, 1), np.uint8)
        n, raw = C.c_size_t(0), C.c_size_t(0)
        self.call("qlmx_q4n_quantize", P, P.size, group, out, cap, C.addressof(n), C.addressof(raw))
        return out[:n.value].copy(), int(raw.value)

    def q4n_dequantize(self, buf, n, group):
        import numpy as np
        P = np.zeros(n, np.float32)
        used = C.c_size_t(0)
        self.call("qlmx_q4n_dequantize", buf, buf.size, P, n, group, C.addressof(used))
        return P, int(used.value)

    def sync(self, stream=None):
        self.call("qlmx_sync", stream)

    def side_fork(self, stream=None):
        """The library's side stream, ordered after what `stream` holds so far (a handle to pass as `stream`)."""
        side = C.c_void_p()
        self.call("qlmx_side_fork", stream, C.byref(side))
        return side.value

    def side_join(self, stream=None):
        self.call("qlmx_side_join", stream)

    def prof_mark(self, label, stream=None):
        """An event on `stream`; the GPU time since the previous mark is charged to `label` (qlmx_prof_mark)."""
        self.call("qlmx_prof_mark", label.encode(), stream)

    def prof_report(self):
        """(text of the table, number of labels) of qlmx_prof_report"""
        buf = C.create_string_buffer(8192); n = C.c_int(0)
        self.call("qlmx_prof_report", buf, len(buf), C.byref(n))
        return buf.value.decode(), int(n.value)

    def pair_begin(self, stream=None):
        """Hold back the next input-gradient and weight-gradient launches on `stream` (qlmx_pair_begin)."""
        self.call("qlmx_pair_begin", stream)

    def pair_end(self, stream=None):
        """Issue what qlmx_pair_begin held back, as one launch when both kinds are there."""
        self.call("qlmx_pair_end", stream)


_cached = None


def load(init=True):
    global _cached
    if _cached is None:
        _cached = Qlmx(init=init)
    return _cached
