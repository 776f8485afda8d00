"""CPU-side checks of the C ABI: the library loads, exports every symbol include/qlmx.h declares,
the host integer helpers agree with the golden vectors, and compute entry points refuse to run
without a bound gfx950 device (there is no CPU fallback)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from __graft_entry__ import load_package, ROOT

pkg = load_package()


def declared_symbols():
    txt = open(os.path.join(ROOT, "include", "qlmx.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(qlmx_[a-z0-9_]+)\s*\(", txt)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(pkg.lib_path()):
        pytest.fail("libqlmx.so not built: run python cudalm-c_amd/build.py (or __graft_entry__.build())")
    return pkg.Qlmx(init=False)


def test_every_declared_symbol_is_exported_and_bound(lib):
    names = declared_symbols()
    assert len(names) >= 20
    raw = C.CDLL(pkg.lib_path())
    for n in names:
        assert hasattr(raw, n), "libqlmx.so does not export %s" % n
    from cudalm_c_amd.binding import SIGNATURES
    assert sorted(SIGNATURES) == names, "binding.SIGNATURES out of step with include/qlmx.h"


def test_span_layout_matches_reference_struct():
    assert pkg.SPAN_DTYPE.itemsize == 48
    assert [pkg.SPAN_DTYPE.fields[k][1] for k in ("pof", "gof", "qi0", "n", "gi0", "ngrp", "sref")] == [0, 8, 16, 24, 32, 36, 40]


def test_host_helpers_match_golden(lib, golden):
    g = golden("hash")
    assert [lib.call("qlmx_qhashu", int(x)) for x in g["x"]] == [int(h) for h in g["h"]]
    got = [lib.call("qlmx_qsri", float(v), int(i), int(t)) for v, i, t in zip(g["v"], g["i"], g["t"])]
    assert got == [int(q) for q in g["q"]]
    n = golden("nibble")
    nq = len(n["vals"])
    d = np.zeros(int(lib.call("qlmx_qd_bytes", nq, 1)), np.int8)
    for k in range(nq):
        lib.call("qlmx_qd_set_host", d, k, int(n["vals"][k]), 1)
    assert np.array_equal(d, n["packed"])
    assert [lib.call("qlmx_qd_get", d, k, 1) for k in range(nq)] == [int(v) for v in n["back"]]
    assert lib.call("qlmx_qclmp", 9, -7, 7) == 7 and lib.call("qlmx_qclmp", -9, -7, 7) == -7


def test_compute_refuses_without_device(lib):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present; the refusal path is for CPU-only hosts")
    with pytest.raises(pkg.QlmxError):
        lib.call("qlmx_init", 0)
    buf = np.zeros(256, np.float32)
    rc = lib.lib.qlmx_render(buf.ctypes.data, buf.ctypes.data, buf.ctypes.data, buf.ctypes.data, 1, 128, 1, 0, 1, None)
    assert rc == -3 and "qlmx_init" in lib.last_error()
