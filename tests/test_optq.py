"""The .opt.q checkpoint format of the host mirror (cudalm-c_amd/host/qlm_host.cpp: qlm_save / qlm_load and the
host-memory entry points over the same writer and reader) against files written by the reference's own
qlm_save (qlm.cuh:702-738; fixtures tests/golden/optq_*.npz, made by tests/golden/make_golden.py): the reader
recovers every array, the iteration, the previous gradient norm and the frozen reference scales; the writer
reproduces the reference's file byte for byte; where the reference build is present its own qlm_load reads
what the mirror wrote. No GPU needed: these entry points work on host memory."""
import ctypes as C
import os

import numpy as np
import pytest

from __graft_entry__ import PKG_DIR
from oracle.binding import SPAN_DTYPE

HOST_SO = os.path.join(PKG_DIR, "libqlmx_host.so")
vp = C.c_void_p


class OptqHost(C.Structure):
    """QlmOptqHost of cudalm-c_amd/host/qlm_host.h"""
    _fields_ = [("dmax", C.c_int), ("group", C.c_int), ("adam", C.c_int), ("nspan", C.c_int), ("packed", C.c_int), ("iter", C.c_int),
                ("nq", C.c_ulonglong), ("ngrp", C.c_ulonglong), ("nfloat", C.c_ulonglong),
                ("Mc", vp), ("Vc", vp), ("d", vp), ("r", vp), ("m8", vp), ("v8", vp), ("s", vp), ("m8s", vp), ("v8s", vp), ("sref", vp),
                ("prev_gn", C.c_float), ("have_sref", C.c_int)]


@pytest.fixture(scope="module")
def host():
    if not os.path.exists(HOST_SO):
        pytest.fail("libqlmx_host.so is not built: run python cudalm-c_amd/build.py")
    lib = C.CDLL(HOST_SO)
    lib.qlm_optq_write_host.restype = C.c_int; lib.qlm_optq_write_host.argtypes = [C.c_char_p, C.POINTER(OptqHost)]
    lib.qlm_optq_read_host.restype = C.c_int; lib.qlm_optq_read_host.argtypes = [C.c_char_p, C.POINTER(OptqHost)]
    return lib


NAMES = ["Mc", "Vc", "d", "r", "m8", "v8", "s", "m8s", "v8s"]


def poisoned(g):
    """arrays of the fixture's shapes with every byte 0x55"""
    out = {}
    for n in NAMES:
        a = np.zeros_like(g[n]); a.view(np.uint8)[:] = 0x55
        out[n] = a
    return out


def view(g, arrays, sref):
    dmax, group, adam, packed, it, nfloat = (int(x) for x in g["dims"])
    tab = g["tab"].view(SPAN_DTYPE)
    v = OptqHost()
    v.dmax, v.group, v.adam, v.nspan, v.packed, v.iter = dmax, group, adam, len(tab), packed, it
    v.nq = int(tab["n"].sum()); v.ngrp = int(tab["ngrp"].sum()); v.nfloat = nfloat
    for n in NAMES:
        setattr(v, n, arrays[n].ctypes.data if (adam or n not in ("v8", "v8s")) else None)
    v.sref = sref.ctypes.data
    v.prev_gn = float(g["prev_gn"][0]); v.have_sref = 0
    return v, tab


@pytest.mark.parametrize("tag", ["adam", "lion"])
def test_reader_recovers_a_reference_written_file(host, golden, tmp_path, tag):
    g = golden("optq_" + tag)
    path = str(tmp_path / "ref.opt.q")
    g["optq"].tofile(path)
    blank = poisoned(g)
    sref = np.zeros(2, np.float32)
    v, tab = view(g, blank, sref)
    v.iter = -1; v.prev_gn = 1.0
    assert host.qlm_optq_read_host(path.encode(), C.byref(v)) == 1
    adam = int(g["dims"][2])
    for n in NAMES:
        if adam or n not in ("v8", "v8s"):
            assert np.array_equal(blank[n].view(np.uint8), g[n].view(np.uint8)), n
        else:
            assert np.all(blank[n].view(np.uint8) == 0x55), n + " must not be touched for the sign optimizer"
    assert v.iter == 4321 and v.prev_gn == 2.5 and v.have_sref == 1
    assert np.array_equal(sref, tab["sref"])


@pytest.mark.parametrize("tag", ["adam", "lion"])
def test_writer_reproduces_the_reference_file_byte_for_byte(host, golden, tmp_path, tag):
    g = golden("optq_" + tag)
    arrays = {n: g[n].copy() for n in NAMES}
    tab0 = g["tab"].view(SPAN_DTYPE)
    sref = tab0["sref"].astype(np.float32).copy()
    v, _ = view(g, arrays, sref)
    path = str(tmp_path / "mine.opt.q")
    assert host.qlm_optq_write_host(path.encode(), C.byref(v)) == 1
    assert not os.path.exists(path + ".tmp")
    mine = np.fromfile(path, dtype=np.uint8)
    assert np.array_equal(mine, g["optq"])


def test_reference_reader_loads_what_the_mirror_wrote(host, golden, ref, tmp_path):
    g = golden("optq_adam")
    arrays = {n: g[n].copy() for n in NAMES}
    tab0 = g["tab"].view(SPAN_DTYPE).copy()
    sref = tab0["sref"].astype(np.float32).copy()
    v, _ = view(g, arrays, sref)
    path = str(tmp_path / "mine.opt.q")
    assert host.qlm_optq_write_host(path.encode(), C.byref(v)) == 1
    blank = {n: np.zeros_like(g[n]) for n in NAMES}
    tab = tab0.copy(); tab["sref"] = 0
    ok, it, pg = ref.qlm_load(path, 7, 128, 1, 1, tab, int(g["dims"][5]), *[blank[n] for n in NAMES])
    assert ok == 1 and it == 4321 and pg == 2.5
    for n in NAMES:
        assert np.array_equal(blank[n].view(np.uint8), g[n].view(np.uint8)), n
    assert np.array_equal(tab["sref"], tab0["sref"])


def test_truncated_and_foreign_files_leave_the_state_alone(host, golden, tmp_path):
    g = golden("optq_adam")
    data = g["optq"]
    blank = poisoned(g)
    sref = np.zeros(2, np.float32)
    trailer = 4 + 4 + 2 * 4 + 4 + 4
    for name, cut in (("short", data[:len(data) - trailer - 10]), ("magic", np.concatenate([np.frombuffer(b"QLMX", np.uint8), data[4:]]))):
        path = str(tmp_path / (name + ".opt.q"))
        cut.tofile(path)
        v, _ = view(g, blank, sref)
        assert host.qlm_optq_read_host(path.encode(), C.byref(v)) == 0, name
        for n in NAMES:
            assert np.all(blank[n].view(np.uint8) == 0x55), (name, n)
    # another group size in the header: refused as a different shape
    other = data.copy(); other[8:12] = np.frombuffer(np.int32(64).tobytes(), np.uint8)
    path = str(tmp_path / "shape.opt.q"); other.tofile(path)
    v, _ = view(g, blank, sref)
    assert host.qlm_optq_read_host(path.encode(), C.byref(v)) == 0
    # a file from before the trailers existed: state loads, the reference scales are reported missing
    path = str(tmp_path / "old.opt.q"); data[:len(data) - trailer].tofile(path)
    v, _ = view(g, blank, sref)
    v.prev_gn = 1.0
    assert host.qlm_optq_read_host(path.encode(), C.byref(v)) == 1 and v.have_sref == 0 and v.prev_gn == 1.0
    assert np.array_equal(blank["d"], g["d"])
