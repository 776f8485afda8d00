"""q4n wire format (quantize_params / dequantize_params qtype 3, cudalm.cu:638-656, 688-696): the
oracle's restatement and the library's host functions against the bytes the compiled reference wrote
(tests/golden/q4n.npz). Host code only, so these run without a GPU; byte-exact both ways."""
import numpy as np
import pytest

from __graft_entry__ import load_package

pkg = load_package()
f32 = np.float32


@pytest.fixture(scope="module")
def lib():
    return pkg.Qlmx(init=False)


def test_oracle_matches_reference_bytes(orc, golden):
    g = golden("q4n")
    n, group = (int(v) for v in g["dims"])
    buf, nraw = orc.q4n_quantize(g["P"], group)
    assert nraw == 1
    assert np.array_equal(buf, g["buf"])
    ok, back = orc.q4n_dequantize(g["buf"], n, group)
    assert ok == 1 and np.array_equal(back.view(np.uint32), g["back"].view(np.uint32))
    assert np.array_equal(back.view(np.uint32), g["P"].view(np.uint32))       # the format is lossless here
    b64, _ = orc.q4n_quantize(g["P"][:300], 64)
    assert np.array_equal(b64, g["buf64"])


def test_library_matches_reference_bytes(lib, golden):
    g = golden("q4n")
    n, group = (int(v) for v in g["dims"])
    buf, nraw = lib.q4n_quantize(g["P"], group)
    assert nraw == 1 and np.array_equal(buf, g["buf"])
    back, used = lib.q4n_dequantize(g["buf"], n, group)
    assert used == g["buf"].size
    assert np.array_equal(back.view(np.uint32), g["back"].view(np.uint32))
    b64, _ = lib.q4n_quantize(g["P"][:300], 64)
    assert np.array_equal(b64, g["buf64"])


def test_layout_closed_form(lib):
    """One group written by hand: scale 0.25, digits -7..7 cycling -> 4 + 64 bytes, nibble rule
    ((b & 15) ^ 8) - 8 with the even element in the low nibble."""
    d = (np.arange(128) % 15 - 7).astype(f32)
    P = (d * f32(0.25)).astype(f32)
    buf, nraw = lib.q4n_quantize(P, 128)
    assert nraw == 0 and buf.size == 4 + 64
    assert buf[:4].view(f32)[0] == f32(0.25)          # amax/7 = 0.25 exactly
    lo = ((buf[4:] & 15).astype(int) ^ 8) - 8
    hi = ((buf[4:] >> 4).astype(int) ^ 8) - 8
    assert np.array_equal(lo, d[0::2]) and np.array_equal(hi, d[1::2])


def test_rendered_qlm_view_round_trips_without_raw_groups(lib, orc):
    from oracle.binding import make_spans
    n, group = 128 * 40, 128
    tab, nq, ng = make_spans([n], group)
    P = orc.normal(n, 5, 1, 0.02)
    d = np.zeros(nq // 2, np.int8); r = np.zeros(nq, np.int8); s = np.zeros(ng, f32)
    orc.encode(P, d, r, s, tab, group, 7, 1, ng)
    orc.render(P, d, s, tab, group, 1, 0, ng)
    buf, nraw = lib.q4n_quantize(P, group)
    assert nraw == 0 and buf.size == ng * (4 + 64)
    back, _ = lib.q4n_dequantize(buf, n, group)
    assert np.array_equal(back.view(np.uint32), P.view(np.uint32))
    ob, oraw = orc.q4n_quantize(P, group)
    assert oraw == 0 and np.array_equal(ob, buf)


def test_truncated_buffer_is_refused(lib, orc, golden):
    g = golden("q4n")
    n, group = (int(v) for v in g["dims"])
    for cut in (3, 40, g["buf"].size - 1):
        with pytest.raises(pkg.QlmxError, match="buffer ends"):
            lib.q4n_dequantize(g["buf"][:cut].copy(), n, group)
        ok, _ = orc.q4n_dequantize(g["buf"][:cut].copy(), n, group)
        assert ok == 0


def test_against_reference_library_when_present(lib, orc, ref):
    rng = np.random.default_rng(7)
    for group in (128, 64, 32):
        n = group * 9 + 10
        s = f32(0.0173)
        P = (rng.integers(-7, 8, n).astype(f32) * s).astype(f32)
        P[group:2 * group] = rng.normal(size=group).astype(f32)
        want = ref.q4n_quantize(P, group)
        got, _ = lib.q4n_quantize(P, group)
        ob, _ = orc.q4n_quantize(P, group)
        assert np.array_equal(got, want) and np.array_equal(ob, want)
