"""CPU tests of the oracle's IQ4_NL / IQ4_XS restatement (oxidize-c/src/compute/quantization.c:1401-1459),
the 4-bit codebook formats the reference takes through its dequantise loop (matvec.c:799-831).

What pins it: rows expanded by the compiled reference on raw random blocks (tests/golden/iq4_types.npz,
written by tests/golden/make_golden.py iq4; every nibble, scale nibble and high-bit pair occurs), the
compiled reference live when it is present, and constructions that set one field at a time so that a
swapped nibble half, a wrong scale bit position or a missing -32 fails."""
import os

import numpy as np
import pytest

import oxlibs
from oxidize_amd import synth

O = oxlibs.oracle()
VALUES = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)
TYPES = (("iq4_nl", 26), ("iq4_xs", 27))


def load():
    return np.load(os.path.join(oxlibs.ROOT, "tests", "golden", "iq4_types.npz"))


def f16_bytes(v):
    return np.array([v], np.float16).view(np.uint8)


@pytest.mark.parametrize("name,qt", TYPES)
def test_dequant_bits_vs_reference_goldens_and_live(name, qt):
    g = load()
    rows, cols, rb = (int(v) for v in g[name + "_shape"])
    w = g[name + "_w"]
    for r in range(rows):
        out = np.zeros(cols, np.float32)
        assert O.oxo_dequant_row(qt, w[r * rb:].ctypes.data, cols, out.ctypes.data) == 0
        assert np.array_equal(out.view(np.uint32), g[name + "_bits"][r])
    ref = oxlibs.ref()
    if ref is not None:
        cols = 1024
        rb = synth.row_bytes(qt, cols)
        w = synth.weights(qt, 4, cols, seed=23, stream=qt)
        for r in range(4):
            a, b = np.zeros(cols, np.float32), np.zeros(cols, np.float32)
            assert O.oxo_dequant_row(qt, w[r * rb:].ctypes.data, cols, a.ctypes.data) == 0
            assert ref.oc_quant_dequant_row(qt, w[r * rb:].ctypes.data, rb, b.ctypes.data, cols) == 0
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_iq4_nl_one_field_at_a_time():
    blk = np.zeros(18, np.uint8)
    blk[0:2] = f16_bytes(0.5)
    out = np.zeros(32, np.float32)
    assert O.oxo_dequant_row(26, blk.ctypes.data, 32, out.ctypes.data) == 0
    assert np.all(out == 0.5 * VALUES[0])                      # code 0 is -127, not 0
    for j in (0, 7, 15):
        for nib in (1, 9, 15):
            b = blk.copy()
            b[2 + j] = nib                                     # low nibble of byte j -> value j
            assert O.oxo_dequant_row(26, b.ctypes.data, 32, out.ctypes.data) == 0
            want = np.full(32, 0.5 * VALUES[0], np.float32)
            want[j] = 0.5 * VALUES[nib]
            assert np.array_equal(out, want)
            b = blk.copy()
            b[2 + j] = nib << 4                                # high nibble -> value j + 16
            assert O.oxo_dequant_row(26, b.ctypes.data, 32, out.ctypes.data) == 0
            want = np.full(32, 0.5 * VALUES[0], np.float32)
            want[j + 16] = 0.5 * VALUES[nib]
            assert np.array_equal(out, want)
    assert O.oxo_dequant_row(26, blk.ctypes.data, 48, out.ctypes.data) == 1     # not a whole number of blocks


def test_iq4_xs_one_field_at_a_time():
    base = np.zeros(136, np.uint8)
    base[0:2] = f16_bytes(2.0)
    base[8:] = 0x88                                            # every code 8: value 1
    out = np.zeros(256, np.float32)
    assert O.oxo_dequant_row(27, base.ctypes.data, 256, out.ctypes.data) == 0
    assert np.all(out == 2.0 * -32.0)                          # scale field 0 means -32
    for ib in range(8):
        for lo4, hi2 in ((5, 0), (0, 1), (15, 3), (9, 2)):
            b = base.copy()
            b[4 + ib // 2] = lo4 << (4 * (ib % 2))
            high = hi2 << (2 * ib)
            b[2], b[3] = high & 0xFF, high >> 8
            assert O.oxo_dequant_row(27, b.ctypes.data, 256, out.ctypes.data) == 0
            want = np.full(256, -64.0, np.float32)
            want[32 * ib:32 * ib + 32] = 2.0 * float((lo4 | (hi2 << 4)) - 32)
            assert np.array_equal(out, want), (ib, lo4, hi2)
    # one code at a time: byte j of sub-block ib is values j (low nibble) and j + 16 (high) of that sub-block
    b = base.copy()
    b[4:8] = 0x11                                              # every scale 1 - 32 = -31
    for ib, j, nib in ((0, 0, 0), (3, 5, 15), (7, 15, 4)):
        c = b.copy()
        c[8 + 16 * ib + j] = (8 << 4) | nib
        assert O.oxo_dequant_row(27, c.ctypes.data, 256, out.ctypes.data) == 0
        want = np.full(256, 2.0 * -31.0 * 1.0, np.float32)
        want[32 * ib + j] = np.float32(2.0 * -31.0) * VALUES[nib]
        assert np.array_equal(out, want)
        c = b.copy()
        c[8 + 16 * ib + j] = (nib << 4) | 8
        assert O.oxo_dequant_row(27, c.ctypes.data, 256, out.ctypes.data) == 0
        want = np.full(256, 2.0 * -31.0 * 1.0, np.float32)
        want[32 * ib + j + 16] = np.float32(2.0 * -31.0) * VALUES[nib]
        assert np.array_equal(out, want)


@pytest.mark.parametrize("name,qt", TYPES)
def test_matvec_dequant_vs_reference_and_double_numpy(name, qt):
    """oxo_matvec_dequant sums in double; the compiled reference's SIMD f32 dot (this host's, in the golden
    file, and live) lies within 4e-6 of the sum of magnitudes of it, and numpy's double dot of the
    expanded rows is the same number."""
    g = load()
    rows, cols, rb = (int(v) for v in g[name + "_api_shape"])
    w, x = g[name + "_api_w"], g[name + "_api_x"]
    out, mag = np.zeros(rows, np.float64), np.zeros(rows, np.float64)
    assert O.oxo_matvec_dequant(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, out.ctypes.data, mag.ctypes.data) == 0
    assert np.all(np.abs(g[name + "_api_out"].astype(np.float64) - out) <= 4e-6 * mag)
    deq = np.zeros((rows, cols), np.float32)
    for r in range(rows):
        assert O.oxo_dequant_row(qt, w[r * rb:].ctypes.data, cols, deq[r].ctypes.data) == 0
    assert np.allclose(deq.astype(np.float64) @ x.astype(np.float64), out, rtol=0, atol=1e-9 * mag.max())
    assert np.allclose(np.abs(deq.astype(np.float64) * x.astype(np.float64)).sum(axis=1), mag, rtol=1e-12)
    assert O.oxo_matvec_dequant(13, w.ctypes.data, rows, cols, rb, x.ctypes.data, out.ctypes.data, mag.ctypes.data) == 1
    assert O.oxo_matvec_dequant(qt, w.ctypes.data, rows, cols, rb + 2, x.ctypes.data, out.ctypes.data, mag.ctypes.data) == 1
    ref = oxlibs.ref()
    if ref is not None:
        ref.oc_parallel_set_threads(1)
        got = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, got.ctypes.data, temp.ctypes.data)
        assert np.all(np.abs(got.astype(np.float64) - out) <= 4e-6 * mag)
