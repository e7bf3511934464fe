"""The oracle's restatements of the two codebook formats (IQ3_S, IQ1_XXXS) against vectors from the
compiled reference (tests/golden/iq_types.npz, written by tests/golden/make_golden.py iq), against the
compiled reference live where it is present, and against constructions that isolate one value at a time
so that a wrong index, sign bit or codebook byte cannot hide."""
import os

import numpy as np
import pytest

import oxlibs
from oxidize_amd import synth

O = oxlibs.oracle()
HERE = os.path.dirname(os.path.abspath(__file__))


def load(name):
    return np.load(os.path.join(HERE, "golden", name))


def f32bits(x):
    return int(np.float32(x).view(np.uint32))


@pytest.mark.parametrize("name", ["iq3_s", "iq1_xxxs"])
def test_raw_block_dots_float_bits_vs_reference(name):
    g = load("iq_types.npz")
    fo = getattr(O, "oxo_dot_%s_q8_k" % name)
    w, act = g[name + "_raw_w"], g[name + "_raw_act"]
    for t in range(w.shape[0]):
        wt, at = np.ascontiguousarray(w[t]), np.ascontiguousarray(act[t])
        for k, blocks in enumerate((1, w.shape[1])):
            got = f32bits(fo(wt.ctypes.data, blocks, at.ctypes.data, None))
            assert got == g[name + "_raw_scalar_bits"][t, k]
            assert got == g[name + "_raw_dispatched_bits"][t, k]


@pytest.mark.parametrize("qt", [25, 36])
def test_matvec_and_batch_vs_reference_goldens(qt):
    g = load("iq_types.npz")
    key = "api%d_" % qt
    rows, cols, rb = (int(v) for v in g[key + "shape"])
    w, x = g[key + "w"], g[key + "x"]
    assert O.oxo_act_kind(qt, cols) == 2 and O.oxo_stride_ok(qt, cols, rb) == 1 and O.oxo_act_kind(qt, 300) == 0
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert O.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data,
                                  out.ctypes.data, temp.ctypes.data) == 0
    act = g[key + "act"]
    assert np.array_equal(temp.view(np.uint8)[:act.size], act)
    assert np.array_equal(out.view(np.uint32), g[key + "out_bits"])
    xs = g[key + "batch_x"]
    n_vec, in_stride = xs.shape
    want = g[key + "batch_out_bits"]
    out_stride = want.shape[1]
    outs = np.full((n_vec, out_stride), -1.0, np.float32)
    scratch = np.zeros(O.oxo_matvec_batch_scratch_bytes(cols), np.uint8)
    assert O.oxo_matvec_quantized_batch(qt, w.ctypes.data, rows, cols, rb, xs.ctypes.data, in_stride,
                                        outs.ctypes.data, out_stride, n_vec, scratch.ctypes.data,
                                        scratch.nbytes) == 0
    assert np.array_equal(outs.view(np.uint32), want)


@pytest.mark.parametrize("qt,name", [(25, "big_iq3_s_2048x4096"), (36, "big_iq1_xxxs_2048x4096")])
def test_full_size_vs_reference_checksums(qt, name):
    import zlib
    g = load("iq_types.npz")
    rows, cols = 2048, 4096
    w = synth.weights(qt, rows, cols, seed=0, stream=0)
    assert zlib.crc32(w.tobytes()) == int(g[name + "_crc_w"][0])
    x = synth.normal(cols, seed=0, stream=1000)
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert O.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, synth.row_bytes(qt, cols), x.ctypes.data,
                                  out.ctypes.data, temp.ctypes.data) == 0
    assert zlib.crc32(out.tobytes()) == int(g[name + "_crc_out"][0])


def one_hot_act(e):
    act = np.zeros(292, np.uint8)
    act[0:4] = np.frombuffer(np.float32(1.0).tobytes(), np.uint8)
    q = np.zeros(256, np.int8)
    q[e] = 1
    act[4:260] = q.view(np.uint8)
    bs = q.reshape(16, 16).sum(axis=1).astype(np.int16)
    act[260:292] = bs.view(np.uint8)
    return act


def test_iq3_s_every_element_is_the_dequantised_weight():
    """With d = 1, activation scale 1 and a single activation value of 1 at position e, the dot is the
    weight at e: +-magnitude * (2*nibble + 1).  Checked for all 256 positions of random blocks against a
    numpy reading of the layout (code byte + ninth bit -> codebook byte e%4; sign bit e%8 of byte e/8 of
    the group), and the eight integer lanes against the position's lane."""
    rng = np.random.default_rng(5)
    import re
    text = open(os.path.join(oxlibs.ROOT, "oxidize_amd", "csrc", "iq_grids.inc")).read()
    body = text.split("OXH_IQ3S_GRID[512] = {")[1].split("};")[0]
    grid = np.array([int(t, 16) for t in re.findall(r"0x([0-9a-f]+)u", body)], np.uint64)
    assert grid.size == 512
    for trial in range(4):
        blk = rng.integers(0, 256, 110).astype(np.uint8)
        blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
        for e in range(256):
            sb, i = e // 32, e % 32
            code = int(blk[2 + 8 * sb + i // 4]) | (((int(blk[66 + sb]) >> (i // 4)) & 1) << 8)
            mag = int((grid[code] >> np.uint64(8 * (i % 4))) & np.uint64(0xFF))
            neg = (int(blk[74 + 4 * sb + i // 8]) >> (i % 8)) & 1
            nib = (int(blk[106 + sb // 2]) >> (4 * (sb & 1))) & 15
            want = (-mag if neg else mag) * (2 * nib + 1)
            act = one_hot_act(e)
            lanes = np.zeros(8, np.int32)
            got = O.oxo_dot_iq3_s_q8_k(blk.ctypes.data, 1, act.ctypes.data, lanes.ctypes.data)
            assert got == float(want), (trial, e)
            expect = np.zeros(8, np.int32)
            expect[i // 4] = want
            assert np.array_equal(lanes, expect)


def test_iq1_xxxs_every_element_and_the_offset_term():
    """One activation value of 1 at position e: main = scale * codebook value, delta = +-scale (the
    group sum is 1), so the dot is scale * (value +- 0.125).  Values and signs read from the layout with
    numpy; the codebook must hold only -1, 0, +1."""
    rng = np.random.default_rng(6)
    import re
    text = open(os.path.join(oxlibs.ROOT, "oxidize_amd", "csrc", "iq_grids.inc")).read()
    body = text.split("OXH_IQ1XXXS_GRID[256] = {")[1].split("};")[0]
    grid = [int(t, 16) for t in re.findall(r"0x([0-9a-f]+)ull", body)]
    assert len(grid) == 256
    for trial in range(4):
        blk = rng.integers(0, 256, 38).astype(np.uint8)
        blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
        for e in range(256):
            g, i = e // 32, e % 32
            byte = (grid[int(blk[2 + 4 * g + i // 8])] >> (8 * (i % 8))) & 0xFF
            val = byte - 256 if byte >= 128 else byte
            assert val in (-1, 0, 1)
            nib = (int(blk[34 + g // 2]) >> (4 * (g & 1))) & 15
            scale = 2 * (nib & 7) + 1
            sgn = -1 if nib & 8 else 1
            act = one_hot_act(e)
            sums = np.zeros(2, np.int32)
            got = O.oxo_dot_iq1_xxxs_q8_k(blk.ctypes.data, 1, act.ctypes.data, sums.ctypes.data)
            assert (int(sums[0]), int(sums[1])) == (scale * val, scale * sgn)
            assert got == float(scale * val) + 0.125 * float(scale * sgn)


def test_live_against_the_compiled_reference_when_present():
    import ctypes
    ref = oxlibs.ref()
    if ref is None:
        pytest.skip("oracle/_ref/liboxref.so not built")
    ref.oc_parallel_set_threads(1)
    for qt in (25, 36):
        for seed, (rows, cols) in enumerate(((5, 256), (31, 2048), (3, 14336))):
            w = synth.weights(qt, rows, cols, seed=seed, stream=qt)
            x = synth.normal(cols, seed=seed, stream=3)
            rb = synth.row_bytes(qt, cols)
            out = np.zeros(rows, np.float32)
            want = np.zeros(rows, np.float32)
            t1, t2 = np.zeros(cols, np.float32), np.zeros(cols, np.float32)
            assert O.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, out.ctypes.data,
                                          t1.ctypes.data) == 0
            ref.oc_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, want.ctypes.data,
                                    t2.ctypes.data)
            assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
