"""CPU tests that pin the oracle (oracle/liboxoracle.so):

  * against the golden vectors taken from the compiled reference
    (tests/golden/*.npz, made by tests/golden/make_golden.py),
  * against the known-answer tests the reference's own suite holds
    (oxidize-c/tests/test_oxk.c, test_oxk_extended.c, test_quant.c),
  * against what the mathematics fixes: closed forms, a dequantised
    double-precision dot product, invariants of the activation format,
  * and, when oracle/_ref/liboxref.so is present, against the live reference.
"""
import ctypes
import os
import zlib

import numpy as np
import pytest

import oxlibs
from oxidize_amd import synth

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
Q80, Q4K, Q5K, Q6K = 7, 13, 15, 16
O = oxlibs.oracle()


def load(name):
    return np.load(os.path.join(GOLD, name))


def f32bits(x):
    return np.float32(x).view(np.uint32)


def f16_le(v):
    b = np.float16(v).view(np.uint16)
    return [int(b) & 255, int(b) >> 8]


# ─── scalar helpers ─────────────────────────────────────────────────────

def test_f16_to_f32_all_values_vs_reference_and_numpy():
    g = load("scalar_helpers.npz")
    mine = np.array([f32bits(O.oxo_f16_to_f32(i)) for i in range(65536)], dtype=np.uint32)
    assert np.array_equal(mine, g["f16_to_f32_bits"])
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    finite = np.isfinite(h)
    assert np.array_equal(mine[finite], h[finite].astype(np.float32).view(np.uint32))


@pytest.mark.parametrize("lo,hi,value", [(0, 0, 0.0), (0x00, 0x3C, 1.0), (0x00, 0xBC, -1.0),
                                         (0x00, 0x38, 0.5), (0x00, 0x40, 2.0), (0x00, 0x64, 1024.0)])
def test_f16_known_answers(lo, hi, value):
    # oxidize-c/tests/test_oxk.c:8-47
    assert O.oxo_f16_to_f32(lo | (hi << 8)) == value


def test_f32_to_f16_half_up_vs_reference():
    g = load("scalar_helpers.npz")
    mine = np.array([O.oxo_f32_to_f16_bits(float(v)) for v in g["f32_in"]], dtype=np.uint16)
    assert np.array_equal(mine, g["f32_to_f16_bits"])


def test_f32_to_f16_is_half_up_not_nearest_even():
    # 1 + 2^-11 is an exact tie between 0x3C00 and 0x3C01: RNE keeps the even
    # 0x3C00, the reference's rule goes up.
    tie = np.uint32(0x3F801000).view(np.float32)
    assert O.oxo_f32_to_f16_bits(float(tie)) == 0x3C01
    assert np.float32(tie).astype(np.float16).view(np.uint16) == 0x3C00
    assert O.oxo_f32_to_f16_bits(65520.0) == 0x7C00          # carries into inf
    assert O.oxo_f32_to_f16_bits(2.9802322e-8) == 0x0001     # half the smallest subnormal rounds up
    assert O.oxo_f32_to_f16_bits(2.9e-8) == 0x0000


def test_scale_min_k4_known_answers_and_golden():
    # oxidize-c/tests/test_oxk.c:72-103
    sc, mn = ctypes.c_uint8(), ctypes.c_uint8()
    s = (ctypes.c_uint8 * 12)()
    s[0], s[4] = 42, 17
    O.oxo_scale_min_k4(0, s, ctypes.byref(sc), ctypes.byref(mn))
    assert (sc.value, mn.value) == (42, 17)
    s = (ctypes.c_uint8 * 12)()
    s[0], s[4], s[8] = 0xC0, 0x80, 0x9A
    O.oxo_scale_min_k4(4, s, ctypes.byref(sc), ctypes.byref(mn))
    assert (sc.value, mn.value) == (0x0A | (3 << 4), 0x09 | (2 << 4))
    g = load("scalar_helpers.npz")
    for i in range(g["k4_scales"].shape[0]):
        row = np.ascontiguousarray(g["k4_scales"][i])
        for j in range(8):
            O.oxo_scale_min_k4(j, row.ctypes.data, ctypes.byref(sc), ctypes.byref(mn))
            assert (sc.value, mn.value) == tuple(g["k4_sc_min"][i, j])


# ─── activation quantisers ──────────────────────────────────────────────

def numpy_q8(x, group):
    """Independent numpy statement of d = amax/127, q = rint(x * (1/d))."""
    x = x.reshape(-1, group).astype(np.float32)
    amax = np.abs(x).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    q = np.clip(np.rint((x * inv[:, None]).astype(np.float32)), -128, 127).astype(np.int8)
    return d, q


def test_quantize_q8_k_against_numpy_and_invariants():
    cols = 4096
    x = synth.normal(cols, seed=0, stream=1000)
    x[256:512] = 0.0
    out = np.zeros(cols // 256 * 292, np.uint8)
    O.oxo_quantize_q8_k(x.ctypes.data, cols, out.ctypes.data)
    blk = out.reshape(-1, 292)
    d, q = numpy_q8(x, 256)
    assert np.array_equal(blk[:, :4].copy().view(np.float32).ravel(), d)
    assert np.array_equal(blk[:, 4:260].copy().view(np.int8), q)
    bs = blk[:, 260:].copy().view(np.int16)
    assert np.array_equal(bs, q.reshape(-1, 16, 16).sum(axis=2).astype(np.int16))
    assert np.all(blk[1] == 0)                       # all-zero block
    assert np.abs(q).max() == 127


def test_quantize_q8_0_against_numpy():
    cols = 896
    x = synth.normal(cols, seed=0, stream=1000)
    out = np.zeros(cols // 32 * 34, np.uint8)
    O.oxo_quantize_q8_0(x.ctypes.data, cols, out.ctypes.data)
    blk = out.reshape(-1, 34)
    d, q = numpy_q8(x, 32)
    assert np.array_equal(blk[:, 2:].copy().view(np.int8), q)
    want = np.array([O.oxo_f32_to_f16_bits(float(v)) for v in d], dtype=np.uint16)
    assert np.array_equal(blk[:, :2].copy().view(np.uint16).ravel(), want)


# ─── block dots ─────────────────────────────────────────────────────────

def dot(name, w, blocks, act, extra=None):
    w = np.ascontiguousarray(w)
    act = np.ascontiguousarray(act)
    if name == "q4_k":
        return O.oxo_dot_q4_k_q8_k(w.ctypes.data, blocks, act.ctypes.data, extra, None)
    if name == "q5_k":
        return O.oxo_dot_q5_k_q8_k(w.ctypes.data, blocks, act.ctypes.data, extra, None)
    if name == "q6_k":
        return O.oxo_dot_q6_k_q8_k(w.ctypes.data, blocks, act.ctypes.data, extra)
    return O.oxo_dot_q8_0_q8_0(w.ctypes.data, blocks, act.ctypes.data, extra)


@pytest.mark.parametrize("name", ["q4_k", "q6_k", "q8_0"])
def test_raw_block_dots_float_bits_vs_reference(name):
    g = load("raw_block_dots.npz")
    w, act = g[name + "_w"], g[name + "_act"]
    for t in range(w.shape[0]):
        for k, blocks in enumerate((1, w.shape[1])):
            got = f32bits(dot(name, w[t], blocks, act[t]))
            assert got == g[name + "_scalar_bits"][t, k]
            assert got == g[name + "_dispatched_bits"][t, k]


def test_known_answer_dots():
    # Q8_0 ones -> 32, twos*threes -> 192 (oxidize-c/tests/test_oxk.c:105-133)
    w = np.array([0x00, 0x3C] + [1] * 32, np.uint8)
    assert dot("q8_0", w, 1, w) == 32.0
    w2 = np.array([0x00, 0x3C] + [2] * 32, np.uint8)
    a3 = np.array([0x00, 0x3C] + [3] * 32, np.uint8)
    assert dot("q8_0", w2, 1, a3) == 192.0
    # all-zero K blocks -> 0 (oxidize-c/tests/test_oxk_extended.c:213-270)
    assert dot("q4_k", np.zeros(144, np.uint8), 1, np.zeros(292, np.uint8)) == 0.0
    assert dot("q6_k", np.zeros(210, np.uint8), 1, np.zeros(292, np.uint8)) == 0.0
    assert dot("q5_k", np.zeros(176, np.uint8), 1, np.zeros(292, np.uint8)) == 0.0


def q8k_block(d, q):
    blk = np.zeros(292, np.uint8)
    blk[:4] = np.array([d], np.float32).view(np.uint8)
    blk[4:260] = np.asarray(q, np.int8).view(np.uint8)
    blk[260:] = np.asarray(q, np.int8).reshape(16, 16).sum(axis=1).astype(np.int16).view(np.uint8)
    return blk


def q4k_block(d, dmin, sc, mn, nib):
    blk = np.zeros(144, np.uint8)
    blk[0:2], blk[2:4] = f16_le(d), f16_le(dmin)
    for j in range(4):
        blk[4 + j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        blk[8 + j] = mn[j] | ((mn[j + 4] >> 4) << 6)
        blk[12 + j] = (sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)
    nib = np.asarray(nib, np.uint8).reshape(4, 2, 32)      # [gp][low/high][l]
    blk[16:] = (nib[:, 0, :] | (nib[:, 1, :] << 4)).ravel()
    return blk


def test_q4_k_closed_form():
    # all nibbles n, all scales s, all mins m, all activations a:
    # dq*(d*256*s*n*a) - dq*(dmin*256*m*a), every factor exact in f32
    d, dmin, dq, s, m, n, a = 0.5, 0.25, 0.125, 3, 5, 7, 2
    w = q4k_block(d, dmin, [s] * 8, [m] * 8, [n] * 256)
    act = q8k_block(dq, [a] * 256)
    assert dot("q4_k", w, 1, act) == dq * d * 256 * s * n * a - dq * dmin * 256 * m * a


def test_q4_k_each_sub_block_uses_its_own_scale_and_nibble_half():
    # one-hot: only sub-block j has a non-zero scale -> result isolates S_j
    rng = np.random.default_rng(5)
    nib = rng.integers(0, 16, 256)
    q = rng.integers(-127, 128, 256)
    act = q8k_block(1.0, q)
    for j in range(8):
        sc = [0] * 8
        sc[j] = 1
        w = q4k_block(1.0, 0.0, sc, [0] * 8, nib)
        want = int(np.dot(nib[32 * j:32 * j + 32], q[32 * j:32 * j + 32]))
        sub = np.zeros(8, np.int32)
        got = dot("q4_k", w, 1, act, sub.ctypes.data)
        assert got == float(want)
        assert sub[j] == want
    # and the min term alone: scales 0, min j = 1 -> -dmin * sum(q over sub-block j)
    for j in range(8):
        mn = [0] * 8
        mn[j] = 1
        w = q4k_block(1.0, 1.0, [0] * 8, mn, nib)
        assert dot("q4_k", w, 1, act) == -float(q[32 * j:32 * j + 32].sum())


def q5k_block(d, dmin, sc, mn, codes):
    """Q5_K from 256 codes in [0,31]: the Q4_K header, then the fifth bits
    (bit j of byte l belongs to element 32j + l), then the nibbles."""
    codes = np.asarray(codes, np.uint8)
    q4 = q4k_block(d, dmin, sc, mn, codes & 15)
    hi = (codes >> 4).reshape(8, 32)
    plane = np.zeros(32, np.uint8)
    for j in range(8):
        plane |= (hi[j] << j).astype(np.uint8)
    return np.concatenate([q4[:16], plane, q4[16:]])


def test_q5_k_raw_block_dots_float_bits_vs_reference():
    g = load("q5_k.npz")
    w, act = g["raw_w"], g["raw_act"]
    for t in range(w.shape[0]):
        for k, blocks in enumerate((1, w.shape[1])):
            got = f32bits(dot("q5_k", w[t], blocks, act[t]))
            assert got == g["raw_scalar_bits"][t, k]
            assert got == g["raw_dispatched_bits"][t, k]


def test_q5_k_closed_form_and_fifth_bit_placement():
    d, dmin, dq, s, m, a = 0.5, 0.25, 0.125, 3, 5, 2
    for code in (7, 16, 23, 31):
        w = q5k_block(d, dmin, [s] * 8, [m] * 8, [code] * 256)
        act = q8k_block(dq, [a] * 256)
        assert dot("q5_k", w, 1, act) == dq * d * 256 * s * code * a - dq * dmin * 256 * m * a
    # one element with only its fifth bit set, one non-zero scale: the result is
    # 16 * that element's activation, for every element position
    rng = np.random.default_rng(11)
    q = rng.integers(-127, 128, 256)
    act = q8k_block(1.0, q)
    for e in list(range(0, 256, 37)) + [31, 32, 63, 64, 255]:
        codes = np.zeros(256, np.uint8)
        codes[e] = 16
        sc = [0] * 8
        sc[e // 32] = 1
        w = q5k_block(1.0, 0.0, sc, [0] * 8, codes)
        sub = np.zeros(8, np.int32)
        assert dot("q5_k", w, 1, act, sub.ctypes.data) == 16.0 * q[e]
        assert sub[e // 32] == 16 * q[e] and np.count_nonzero(sub) == (1 if q[e] else 0)
    # one-hot scales isolate each sub-block's integer sum
    codes = rng.integers(0, 32, 256)
    for j in range(8):
        sc = [0] * 8
        sc[j] = 1
        w = q5k_block(1.0, 0.0, sc, [0] * 8, codes)
        assert dot("q5_k", w, 1, act) == float(np.dot(codes[32 * j:32 * j + 32], q[32 * j:32 * j + 32]))


@pytest.mark.parametrize("qt", [15, 14])
def test_q5_k_matvec_and_batch_vs_reference_goldens(qt):
    g = load("q5_k.npz")
    key = "api%d_" % qt
    rows, cols, rb = (int(v) for v in g[key + "shape"])
    w, x = g[key + "w"], g[key + "x"]
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


@pytest.mark.parametrize("name,rows,cols", [("big_4096x4096", 4096, 4096), ("big_4096x14336", 4096, 14336)])
def test_q5_k_full_size_vs_reference_checksums(name, rows, cols):
    g = load("q5_k.npz")
    w = synth.weights(Q5K, rows, cols, seed=0, stream=0)
    x = synth.normal(cols, seed=0, stream=1000)
    assert zlib.crc32(w.tobytes()) == int(g[name + "_crc_w"][0])
    assert zlib.crc32(x.tobytes()) == int(g[name + "_crc_x"][0])
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert O.oxo_matvec_quantized(Q5K, w.ctypes.data, rows, cols, synth.row_bytes(Q5K, cols),
                                  x.ctypes.data, out.ctypes.data, temp.ctypes.data) == 0
    assert zlib.crc32(out.tobytes()) == int(g[name + "_crc_out"][0])
    assert np.array_equal(out, g[name + "_out"])


# ── Q2_K and Q3_K ────────────────────────────────────────────────────────

@pytest.mark.parametrize("name", ["q2_k", "q3_k"])
def test_q23_k_raw_block_dots_float_bits_vs_reference(name):
    g = load("q23_k.npz")
    fo = getattr(O, "oxo_dot_%s_q8_k" % name)
    w, act = g[name + "_raw_w"], g[name + "_raw_act"]
    for t in range(w.shape[0]):
        wt, at = np.ascontiguousarray(w[t]), np.ascontiguousarray(act[t])
        for k, blocks in enumerate((1, w.shape[1])):
            got = f32bits(fo(wt.ctypes.data, blocks, at.ctypes.data, None))
            assert got == g[name + "_raw_scalar_bits"][t, k]
            assert got == g[name + "_raw_dispatched_bits"][t, k]


def test_q3_k_rewritten_as_q6_k_is_the_same_dot_and_the_same_row():
    # the rewrite the batch path of the library uses for Q3_K weights: the Q6_K dot of the rewritten
    # blocks has the float bits of the Q3_K dot (which the reference vectors above pin), and the rows
    # dequantise to the same floats
    from q3k_rewrite import q3k_as_q6k
    g = load("q23_k.npz")
    w, act = g["q3_k_raw_w"], g["q3_k_raw_act"]
    for t in range(w.shape[0]):
        at = np.ascontiguousarray(act[t])
        w6 = q3k_as_q6k(w[t])
        for k, blocks in enumerate((1, w.shape[1])):
            got = f32bits(O.oxo_dot_q6_k_q8_k(w6.ctypes.data, blocks, at.ctypes.data, None))
            assert got == g["q3_k_raw_scalar_bits"][t, k]
    rows, cols = 9, 1024
    w3 = synth.weights(10, rows, cols, seed=77)
    w6 = q3k_as_q6k(w3)
    a = np.zeros((rows, cols), np.float32)
    b = np.zeros((rows, cols), np.float32)
    for r in range(rows):
        assert O.oxo_dequant_row(10, w3[r * (cols // 256) * 110:].ctypes.data, cols, a[r].ctypes.data) == 0
        assert O.oxo_dequant_row(16, w6[r * (cols // 256) * 210:].ctypes.data, cols, b[r].ctypes.data) == 0
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_q2_k_widened_blocks_give_the_reference_bits():
    # the widening the batch path of the library uses for Q2_K weights, and the arithmetic its tile
    # kernel runs on the result (one integer dot with scale * code, one with the group minima spread
    # over their elements, then dq * (d * pos - dmin * min)): float bits of the reference's Q2_K dot
    from q3k_rewrite import q2k_widen
    g = load("q23_k.npz")
    w, act = g["q2_k_raw_w"], g["q2_k_raw_act"]
    e = np.arange(256)
    n, k, l = e // 128, (e // 32) % 4, e % 32
    for t in range(w.shape[0]):
        wide = q2k_widen(w[t]).reshape(-1, 210).astype(np.int64)
        total = np.float32(0)
        for b in range(w.shape[1]):
            blk, a = wide[b], np.ascontiguousarray(act[t, b])
            dq = a[:4].view(np.float32)[0]
            q = a[4:260].view(np.int8).astype(np.int64)
            byte = blk[64 * n + 32 * (k & 1) + l]
            c6 = np.where(k >= 2, byte >> 4, byte & 15) | (((blk[128 + 32 * n + l] >> (2 * k)) & 3) << 4)
            mb = blk[192 + e // 32]
            m = np.where((e // 16) & 1, mb >> 4, mb & 15)
            d = blk[208:210].astype(np.uint8).view(np.float16)[0].astype(np.float32)
            dmin = blk[200:202].astype(np.uint8).view(np.float16)[0].astype(np.float32)
            pos, mn = np.float32(int((c6 * q).sum())), np.float32(int((m * q).sum()))
            with np.errstate(all="ignore"):
                total = np.float32(total + np.float32(dq * np.float32(np.float32(d * pos) - np.float32(dmin * mn))))
        assert f32bits(total) == g["q2_k_raw_scalar_bits"][t, 1]


@pytest.mark.parametrize("qt", [8, 9, 10, 11])
def test_q23_k_matvec_batch_and_dequant_vs_reference_goldens(qt):
    g = load("q23_k.npz")
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
    for r in range(2):
        deq = np.zeros(cols, np.float32)
        assert O.oxo_dequant_row(qt, w[r * rb:].ctypes.data, cols, deq.ctypes.data) == 0
        assert np.array_equal(deq.view(np.uint32), g[key + "dequant_bits"][r])


@pytest.mark.parametrize("qt,name", [(8, "big_q2_k_4096x4096"), (10, "big_q3_k_4096x4096")])
def test_q23_k_full_size_vs_reference_checksums(qt, name):
    g = load("q23_k.npz")
    w = synth.weights(qt, 4096, 4096, seed=0, stream=0)
    x = synth.normal(4096, seed=0, stream=1000)
    assert zlib.crc32(w.tobytes()) == int(g[name + "_crc_w"][0])
    out = np.zeros(4096, np.float32)
    temp = np.zeros(4096, np.float32)
    assert O.oxo_matvec_quantized(qt, w.ctypes.data, 4096, 4096, synth.row_bytes(qt, 4096),
                                  x.ctypes.data, out.ctypes.data, temp.ctypes.data) == 0
    assert zlib.crc32(out.tobytes()) == int(g[name + "_crc_out"][0])
    assert np.array_equal(out, g[name + "_out"])


def test_q2_k_closed_form_and_element_placement():
    """All codes c, scales s, mins m, activations a: dq*(d*256*s*c*a - dmin*256*m*a)
    (oxidize-c/src/compute/oxk.c:592-622); then one code at a time, which fixes
    element e = 128*outer + 32*inner + l <- bits 2*inner of qs[32*outer + l]
    and group e/16's scale."""
    d, dmin, dq, a = 0.5, 0.25, 0.125, 3
    for c, s_, m in ((1, 5, 2), (3, 15, 15), (2, 0, 7)):
        blk = np.zeros(84, np.uint8)
        blk[0:16] = s_ | (m << 4)
        blk[16:80] = c * 0x55
        blk[80:82], blk[82:84] = f16_le(d), f16_le(dmin)
        act = q8k_block(dq, np.full(256, a))
        assert O.oxo_dot_q2_k_q8_k(blk.ctypes.data, 1, act.ctypes.data, None) == \
            dq * (d * 256 * s_ * c * a - dmin * 256 * m * a)
    rng = np.random.default_rng(5)
    q = rng.integers(-127, 128, 256)
    act = q8k_block(1.0, q)
    scales = rng.integers(1, 16, 16)
    for e in range(256):
        blk = np.zeros(84, np.uint8)
        blk[0:16] = scales                                  # mins 0
        blk[80:82] = f16_le(1.0)
        outer, inner, l = e >> 7, (e >> 5) & 3, e & 31
        blk[16 + 32 * outer + l] = 3 << (2 * inner)
        grp = np.zeros(16, np.int32)
        got = O.oxo_dot_q2_k_q8_k(blk.ctypes.data, 1, act.ctypes.data, grp.ctypes.data)
        assert got == float(3 * int(scales[e >> 4]) * int(q[e])), "element %d" % e
        assert grp[e >> 4] == 3 * q[e] and np.count_nonzero(grp) == (1 if q[e] else 0)


def test_q3_k_closed_form_and_element_placement():
    """Codes 0..7 with a uniform offset of 4 and int8 scales sc - 32
    (oxidize-c/src/compute/oxk.c:624-652): all-equal blocks, then one 2-bit code
    and one third bit at a time (bit 4*outer + inner of hmask[l]), and each of
    the sixteen 6-bit scales in turn."""
    d, dq, a = 0.5, 0.25, 3

    def pack_scales(sc):                                    # sixteen values 0..63 into 12 bytes
        out = np.zeros(12, np.uint8)
        for j in range(16):
            lo, hi = sc[j] & 15, sc[j] >> 4
            out[j % 8] |= lo << (4 * (j // 8))
            out[8 + j % 4] |= hi << (2 * (j // 4))
        return out

    for code, raw_sc in ((7, 40), (0, 33), (5, 0), (4, 63)):
        blk = np.zeros(110, np.uint8)
        blk[0:32] = 0xFF if code & 4 else 0
        blk[32:96] = (code & 3) * 0x55
        blk[96:108] = pack_scales([raw_sc] * 16)
        blk[108:110] = f16_le(d)
        act = q8k_block(dq, np.full(256, a))
        assert O.oxo_dot_q3_k_q8_k(blk.ctypes.data, 1, act.ctypes.data, None) == \
            d * dq * 256 * (raw_sc - 32) * (code - 4) * a
    rng = np.random.default_rng(6)
    q = rng.integers(-127, 128, 256)
    act = q8k_block(1.0, q)
    raw = rng.integers(0, 64, 16)
    raw[raw == 32] = 33
    base_blk = np.zeros(110, np.uint8)
    base_blk[96:108] = pack_scales(list(raw))
    base_blk[108:110] = f16_le(1.0)
    base = O.oxo_dot_q3_k_q8_k(base_blk.ctypes.data, 1, act.ctypes.data, None)      # every code 0 -> weight -4*sc
    assert base == float(sum(-4 * (int(raw[g]) - 32) * int(q[16 * g:16 * g + 16].sum()) for g in range(16)))
    for e in range(256):
        outer, inner, l = e >> 7, (e >> 5) & 3, e & 31
        sc = int(raw[e >> 4]) - 32
        blk = base_blk.copy()
        blk[32 + 32 * outer + l] = 2 << (2 * inner)
        assert O.oxo_dot_q3_k_q8_k(blk.ctypes.data, 1, act.ctypes.data, None) == base + 2.0 * sc * q[e], e
        blk = base_blk.copy()
        blk[l] = 1 << (4 * outer + inner)
        assert O.oxo_dot_q3_k_q8_k(blk.ctypes.data, 1, act.ctypes.data, None) == base + 4.0 * sc * q[e], e


def test_q6_k_codes_zero_give_minus_32_times_scale_sum():
    # all codes 0 -> every weight is d*sc*(-32)  (oxidize-c/tests/test_quant.c:290-310)
    blk = np.zeros(210, np.uint8)
    blk[192:208] = np.arange(1, 17, dtype=np.int8).view(np.uint8)
    blk[208:210] = f16_le(1.0)
    q = np.arange(256) % 7 - 3
    act = q8k_block(1.0, q)
    want = sum(-32 * (g + 1) * int(q[16 * g:16 * g + 16].sum()) for g in range(16))
    assert dot("q6_k", blk, 1, act) == float(want)


@pytest.mark.parametrize("name,qt,group", [("q4_k", Q4K, 256), ("q5_k", Q5K, 256), ("q6_k", Q6K, 256),
                                           ("q8_0", Q80, 32)])
def test_dot_agrees_with_dequantised_double_precision(name, qt, group):
    """Kernel-vs-layout check of oxidize-c/tests/test_oxk_gguf_layout.c:104-141:
    dot the dequantised weights with the dequantised activation in double."""
    cols = 2048
    w = synth.weights(qt, 1, cols, seed=9, stream=qt)
    x = synth.normal(cols, seed=9)
    wf = np.zeros(cols, np.float32)
    assert O.oxo_dequant_row(qt, w.ctypes.data, cols, wf.ctypes.data) == 0
    if qt == Q80:
        act = np.zeros(cols // 32 * 34, np.uint8)
        O.oxo_quantize_q8_0(x.ctypes.data, cols, act.ctypes.data)
        b = act.reshape(-1, 34)
        dq = b[:, :2].copy().view(np.float16).astype(np.float64)
        xq = b[:, 2:].copy().view(np.int8).astype(np.float64) * dq
    else:
        act = np.zeros(cols // 256 * 292, np.uint8)
        O.oxo_quantize_q8_k(x.ctypes.data, cols, act.ctypes.data)
        b = act.reshape(-1, 292)
        dq = b[:, :4].copy().view(np.float32).astype(np.float64)
        xq = b[:, 4:260].copy().view(np.int8).astype(np.float64) * dq
    want = float(np.dot(wf.astype(np.float64), xq.ravel()))
    got = dot(name, w, cols // group, act)
    scale = float(np.abs(wf.astype(np.float64) * xq.ravel()).sum())
    assert abs(got - want) <= 1e-6 * scale


def test_every_weight_byte_influences_the_dot():
    # oxidize-c/tests/test_quant.c:569-583, applied to the dot kernels
    rng = np.random.default_rng(3)
    for name, qt, size in (("q4_k", Q4K, 144), ("q5_k", Q5K, 176), ("q6_k", Q6K, 210), ("q8_0", Q80, 34)):
        group = 32 if qt == Q80 else 256
        w = synth.weights(qt, 1, group, seed=13, stream=qt)
        if qt == Q80:
            act = np.concatenate([np.array(f16_le(0.5), np.uint8),
                                  rng.integers(1, 100, 32).astype(np.uint8)])
        else:
            act = q8k_block(0.5, rng.integers(1, 100, 256))
        base = f32bits(dot(name, w, 1, act))
        for i in range(size):
            w2 = w.copy()
            w2[i] ^= 0x15 if qt != Q80 or i >= 2 else 0x04
            assert f32bits(dot(name, w2, 1, act)) != base, "%s byte %d" % (name, i)


# ─── API level ──────────────────────────────────────────────────────────

@pytest.mark.parametrize("name,qt", [("q4_k", Q4K), ("q6_k", Q6K), ("q8_0", Q80)])
def test_matvec_and_batch_vs_reference_goldens(name, qt):
    g = load("matvec_api.npz")
    rows, cols, rb = (int(v) for v in g[name + "_shape"])
    w, x = g[name + "_w"], g[name + "_x"]
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert O.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data,
                                  out.ctypes.data, temp.ctypes.data) == 0
    act = g[name + "_act"]
    assert np.array_equal(temp.view(np.uint8)[:act.size], act)
    ref_out = g[name + "_out_bits"].view(np.float32)
    if qt == Q80:   # the reference's decode kernel reassociates the f32 sum
        assert np.all(np.abs(out - ref_out) <= 1e-4 + 1e-5 * np.abs(ref_out))
    else:
        assert np.array_equal(out.view(np.uint32), g[name + "_out_bits"])
    xs = g[name + "_batch_x"]
    n_vec, in_stride = xs.shape
    want = g[name + "_batch_out_bits"].view(np.float32)
    out_stride = want.shape[1]
    outs = np.full((n_vec, out_stride), -1.0, np.float32)
    scratch = np.zeros(O.oxo_matvec_batch_scratch_bytes(cols), np.uint8)
    assert O.oxo_matvec_quantized_batch(qt, w.ctypes.data, rows, cols, rb, xs.ctypes.data, in_stride,
                                        outs.ctypes.data, out_stride, n_vec, scratch.ctypes.data,
                                        scratch.nbytes) == 0
    if qt == Q80:
        assert np.all(np.abs(outs - want) <= 1e-4 + 1e-5 * np.abs(want))
    else:
        assert np.array_equal(outs.view(np.uint32), want.view(np.uint32))
    assert np.all(outs[:, rows:] == -1.0)


@pytest.mark.parametrize("name,qt,rows,cols", [("cfg0_q4k_4096x4096", Q4K, 4096, 4096),
                                               ("down_q6k_4096x14336", Q6K, 4096, 14336),
                                               ("ffn_q80_4864x896", Q80, 4864, 896)])
def test_full_size_configs_vs_reference_checksums(name, qt, rows, cols):
    g = load("full_size.npz")
    w = synth.weights(qt, rows, cols, seed=0, stream=0)
    x = synth.normal(cols, seed=0, stream=1000)
    assert zlib.crc32(w.tobytes()) == int(g[name + "_crc_w"][0])      # generator is stable
    assert zlib.crc32(x.tobytes()) == int(g[name + "_crc_x"][0])
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert O.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, synth.row_bytes(qt, cols),
                                  x.ctypes.data, out.ctypes.data, temp.ctypes.data) == 0
    nact = cols // synth.BLOCK_ELEMS[qt] * (34 if qt == Q80 else 292)
    assert zlib.crc32(temp.view(np.uint8)[:nact].tobytes()) == int(g[name + "_crc_act"][0])
    if qt == Q80:
        assert np.all(np.abs(out - g[name + "_out"]) <= 1e-4 + 1e-5 * np.abs(g[name + "_out"]))
    else:
        assert zlib.crc32(out.tobytes()) == int(g[name + "_crc_out"][0])


# ─── float steps in front of the quantiser ──────────────────────────────

FLOAT_RTOL = 4e-6      # scalar, SIMD-lane and tree summation orders differ by rounding only


def test_rms_norm_vs_reference_goldens_and_double_precision():
    g = load("float_steps.npz")
    for n in (256, 896, 4096):
        x, w = g["rms_%d_x" % n], g["rms_%d_w" % n]
        for eps in (1e-5, 1e-6):
            out = np.zeros(n, np.float32)
            O.oxo_rms_norm_f32(x.ctypes.data, w.ctypes.data, out.ctypes.data, n, eps)
            want = g["rms_%d_%g_out" % (n, eps)]
            assert np.all(np.abs(out - want) <= FLOAT_RTOL * np.abs(want))
            xd = x.astype(np.float64)
            exact = xd / np.sqrt((xd * xd).mean() + eps) * w
            assert np.all(np.abs(out - exact) <= FLOAT_RTOL * np.abs(exact))
    # closed form: a constant vector c with unit weights normalises to c/sqrt(c^2 + eps)
    x = np.full(512, 3.0, np.float32)
    out = np.zeros(512, np.float32)
    ones = np.ones(512, np.float32)
    O.oxo_rms_norm_f32(x.ctypes.data, ones.ctypes.data, out.ctypes.data, 512, 0.0)
    assert np.all(out == 1.0)
    # the weight multiplies element-wise and the sign of x survives
    w = np.arange(512, dtype=np.float32)
    x[::2] = -3.0
    O.oxo_rms_norm_f32(x.ctypes.data, w.ctypes.data, out.ctypes.data, 512, 0.0)
    assert np.array_equal(out, np.where(np.arange(512) % 2 == 0, -w, w))


def test_swiglu_vs_reference_goldens_and_double_precision():
    g = load("float_steps.npz")
    gate, up, want = g["swiglu_gate"], g["swiglu_up"], g["swiglu_out"]
    out = np.zeros(gate.size, np.float32)
    O.oxo_swiglu_f32(gate.ctypes.data, up.ctypes.data, out.ctypes.data, gate.size)
    # the reference's x86 exp clamps its argument at +-88: beyond that silu(g) is
    # 0 or g to more digits than f32 holds, but a denormal-range product may differ
    assert np.all(np.abs(out - want) <= FLOAT_RTOL * np.abs(want) + 1e-30)
    gd = gate.astype(np.float64)
    with np.errstate(over="ignore"):
        exact = gd / (1.0 + np.exp(-gd)) * up
    assert np.all(np.abs(out - exact) <= FLOAT_RTOL * np.abs(exact) + 1e-30)
    z, ones = np.zeros(4, np.float32), np.ones(4, np.float32)
    O.oxo_swiglu_f32(z.ctypes.data, ones.ctypes.data, out.ctypes.data, 4)
    assert np.all(out[:4] == 0.0)
    big, two = np.array([50.0, -50.0], np.float32), np.array([2.0, 2.0], np.float32)
    O.oxo_swiglu_f32(big.ctypes.data, two.ctypes.data, out.ctypes.data, 2)
    assert out[0] == 100.0 and abs(out[1]) < 1e-18


@pytest.mark.parametrize("name,qt", [("q4_k", Q4K), ("q5_k", Q5K), ("q6_k", Q6K), ("q8_0", Q80), ("q4_0", 3),
                                     ("q4_1", 4), ("q5_0", 5), ("q5_1", 6)])
def test_dequant_row_bits_vs_reference(name, qt):
    """oxo_dequant_row is the checker of the embedding lookup: bit-identical to
    the compiled reference's oc_quant_dequant_row on the committed vectors, and
    live when the compiled reference is present."""
    g = load("dequant_rows.npz")
    rows, cols, rb = (int(v) for v in g[name + "_shape"])
    w = g[name + "_w"]
    for r in range(rows):
        out = np.zeros(cols, np.float32)
        assert O.oxo_dequant_row(qt, w[r * rb:].ctypes.data, cols, out.ctypes.data) == 0
        assert np.array_equal(out.view(np.uint32), g[name + "_bits"][r])
    ref = oxlibs.ref()
    if ref is not None:
        cols = 2048 if qt in (Q4K, Q5K, Q6K) else 896
        rb = synth.row_bytes(qt, cols)
        w = synth.weights(qt, 5, cols, seed=19, stream=qt)
        for r in range(5):
            a, b = np.zeros(cols, np.float32), np.zeros(cols, np.float32)
            assert O.oxo_dequant_row(qt, w[r * rb:].ctypes.data, cols, a.ctypes.data) == 0
            assert ref.oc_quant_dequant_row(qt, w[r * rb:].ctypes.data, rb, b.ctypes.data, cols) == 0
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


LEGACY = (("q4_0", 3, 18), ("q4_1", 4, 20), ("q5_0", 5, 22), ("q5_1", 6, 24))
LEGACY_ALL = LEGACY + (("al5_xs", 18, 14),)


@pytest.mark.parametrize("name,qt,bsize", LEGACY_ALL)
def test_legacy_formats_vs_reference_goldens(name, qt, bsize):
    g = load("legacy_formats.npz")
    fo = getattr(O, "oxo_dot_%s_q8_0" % name)
    w, act = g[name + "_w"], g[name + "_act"]
    for t in range(w.shape[0]):
        wt, at = np.ascontiguousarray(w[t]), np.ascontiguousarray(act[t])
        for k, blocks in enumerate((1, w.shape[1])):
            got = f32bits(fo(wt.ctypes.data, blocks, at.ctypes.data, None))
            assert got == g[name + "_scalar_bits"][t, k]
            assert got == g[name + "_dispatched_bits"][t, k]
    rows, cols, rb = (int(v) for v in g[name + "_api_shape"])
    wm, x = g[name + "_api_w"], g[name + "_api_x"]
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert O.oxo_matvec_quantized(qt, wm.ctypes.data, rows, cols, rb, x.ctypes.data, out.ctypes.data,
                                  temp.ctypes.data) == 0
    a = g[name + "_api_act"]
    assert np.array_equal(temp.view(np.uint8)[:a.size], a)
    want = g[name + "_api_out"]
    assert np.all(np.abs(out - want) <= 1e-4 + 1e-5 * np.abs(want))


def test_al5_xs_closed_form_placement_and_dequant():
    """Thirty-two 3-bit codes, least significant bit first, offset 4
    (oxidize-c/src/compute/oxk.c:195-222): all-equal blocks, one code at a time,
    and the dequantised rows of the compiled reference."""
    d, dq, a = 0.5, 0.25, 3
    act = np.concatenate([np.array(f16_le(dq), np.uint8), np.full(32, a, np.int8).view(np.uint8)])
    for code in range(8):
        bits_ = "".join(format(code, "03b")[::-1] for _ in range(32))
        packed = np.array([int(bits_[8 * i:8 * i + 8][::-1], 2) for i in range(12)], np.uint8)
        blk = np.concatenate([np.array(f16_le(d), np.uint8), packed])
        assert O.oxo_dot_al5_xs_q8_0(blk.ctypes.data, 1, act.ctypes.data, None) == d * dq * 32 * (code - 4) * a
    rng = np.random.default_rng(9)
    q = rng.integers(-127, 128, 32).astype(np.int8)
    act = np.concatenate([np.array(f16_le(1.0), np.uint8), q.view(np.uint8)])
    base_blk = np.zeros(14, np.uint8)
    base_blk[0:2] = f16_le(1.0)
    base = O.oxo_dot_al5_xs_q8_0(base_blk.ctypes.data, 1, act.ctypes.data, None)
    assert base == float(-4 * int(q.sum()))
    for e in range(32):
        for bit in range(3):
            blk = base_blk.copy()
            pos = 3 * e + bit
            blk[2 + pos // 8] = 1 << (pos % 8)
            isum = np.zeros(1, np.int32)
            got = O.oxo_dot_al5_xs_q8_0(blk.ctypes.data, 1, act.ctypes.data, isum.ctypes.data)
            assert got == base + float((1 << bit) * int(q[e])), (e, bit)
    g = load("legacy_formats.npz")
    rows, cols, rb = (int(v) for v in g["al5_xs_api_shape"])
    wm = g["al5_xs_api_w"]
    for r in range(2):
        deq = np.zeros(cols, np.float32)
        assert O.oxo_dequant_row(18, wm[r * rb:].ctypes.data, cols, deq.ctypes.data) == 0
        assert np.array_equal(deq.view(np.uint32), g["al5_xs_dequant_bits"][r])


@pytest.mark.parametrize("name,qt,base", [("al5", 17, 3), ("al6", 19, 5), ("al8", 20, 7)])
def test_alias_types_vs_reference_goldens(name, qt, base):
    """AL5 / AL6 / AL8 are the Q4_0 / Q5_0 / Q8_0 layouts under other ids
    (oxidize-c/src/compute/quantization.c:207-214, matvec.c:323-329): the
    compiled reference's outputs for the alias id, and the oracle's for the
    alias and the base id, which must not differ by a bit."""
    g = load("legacy_formats.npz")
    rows, cols, rb = (int(v) for v in g[name + "_api_shape"])
    wm, x = g[name + "_api_w"], g[name + "_api_x"]
    outs = []
    for t in (qt, base):
        out, temp = np.zeros(rows, np.float32), np.zeros(cols, np.float32)
        assert O.oxo_act_kind(t, cols) == 1 and O.oxo_stride_ok(t, cols, rb) == 1
        assert O.oxo_matvec_quantized(t, wm.ctypes.data, rows, cols, rb, x.ctypes.data, out.ctypes.data,
                                      temp.ctypes.data) == 0
        a = g[name + "_api_act"]
        assert np.array_equal(temp.view(np.uint8)[:a.size], a)
        outs.append(out)
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    want = g[name + "_api_out"]
    assert np.all(np.abs(outs[0] - want) <= 1e-4 + 1e-5 * np.abs(want))
    for r in range(2):
        deq = np.zeros(cols, np.float32)
        assert O.oxo_dequant_row(qt, wm[r * rb:].ctypes.data, cols, deq.ctypes.data) == 0
        assert np.array_equal(deq.view(np.uint32), g[name + "_dequant_bits"][r])


@pytest.mark.parametrize("name,qt,bsize", LEGACY)
def test_legacy_formats_closed_forms_and_layout(name, qt, bsize):
    """Codes c everywhere, activations a everywhere: 32*(c - offset)*a*d*dq, plus
    32*a*m*dq for the _1 formats; and one element at a time, which fixes the
    nibble halves (byte i: low nibble = element i, high = element i + 16) and
    the fifth-bit order."""
    fo = getattr(O, "oxo_dot_%s_q8_0" % name)
    has_m, five = name.endswith("_1"), name.startswith("q5")
    qs_at = bsize - 16
    d, m, dq, a = 0.5, 0.25, 0.125, 3
    act = np.concatenate([np.array(f16_le(dq), np.uint8), np.full(32, a, np.int8).view(np.uint8)])
    for code in ((5, 12) if not five else (5, 21, 31)):
        blk = np.zeros(bsize, np.uint8)
        blk[0:2] = f16_le(d)
        if has_m:
            blk[2:4] = f16_le(m)
        blk[qs_at:] = (code & 15) | ((code & 15) << 4)
        if five and code & 16:
            blk[qs_at - 4:qs_at] = 0xFF
        off = 0 if has_m else (16 if five else 8)
        want = dq * d * 32 * (code - off) * a + (dq * m * 32 * a if has_m else 0.0)
        assert fo(blk.ctypes.data, 1, act.ctypes.data, None) == want
    rng = np.random.default_rng(9)
    q = rng.integers(-127, 128, 32).astype(np.int8)
    act = np.concatenate([np.array(f16_le(1.0), np.uint8), q.view(np.uint8)])
    off = 0 if has_m else (16 if five else 8)
    base_blk = np.zeros(bsize, np.uint8)
    base_blk[0:2] = f16_le(1.0)
    base = fo(base_blk.ctypes.data, 1, act.ctypes.data, None)          # all codes 0
    assert base == float(-off * int(q.sum()))
    for e in range(32):
        blk = base_blk.copy()
        blk[qs_at + (e & 15)] = 7 << (4 * (e >> 4))
        isum = np.zeros(1, np.int32)
        got = fo(blk.ctypes.data, 1, act.ctypes.data, isum.ctypes.data)
        assert got == base + 7.0 * q[e], "element %d" % e
        if five:
            blk = base_blk.copy()
            blk[qs_at - 4 + (e >> 3)] = 1 << (e & 7)
            assert fo(blk.ctypes.data, 1, act.ctypes.data, None) == base + 16.0 * q[e], "fifth bit %d" % e


def test_eligibility_rules():
    # oxidize-c/src/compute/matvec.c:99-127, :961-985
    assert O.oxo_act_kind(Q4K, 4096) == 2 and O.oxo_act_kind(Q4K, 896) == 0
    assert O.oxo_act_kind(Q6K, 256) == 2 and O.oxo_act_kind(12, 512) == 2
    assert O.oxo_act_kind(Q80, 896) == 1 and O.oxo_act_kind(Q80, 900) == 0
    assert O.oxo_act_kind(0, 4096) == 0 and O.oxo_act_kind(1, 4096) == 0
    for qt, rb in ((3, 18), (4, 20), (5, 22), (6, 24)):
        assert O.oxo_act_kind(qt, 896) == 1 and O.oxo_act_kind(qt, 900) == 0
        assert O.oxo_stride_ok(qt, 896, 28 * rb) == 1 and O.oxo_stride_ok(qt, 896, 28 * rb + 2) == 0
    assert O.oxo_act_kind(14, 512) == 2 and O.oxo_act_kind(Q5K, 4096) == 2 and O.oxo_act_kind(Q5K, 4000) == 0
    assert O.oxo_stride_ok(Q5K, 4096, 2816) == 1 and O.oxo_stride_ok(Q5K, 4096, 2304) == 0
    assert O.oxo_stride_ok(Q4K, 4096, 2304) == 1 and O.oxo_stride_ok(Q4K, 4096, 2320) == 0
    assert O.oxo_stride_ok(Q6K, 14336, 11760) == 1 and O.oxo_stride_ok(Q80, 896, 952) == 1
    assert O.oxo_matvec_batch_scratch_bytes(4096) == 4 << 20


def test_moe_route_brute_force():
    """Top-2 of 8 by softmax probability (oxidize-c/src/model/llama.c:5965-6031):
    selection is order-only, so it must equal a stable descending sort."""
    logits = synth.normal(16 * 8, seed=0, stream=4242).reshape(16, 8)
    ids = np.zeros((16, 2), np.int32)
    wts = np.zeros((16, 2), np.float32)
    O.oxo_moe_route(logits.ctypes.data, 16, 8, 2, 1, ids.ctypes.data, wts.ctypes.data)
    for t in range(16):
        order = np.argsort(-logits[t], kind="stable")[:2]
        assert list(ids[t]) == list(order)
        p = np.exp(logits[t].astype(np.float64) - logits[t].max())
        p /= p.sum()
        assert np.allclose(wts[t], p[order] / p[order].sum(), rtol=1e-5)
        assert abs(wts[t].sum() - 1.0) < 1e-6


def test_moe_route_ties_known_answers():
    """Worked by hand from the swapping selection of llama.c:5998-6012: after
    expert 3 wins the first round of [0, 0, 0, 5], the index list reads
    [3, 1, 2, 0], so the equal rest is taken as 1, 2 (not 0, 1)."""
    rows = np.array([[0, 0, 0, 5], [5, 0, 0, 0], [0, 5, 0, 0], [1, 1, 1, 1], [0, 2, 2, 0], [3, 0, 3, 0]], np.float32)
    ids = np.zeros((6, 3), np.int32)
    wts = np.zeros((6, 3), np.float32)
    O.oxo_moe_route(rows.ctypes.data, 6, 4, 3, 0, ids.ctypes.data, wts.ctypes.data)
    assert ids.tolist() == [[3, 1, 2], [0, 1, 2], [1, 0, 2], [0, 1, 2], [1, 2, 0], [0, 2, 1]]
    assert np.allclose(wts[3], 0.25) and np.allclose(wts[0, 0], np.exp(5) / (np.exp(5) + 3), rtol=1e-6)


def dequant_matrix(qt, w, rows, cols):
    rb = synth.row_bytes(qt, cols)
    out = np.zeros((rows, cols), np.float32)
    for r in range(rows):
        assert O.oxo_dequant_row(qt, w[r * rb:].ctypes.data, cols, out[r].ctypes.data) == 0
    return out.astype(np.float64)


@pytest.mark.parametrize("qt_gu,qt_dn,renorm", [(Q4K, Q6K, 1), (Q5K, Q4K, 0)])
def test_moe_ffn_against_dense_restatement(qt_gu, qt_dn, renorm):
    """The layer of oxidize-c/src/model/llama.c:5965-6160 written a second way:
    double-precision dense products of the dequantised expert matrices, experts
    picked by a stable sort.  Agreement is to the activation quantisation
    (about 1 %), which is what a wrong expert index, a swapped gate/up, a
    missing gate weight or a token gathered from the wrong row would exceed by
    orders of magnitude."""
    n_exp, k, hidden, ffn, n_tok = 4, 2, 256, 512, 7
    rb_gu, rb_dn = synth.row_bytes(qt_gu, hidden), synth.row_bytes(qt_dn, ffn)
    wg = synth.weights(qt_gu, n_exp * ffn, hidden, seed=5, stream=1)
    wu = synth.weights(qt_gu, n_exp * ffn, hidden, seed=5, stream=2)
    wd = synth.weights(qt_dn, n_exp * hidden, ffn, seed=5, stream=3)
    logits = synth.normal(n_tok * n_exp, seed=5, stream=4).reshape(n_tok, n_exp)
    logits[:, 3] = -30.0                                   # an expert nobody selects
    x = synth.normal(n_tok * hidden, seed=5, stream=5).reshape(n_tok, hidden)
    out = np.full((n_tok, hidden), np.nan, np.float32)
    assert O.oxo_moe_ffn(qt_gu, qt_dn, wg.ctypes.data, wu.ctypes.data, wd.ctypes.data, n_exp, k, hidden, ffn,
                         renorm, logits.ctypes.data, x.ctypes.data, n_tok, out.ctypes.data) == 0
    G, U, D = (dequant_matrix(qt_gu, wg, n_exp * ffn, hidden), dequant_matrix(qt_gu, wu, n_exp * ffn, hidden),
               dequant_matrix(qt_dn, wd, n_exp * hidden, ffn))
    want = np.zeros((n_tok, hidden))
    for t in range(n_tok):
        p = np.exp(logits[t].astype(np.float64) - logits[t].max())
        p /= p.sum()
        sel = np.argsort(-logits[t], kind="stable")[:k]
        assert 3 not in sel
        gw = p[sel] / p[sel].sum() if renorm else p[sel]
        for e, w in zip(sel, gw):
            g = G[e * ffn:(e + 1) * ffn] @ x[t]
            u = U[e * ffn:(e + 1) * ffn] @ x[t]
            with np.errstate(over="ignore"):
                h = g / (1.0 + np.exp(-g)) * u
            want[t] += w * (D[e * hidden:(e + 1) * hidden] @ h)
    scale = np.abs(want).max()
    assert np.abs(out - want).max() < 0.03 * scale


@pytest.mark.skipif(oxlibs.ref() is None, reason="compiled reference not present")
def test_oracle_vs_live_reference_many_rows():
    ref = oxlibs.ref()
    ref.oc_parallel_set_threads(2)
    for qt, rows, cols in ((Q4K, 700, 4096), (Q6K, 300, 14336), (Q4K, 513, 2816), (Q6K, 64, 256),
                           (Q5K, 300, 4096), (14, 65, 768)):
        rb = synth.row_bytes(qt, cols)
        w = synth.weights(qt, rows, cols, seed=77, stream=rows)
        x = synth.normal(cols, seed=77)
        a, b = np.zeros(rows, np.float32), np.zeros(rows, np.float32)
        ta, tb = np.zeros(cols, np.float32), np.zeros(cols, np.float32)
        O.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, a.ctypes.data, ta.ctypes.data)
        ref.oc_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, b.ctypes.data, tb.ctypes.data)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert np.array_equal(ta.view(np.uint8), tb.view(np.uint8))


@pytest.mark.parametrize("qt", [3, 4, 5, 6, 7, 8, 10, 13, 15, 16, 18])
def test_extreme_integers_oracle_vs_compiled_reference(qt):
    # every code, scale and minimum at its bound, activations at +-127: the restatement must keep the
    # reference's bits there too (the GPU test on the same inputs checks the kernels against it)
    from extremes import TYPES, extreme_inputs, extreme_weights
    ref = oxlibs.ref()
    if ref is None:
        pytest.skip("oracle/_ref was not built")
    layout, fields = TYPES[qt]
    rows, cols, n_vec = 130, (1024 if synth.BLOCK_ELEMS[layout] == 256 else 512), 6
    rb = synth.row_bytes(layout, cols)
    w = extreme_weights(layout, fields, rows, cols)
    xs = extreme_inputs(n_vec, cols)
    for v in range(n_vec):
        x = np.ascontiguousarray(xs[v])
        mine, theirs = np.zeros(rows, np.float32), np.zeros(rows, np.float32)
        t1, t2 = np.zeros(cols, np.float32), np.zeros(cols, np.float32)
        assert O.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, mine.ctypes.data,
                                      t1.ctypes.data) == 0
        ref.oc_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, theirs.ctypes.data,
                                t2.ctypes.data)
        nact = cols // 256 * 292 if synth.BLOCK_ELEMS[layout] == 256 else cols // 32 * 34
        assert np.array_equal(t1.view(np.uint8)[:nact], t2.view(np.uint8)[:nact])
        if synth.BLOCK_ELEMS[layout] == 256:
            assert np.array_equal(mine.view(np.uint32), theirs.view(np.uint32)), (qt, v)
        else:       # the x86 kernels of the 32-value formats sum in another order
            assert np.allclose(mine, theirs, rtol=1e-5, atol=1e-4 * float(np.abs(theirs).max()))


@pytest.mark.parametrize("qt", [13, 7])
def test_quantiser_edge_inputs_oracle_vs_compiled_reference(qt):
    # rounding ties, the largest floats, subnormal block scales (not: blocks whose 1/d overflows and
    # non-finite inputs, where the reference's scalar and AVX-512 quantisers disagree with each other)
    from extremes import quantiser_edge_inputs
    ref = oxlibs.ref()
    if ref is None:
        pytest.skip("oracle/_ref was not built")
    n = 512
    fn = O.oxo_quantize_q8_k if qt == 13 else O.oxo_quantize_q8_0
    nb = n // 256 * 292 if qt == 13 else n // 32 * 34
    w = synth.weights(qt, 4, n, seed=2)
    for name, x in quantiser_edge_inputs(n).items():
        want = np.zeros(nb, np.uint8)
        fn(x.ctypes.data, n, want.ctypes.data)
        out, temp = np.zeros(4, np.float32), np.zeros(n, np.float32)
        ref.oc_matvec_quantized(qt, w.ctypes.data, 4, n, synth.row_bytes(qt, n), x.ctypes.data, out.ctypes.data,
                                temp.ctypes.data)
        assert np.array_equal(temp.view(np.uint8)[:nb], want), name

