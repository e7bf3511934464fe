"""GPU parity for Q5_K weights (type ids 14 and 15) through the C ABI, against
the CPU oracle, the committed vectors of the compiled reference
(tests/golden/q5_k.npz) and, when present, the live compiled reference.

Bars: Q8_K activation bytes, the eight integer sub-block sums per super-block
and the f32 outputs are all bit-exact (the reference's Q5_K kernels agree with
one another to the bit, oxidize-c/tests/test_oxk_avx2_parity.c:361-383).
"""
import os
import zlib

import numpy as np
import pytest

import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "q5_k.npz")
Q4K, Q5KS, Q5K = 13, 14, 15


def oracle_matvec(qtype, w, rows, cols, x):
    o = oxlibs.oracle()
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    rc = o.oxo_matvec_quantized(qtype, w.ctypes.data, rows, cols, synth.row_bytes(qtype, cols),
                                x.ctypes.data, out.ctypes.data, temp.ctypes.data)
    assert rc == 0
    return out, temp


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


@pytest.mark.parametrize("qtype,rows,cols", [
    (Q5K, 1, 256), (Q5K, 7, 256), (Q5KS, 64, 512), (Q5K, 333, 4096), (Q5K, 4096, 4096),
    (Q5K, 100, 14336), (Q5KS, 33, 2816), (Q5K, 4100, 1024),
])
def test_matvec_quantized_q5k_bits(oxh, qtype, rows, cols):
    w = synth.weights(qtype, rows, cols, seed=25, stream=rows)
    x = synth.normal(cols, seed=25, stream=9)
    out = np.full(rows, np.nan, np.float32)
    temp = np.zeros(cols, np.float32)
    rb = synth.row_bytes(qtype, cols)
    assert mv.matvec_quantized(qtype, w, rows, cols, rb, x, out, temp) == 0
    want, want_temp = oracle_matvec(qtype, w, rows, cols, x)
    nact = mv.act_bytes(qtype, cols)
    assert np.array_equal(temp.view(np.uint8)[:nact], want_temp.view(np.uint8)[:nact])
    assert np.array_equal(bits(out), bits(want))
    ref = oxlibs.ref()
    if ref is not None:
        r_out = np.zeros(rows, np.float32)
        r_tmp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qtype, w.ctypes.data, rows, cols, rb, x.ctypes.data,
                                r_out.ctypes.data, r_tmp.ctypes.data)
        assert np.array_equal(bits(out), bits(r_out))


def test_q5k_subblock_sums_bit_exact(oxh):
    rows, cols = 37, 4096
    w = synth.weights(Q5K, rows, cols, seed=6)
    x = synth.normal(cols, seed=6)
    o = oxlibs.oracle()
    act = np.zeros(mv.act_bytes(Q5K, cols), np.uint8)
    o.oxo_quantize_q8_k(x.ctypes.data, cols, act.ctypes.data)
    blocks, rb = cols // 256, synth.row_bytes(Q5K, cols)
    want = np.zeros((rows, blocks, 8), np.int32)
    for r in range(rows):
        o.oxo_dot_q5_k_q8_k(w[r * rb:].ctypes.data, blocks, act.ctypes.data, want[r].ctypes.data, None)
    d_w = mv.DeviceBuffer.from_host(w)
    d_a = mv.DeviceBuffer.from_host(act)
    d_s = mv.DeviceBuffer(want.nbytes)
    mv.debug_subblock_sums(Q5K, d_w.ptr, rows, cols, d_a.ptr, d_s.ptr)
    got = d_s.download(np.int32, want.size).reshape(want.shape)
    assert np.array_equal(got, want)


def test_q5k_fifth_bit_of_every_element_position(oxh):
    """One row per element position: only that element's fifth bit is set and
    only its sub-block's scale is 1, so the output is 16 x that element's
    quantised activation x d (a wrong bit-to-element map shows as a wrong row)."""
    cols = 256
    w = np.zeros((256, 176), np.uint8)
    w[:, 0:2] = np.array([0x00, 0x3C], np.uint8)          # d = 1.0, dmin = 0
    for e in range(256):
        j, l = e // 32, e % 32
        if j < 4:
            w[e, 4 + j] = 1
        else:
            w[e, 12 + (j - 4)] = 1
        w[e, 16 + l] = 1 << j
    w = np.ascontiguousarray(w.ravel())
    x = synth.normal(cols, seed=3)
    out = np.zeros(256, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(Q5K, w, 256, cols, 176, x, out, temp) == 0
    d = temp.view(np.float32)[0]
    q = temp.view(np.int8)[4:260].astype(np.float32)
    assert np.array_equal(out, (np.float32(1.0) * d) * (16.0 * q))
    want, _ = oracle_matvec(Q5K, w, 256, cols, x)
    assert np.array_equal(bits(out), bits(want))


@pytest.mark.parametrize("qt", [15, 14])
def test_q5k_api_goldens_from_the_compiled_reference(oxh, qt):
    g = np.load(GOLD)
    key = "api%d_" % qt
    rows, cols, rb = (int(v) for v in g[key + "shape"])
    w, x = g[key + "w"], g[key + "x"]
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(qt, w, rows, cols, rb, x, out, temp) == 0
    act = g[key + "act"]
    assert np.array_equal(temp.view(np.uint8)[:act.size], act)
    assert np.array_equal(bits(out), g[key + "out_bits"])
    xs = np.ascontiguousarray(g[key + "batch_x"])
    n_vec, in_stride = xs.shape
    want = g[key + "batch_out_bits"]
    out_stride = want.shape[1]
    outs = np.full((n_vec, out_stride), -1.0, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    assert mv.matvec_quantized_batch(qt, w, rows, cols, rb, xs, in_stride, outs, out_stride, n_vec,
                                     temp, scratch) == 0
    assert np.array_equal(bits(outs), want)


@pytest.mark.parametrize("name,rows,cols", [("big_4096x4096", 4096, 4096), ("big_4096x14336", 4096, 14336)])
def test_q5k_full_size_against_reference_checksums(oxh, name, rows, cols):
    g = np.load(GOLD)
    w = synth.weights(Q5K, rows, cols, seed=0, stream=0)
    x = synth.normal(cols, seed=0, stream=1000)
    assert zlib.crc32(w.tobytes()) == int(g[name + "_crc_w"][0])
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(Q5K, w, rows, cols, synth.row_bytes(Q5K, cols), x, out, temp) == 0
    assert zlib.crc32(out.tobytes()) == int(g[name + "_crc_out"][0])
    assert np.array_equal(out, g[name + "_out"])


@pytest.mark.parametrize("cols,rows", [(4096, [4096, 1024, 1024]), (2048, [300, 0, 5])])
def test_q5k_fused_equals_separate(oxh, cols, rows):
    rb = synth.row_bytes(Q5K, cols)
    ws = [synth.weights(Q5K, r, cols, seed=31, stream=i) if r else np.zeros(1, np.uint8)
          for i, r in enumerate(rows)]
    x = synth.normal(cols, seed=31, stream=99)
    outs = [np.full(max(r, 1), np.nan, np.float32) for r in rows]
    temp = np.zeros(cols, np.float32)
    oxh.oc_matvec_fused_test_reset()
    assert mv.matvec_quantized_fused([Q5K] * len(rows), ws, rows, cols, [rb] * len(rows), x, outs, temp) == 0
    st = oxh.oc_matvec_fused_test_stats()
    assert (st.activation_quantizations, st.parallel_dispatches, st.fallback_calls) == (1, 1, 0)
    for w, r, out in zip(ws, rows, outs):
        if r:
            want, _ = oracle_matvec(Q5K, w, r, cols, x)
            assert np.array_equal(bits(out[:r]), bits(want))


def test_q5k_mixed_with_q4k_falls_back_per_matrix(oxh):
    # oxidize-c/tests/test_matvec_fused.c:119-136
    cols, rows, qts = 1024, [40, 24], [Q4K, Q5K]
    ws = [synth.weights(q, r, cols, seed=32, stream=i) for i, (q, r) in enumerate(zip(qts, rows))]
    x = synth.normal(cols, seed=32)
    outs = [np.zeros(r, np.float32) for r in rows]
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized_fused(qts, ws, rows, cols, [synth.row_bytes(q, cols) for q in qts],
                                     x, outs, temp) == 0
    for q, w, r, out in zip(qts, ws, rows, outs):
        want, _ = oracle_matvec(q, w, r, cols, x)
        assert np.array_equal(bits(out), bits(want))


def test_q5k_multi_input_equals_separate(oxh):
    cols, rows = 768, [3, 17, 1, 40]
    rb = synth.row_bytes(Q5K, cols)
    ws = [synth.weights(Q5K, r, cols, seed=41, stream=i) for i, r in enumerate(rows)]
    xs = [synth.normal(cols, seed=41, stream=200 + i) for i in range(len(rows))]
    outs = [np.full(r, np.nan, np.float32) for r in rows]
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized_multi_input([Q5K] * len(rows), ws, rows, cols, [rb] * len(rows),
                                           xs, outs, temp) == 0
    for w, r, x, out in zip(ws, rows, xs, outs):
        want, _ = oracle_matvec(Q5K, w, r, cols, x)
        assert np.array_equal(bits(out), bits(want))


@pytest.mark.parametrize("rows,cols,n_vec,in_pad,out_pad", [
    (96, 1024, 1, 0, 0), (96, 1024, 5, 3, 7), (64, 14336, 8, 0, 0), (40, 512, 13, 0, 3),
    (130, 1024, 9, 0, 0), (128, 4096, 64, 0, 0), (200, 2816, 100, 0, 5), (257, 512, 65, 0, 1),
    (32, 256, 32, 0, 0),
])
def test_q5k_batch_equals_single(oxh, rows, cols, n_vec, in_pad, out_pad):
    in_stride, out_stride = cols + in_pad, rows + out_pad
    w = synth.weights(Q5K, rows, cols, seed=51, stream=rows)
    xs = synth.normal(n_vec * in_stride, seed=51, stream=3).reshape(n_vec, in_stride)
    if n_vec > 3:
        xs[3, :256] = 0.0
    outs = np.full((n_vec, out_stride), -7.25, np.float32)
    temp = np.zeros(cols, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    assert mv.matvec_quantized_batch(Q5K, w, rows, cols, synth.row_bytes(Q5K, cols), xs, in_stride,
                                     outs, out_stride, n_vec, temp, scratch) == 0
    for v in range(n_vec):
        want, _ = oracle_matvec(Q5K, w, rows, cols, np.ascontiguousarray(xs[v, :cols]))
        assert np.array_equal(bits(outs[v, :rows]), bits(want)), "vector %d" % v
        assert np.all(outs[v, rows:] == -7.25)


def test_q5k_subnormal_and_extreme_f16_scales(oxh):
    rows, cols = 64, 1024
    w = synth.weights(Q5K, rows, cols, seed=81)
    blk = w.reshape(-1, 176)
    pats = np.array([0x0001, 0x0002, 0x03FF, 0x0400, 0x7BFF, 0x8001, 0x83FF, 0xBC00, 0x0000, 0x8000,
                     0x0155, 0x3555], np.uint16)
    sel = pats[np.arange(blk.shape[0]) % pats.size]
    sel2 = pats[(np.arange(blk.shape[0]) * 5 + 3) % pats.size]
    blk[:, 0], blk[:, 1] = sel & 0xFF, sel >> 8
    blk[:, 2], blk[:, 3] = sel2 & 0xFF, sel2 >> 8
    x = synth.normal(cols, seed=81)
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(Q5K, w, rows, cols, synth.row_bytes(Q5K, cols), x, out, temp) == 0
    want, _ = oracle_matvec(Q5K, w, rows, cols, x)
    assert np.array_equal(bits(out), bits(want))


@pytest.mark.parametrize("rows,cols,n_vec", [(100, 4096, 1), (60, 2048, 3), (90, 1024, 8)])
def test_q5k_prequantised_and_fused_paths_agree(oxh, rows, cols, n_vec):
    w = synth.weights(Q5K, rows, cols, seed=91)
    xs = synth.normal(n_vec * cols, seed=91).reshape(n_vec, cols)
    d_w = mv.DeviceBuffer.from_host(w)
    d_x = mv.DeviceBuffer.from_host(xs)
    nact = mv.act_bytes(Q5K, cols)
    d_a1, d_a2 = mv.DeviceBuffer(n_vec * nact), mv.DeviceBuffer(n_vec * nact)
    d_o1, d_o2 = mv.DeviceBuffer(n_vec * rows * 4), mv.DeviceBuffer(n_vec * rows * 4)
    mv.quantize(Q5K, d_x.ptr, cols, n_vec, cols, d_a1.ptr)
    mv.gemv_segments(Q5K, mv.make_segments([(d_w.ptr, d_o1.ptr, rows, 0)]), cols, d_a1.ptr, n_vec, rows)
    mv.gemv_segments_f32(Q5K, mv.make_segments([(d_w.ptr, d_o2.ptr, rows, 0)]), cols, d_x.ptr, cols,
                         d_a2.ptr, n_vec, rows)
    assert np.array_equal(d_a1.download(np.uint8, n_vec * nact), d_a2.download(np.uint8, n_vec * nact))
    o1 = d_o1.download(np.float32, n_vec * rows)
    o2 = d_o2.download(np.float32, n_vec * rows)
    assert np.array_equal(bits(o1), bits(o2))
    for v in range(n_vec):
        want, _ = oracle_matvec(Q5K, w, rows, cols, np.ascontiguousarray(xs[v]))
        assert np.array_equal(bits(o1[v * rows:(v + 1) * rows]), bits(want))
