"""IQ3_S and IQ1_XXXS (the two codebook formats the reference's integer path accepts,
oxidize-c/src/compute/matvec.c:121-122) through the C ABI against the oracle, which is pinned on the
compiled reference for both (tests/test_oracle_iq.py): outputs bit for bit, single vector, grouped,
small batches, padded batches, the device-resident layer with several activations, and fused prologues."""
import ctypes

import numpy as np
import pytest

import oxlibs
from oxidize_amd import _lib, synth
from oxidize_amd import matvec as mv

pytestmark = pytest.mark.gpu
IQ3S, IQ1X = 25, 36


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def oracle_matvec(qt, w, rows, cols, x):
    o = oxlibs.oracle()
    want = np.zeros(rows, np.float32)
    tmp = np.zeros(cols, np.float32)
    assert o.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, synth.row_bytes(qt, cols), x.ctypes.data,
                                  want.ctypes.data, tmp.ctypes.data) == 0
    return want, tmp.view(np.uint8)[:cols // 256 * 292].copy()


@pytest.mark.parametrize("qt", [IQ3S, IQ1X])
@pytest.mark.parametrize("rows,cols", [(1, 256), (37, 512), (300, 4096), (4096, 4096), (130, 14336), (5000, 1024)])
def test_matvec_bits(oxh, qt, rows, cols):
    assert oxh.oxh_act_kind(qt, cols) == 2 and oxh.oxh_row_bytes(qt, cols) == synth.row_bytes(qt, cols)
    w = synth.weights(qt, rows, cols, seed=rows, stream=qt)
    x = synth.normal(cols, seed=cols, stream=qt)
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(qt, w, rows, cols, synth.row_bytes(qt, cols), x, out, temp) == 0
    want, act = oracle_matvec(qt, w, rows, cols, x)
    assert np.array_equal(temp.view(np.uint8)[:act.size], act)
    assert np.array_equal(bits(out), bits(want))


@pytest.mark.parametrize("qt", [IQ3S, IQ1X])
def test_golden_vectors_from_the_reference(oxh, qt):
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "iq_types.npz"))
    key = "api%d_" % qt
    rows, cols, rb = (int(v) for v in g[key + "shape"])
    w, x = np.ascontiguousarray(g[key + "w"]), np.ascontiguousarray(g[key + "x"])
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(qt, w, rows, cols, rb, x, out, temp) == 0
    assert np.array_equal(bits(out), g[key + "out_bits"])
    xs = np.ascontiguousarray(g[key + "batch_x"])
    n_vec, in_stride = xs.shape
    want = g[key + "batch_out_bits"]
    outs = np.full(want.shape, -1.0, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    assert mv.matvec_quantized_batch(qt, w, rows, cols, rb, xs, in_stride, outs, want.shape[1], n_vec, temp,
                                     scratch) == 0
    assert np.array_equal(bits(outs), want)


@pytest.mark.parametrize("qt", [IQ3S, IQ1X])
def test_grouped_batch_and_declines(oxh, qt):
    rows, cols = 96, 1024
    rb = synth.row_bytes(qt, cols)
    ws = [synth.weights(qt, rows + 8 * k, cols, seed=3, stream=k) for k in range(3)]
    x = synth.normal(cols, seed=4)
    outs = [np.zeros(rows + 8 * k, np.float32) for k in range(3)]
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized_fused([qt] * 3, ws, [rows, rows + 8, rows + 16], cols, [rb] * 3, x, outs, temp) == 0
    for k in range(3):
        want, _ = oracle_matvec(qt, ws[k], rows + 8 * k, cols, x)
        assert np.array_equal(bits(outs[k]), bits(want))
    # 21 vectors: slices of at most 8 through the same kernels
    n_vec = 21
    xs = synth.normal(n_vec * cols, seed=5).reshape(n_vec, cols)
    got = np.zeros((n_vec, rows), np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    assert mv.matvec_quantized_batch(qt, ws[0], rows, cols, rb, xs, cols, got, rows, n_vec, temp, scratch) == 0
    for v in range(n_vec):
        want, _ = oracle_matvec(qt, ws[0], rows, cols, xs[v])
        assert np.array_equal(bits(got[v]), bits(want)), v
    # cols not in whole 256-blocks: declined like the reference (matvec.c:99-127)
    assert mv.matvec_quantized(qt, ws[0], 4, 1000, 1000 // 256 * synth.BLOCK_BYTES[qt], x, outs[0], temp) == mv.DECLINED


@pytest.mark.parametrize("qt", [IQ3S, IQ1X])
def test_device_layer_several_activations_and_pairs(oxh, qt):
    rows, cols, nv = 200, 2048, 5
    w = synth.weights(qt, rows, cols, seed=11, stream=qt)
    w2 = synth.weights(qt, rows, cols, seed=12, stream=qt)
    xs = synth.normal(nv * cols, seed=13).reshape(nv, cols)
    d_w, d_w2 = mv.DeviceBuffer.from_host(w), mv.DeviceBuffer.from_host(w2)
    d_x = mv.DeviceBuffer.from_host(xs)
    d_o = mv.DeviceBuffer(nv * rows * 4)
    segs = mv.make_segments([(d_w.ptr, d_o.ptr, rows, 0)])
    mv.gemv_segments_f32(qt, segs, cols, d_x.ptr, cols, None, nv, rows)
    mv.sync()
    got = d_o.download(np.float32, nv * rows).reshape(nv, rows)
    for v in range(nv):
        want, _ = oracle_matvec(qt, w, rows, cols, xs[v])
        assert np.array_equal(bits(got[v]), bits(want)), v
    # a gate/up pair: silu(first) * second from the oracle's two dots (expf on the device vs libm: rounding)
    segs = mv.make_segments([(d_w.ptr, d_o.ptr, rows, 0, 0, d_w2.ptr)])
    _lib.check(oxh.oxh_gemv_segments_fused(qt, segs, 1, cols, ctypes.c_void_p(d_x.ptr), cols, None, None, 1, rows, None))
    mv.sync()
    h = d_o.download(np.float32, rows)
    g, _ = oracle_matvec(qt, w, rows, cols, xs[0])
    u, _ = oracle_matvec(qt, w2, rows, cols, xs[0])
    ref = (g.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64))) * u.astype(np.float64))
    assert np.allclose(h, ref, rtol=3e-6, atol=1e-6)


def test_what_stays_declined_for_codebook_formats(oxh):
    d = mv.DeviceBuffer(1 << 16)
    ids = mv.DeviceBuffer.from_host(np.zeros(4, np.uint32))
    out = mv.DeviceBuffer(4 * 1024 * 4)
    for qt in (IQ3S, IQ1X):
        assert oxh.oxh_get_rows(qt, ctypes.c_void_p(d.ptr), 8, 1024, ctypes.c_void_p(ids.ptr), 4,
                                ctypes.c_void_p(out.ptr), 1024, None) == _lib.DECLINED
        assert oxh.oxh_mmq(qt, ctypes.c_void_p(d.ptr), 8, 1024, ctypes.c_void_p(d.ptr), 16,
                           ctypes.c_void_p(out.ptr), 8, None) == _lib.DECLINED
    for qt in (21, 22, 23, 24, 26, 27, 28, 29):          # every other IQ id: no integer path in the reference either
        assert oxh.oxh_act_kind(qt, 4096) == 0
