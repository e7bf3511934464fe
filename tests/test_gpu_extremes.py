"""GPU parity on the largest integers the formats can produce: every code, scale
and minimum at its maximum (or minimum), activations that quantise to +127 or
-127 throughout, so that sub-block sums, the scale-folded int8 operands of the
matrix-core kernels, their 16-bit intermediate steps, the f16 sums behind the
Q4_K / Q5_K minimum term and the 24-bit multiplies of the dot kernels all sit at
their bounds.  Every path (one vector, small batches on the matrix cores, the
prefill tiles) must still give the oracle's bits."""
import numpy as np
import pytest

import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth

pytestmark = pytest.mark.gpu

from extremes import TYPES, bits, extreme_inputs, extreme_weights, quantiser_edge_inputs


@pytest.mark.parametrize("n_vec", [1, 4, 8, 12, 40, 200])
@pytest.mark.parametrize("qt", sorted(TYPES))
def test_extreme_integers_every_path(oxh, qt, n_vec):
    layout, fields = TYPES[qt]
    per = synth.BLOCK_ELEMS[layout]
    rows, cols = 130, (1024 if per == 256 else 512)
    rb = synth.row_bytes(layout, cols)
    w = extreme_weights(layout, fields, rows, cols)
    xs = extreme_inputs(n_vec, cols)
    o = oxlibs.oracle()
    want = np.zeros((n_vec, rows), np.float32)
    sc = np.zeros(o.oxo_matvec_batch_scratch_bytes(cols), np.uint8)
    assert o.oxo_matvec_quantized_batch(qt, w.ctypes.data, rows, cols, rb, xs.ctypes.data, cols,
                                        want.ctypes.data, rows, n_vec, sc.ctypes.data, sc.nbytes) == 0
    assert np.all(np.isfinite(want))
    act = np.frombuffer(sc.tobytes()[:mv.act_bytes(qt, cols)], np.uint8)
    q = act[4:260].view(np.int8) if per == 256 else act[2:34].view(np.int8)
    assert set(np.abs(q.astype(np.int32))) == {127}                       # the inputs do sit at the bound
    got = np.full((n_vec, rows), -1.0, np.float32)
    temp = np.zeros(cols, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    assert mv.matvec_quantized_batch(qt, w, rows, cols, rb, xs, cols, got, rows, n_vec, temp, scratch) == 0
    assert np.array_equal(bits(got), bits(want)), (qt, n_vec)
    if n_vec == 1:
        one = np.zeros(rows, np.float32)
        assert mv.matvec_quantized(qt, w, rows, cols, rb, np.ascontiguousarray(xs[0]), one, temp) == 0
        assert np.array_equal(bits(one), bits(want[0]))
    # the device-resident layer with a buffer for the quantised activations: three or more vectors of
    # a K-quant and five or more of a 32-value format run on the matrix cores
    if 3 <= n_vec <= 12:
        d_w, d_x = mv.DeviceBuffer.from_host(w), mv.DeviceBuffer.from_host(xs)
        d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(qt, cols))
        d_o = mv.DeviceBuffer(n_vec * rows * 4)
        if n_vec <= 8 or qt in (13, 15, 16, 7, 3, 4, 5, 6, 18):
            mv.gemv_segments_f32(qt, mv.make_segments([(d_w.ptr, d_o.ptr, rows, 0)]), cols, d_x.ptr, cols,
                                 d_a.ptr, n_vec, rows)
            dev = d_o.download(np.float32, n_vec * rows).reshape(n_vec, rows)
            assert np.array_equal(bits(dev), bits(want)), (qt, n_vec, "segments")


@pytest.mark.parametrize("rows", [14336, 4096])
@pytest.mark.parametrize("qt", [13, 15, 16, 8, 10])
def test_extreme_integers_large_prefill_tiles(oxh, qt, rows):
    """The same bounds through the large prefill tiles (256 x 128 and 128 x 128 at 14336 rows, 128 x 64 and
    Q6_K's 64 x 128 at 4096 rows on a 256-CU device; Q2_K and Q3_K through their rewrite), 512 vectors, a
    sample of them against the oracle."""
    layout, fields = TYPES[qt]
    cols, n_vec = 512, 512
    rb = synth.row_bytes(layout, cols)
    w = extreme_weights(layout, fields, rows, cols)
    xs = extreme_inputs(n_vec, cols)
    got = np.zeros((n_vec, rows), np.float32)
    temp = np.zeros(cols, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    assert mv.matvec_quantized_batch(qt, w, rows, cols, rb, xs, cols, got, rows, n_vec, temp, scratch) == 0
    o = oxlibs.oracle()
    for v in (0, 1, 2, 3, 4, 5, 130, 511):
        want = np.zeros(rows, np.float32)
        assert o.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, np.ascontiguousarray(xs[v]).ctypes.data,
                                      want.ctypes.data, temp.ctypes.data) == 0
        assert np.array_equal(bits(got[v]), bits(want)), (qt, rows, v)


@pytest.mark.parametrize("qt", [13, 7])
def test_quantiser_edge_inputs_bit_exact(oxh, qt):
    """Rounding ties, magnitudes up to the largest float, subnormal block scales: the stand-alone
    quantiser and the one fused into a GEMV launch both give the oracle's bytes.  (Blocks whose largest
    magnitude is below 3.7e-37, where 1/d overflows, and non-finite inputs are not compared: there the
    reference's own scalar and AVX-512 quantisers disagree with each other.)"""
    n = 512
    o = oxlibs.oracle()
    fn = o.oxo_quantize_q8_k if qt == 13 else o.oxo_quantize_q8_0
    nb = mv.act_bytes(qt, n)
    w = synth.weights(qt, 16, n, seed=2)
    d_w, d_o = mv.DeviceBuffer.from_host(w), mv.DeviceBuffer(64)
    for name, x in quantiser_edge_inputs(n).items():
        want = np.zeros(nb, np.uint8)
        fn(x.ctypes.data, n, want.ctypes.data)
        d_x, d_a, d_a2 = mv.DeviceBuffer.from_host(x), mv.DeviceBuffer(nb), mv.DeviceBuffer(nb)
        mv.quantize(qt, d_x.ptr, n, 1, n, d_a.ptr)
        assert np.array_equal(d_a.download(np.uint8, nb), want), name
        mv.gemv_segments_f32(qt, mv.make_segments([(d_w.ptr, d_o.ptr, 16, 0)]), n, d_x.ptr, n, d_a2.ptr, 1, 16)
        assert np.array_equal(d_a2.download(np.uint8, nb), want), name + " (fused)"
        ref = oxlibs.ref()
        if ref is not None:
            out, temp = np.zeros(16, np.float32), np.zeros(n, np.float32)
            ref.oc_matvec_quantized(qt, w.ctypes.data, 16, n, synth.row_bytes(qt, n), x.ctypes.data,
                                    out.ctypes.data, temp.ctypes.data)
            assert np.array_equal(temp.view(np.uint8)[:nb], want), name + " (compiled reference)"
