"""IQ4_NL and IQ4_XS on the device (the 4-bit codebook formats of the reference's dequantise path,
oxidize-c/src/compute/matvec.c:799-831, :886-907; its own device path has kernels for them,
oxidize-c/src/backends/cuda_mmq.cu:355-450).

Bars.  The embedding lookup expands rows to the oracle's bits (oxo_dequant_row, itself the compiled
reference's bits: tests/test_oracle_iq4.py).  The matvec is an f32 dot over those values, so it is held
to the double-precision restatement within 4e-6 of the row's sum of magnitudes: what f32 summation in
another order can differ by, and far inside the 1e-2 of the reference's own variant tests
(oxidize-c/tests/test_oxk_iq3_s.c:266-270).  The host entry points decline these types unless the
process opted in (OXH_F32_PATH_TYPES=1), which a separate process checks."""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

import oxlibs
from oxidize_amd import _lib, synth
from oxidize_amd import matvec as mv

pytestmark = pytest.mark.gpu
TYPES = (26, 27)
TOL = 4e-6


def want_rows(qt, w, rows, cols, x):
    o = oxlibs.oracle()
    out, mag = np.zeros(rows, np.float64), np.zeros(rows, np.float64)
    assert o.oxo_matvec_dequant(qt, w.ctypes.data, rows, cols, synth.row_bytes(qt, cols), x.ctypes.data,
                                out.ctypes.data, mag.ctypes.data) == 0
    return out, mag


@pytest.mark.parametrize("qt", TYPES)
@pytest.mark.parametrize("rows,cols", [(1, 256), (37, 512), (300, 4096), (4100, 4096), (130, 14336), (5000, 1024)])
def test_f32_path_gemv(oxh, qt, rows, cols):
    assert oxh.oxh_act_kind(qt, cols) == 0 and oxh.oxh_row_bytes(qt, cols) == 0        # no integer path
    assert oxh.oxh_f32_path_row_bytes(qt, cols) == synth.row_bytes(qt, cols)
    w = synth.weights(qt, rows, cols, seed=rows, stream=qt)
    x = synth.normal(cols, seed=cols, stream=qt)
    d_w, d_x = mv.DeviceBuffer.from_host(w), mv.DeviceBuffer.from_host(x)
    d_o = mv.DeviceBuffer(rows * 4)
    segs = (_lib.OxhSegment * 1)(_lib.OxhSegment(d_w.ptr, d_o.ptr, rows, 0, 0, None))
    mv.gemv_segments_f32(qt, segs, cols, d_x.ptr, cols, None, 1, rows)
    got = d_o.download(np.float32, rows)
    want, mag = want_rows(qt, w, rows, cols, x)
    assert np.all(np.abs(got.astype(np.float64) - want) <= TOL * mag + 1e-30)
    for b in (d_w, d_x, d_o):
        b.free()


@pytest.mark.parametrize("qt", TYPES)
def test_segments_with_their_own_runs_of_inputs(oxh, qt):
    """Two matrices in one call, the second over inputs 2..4 of a padded batch."""
    cols, stride = 1024, 1032
    shapes = [(96, 0, 2), (61, 2, 3)]
    xs = synth.normal(5 * stride, seed=3, stream=qt).reshape(5, stride)
    d_x = mv.DeviceBuffer.from_host(xs)
    ws = [synth.weights(qt, r, cols, seed=5, stream=i) for i, (r, _, _) in enumerate(shapes)]
    d_ws = [mv.DeviceBuffer.from_host(w) for w in ws]
    out_stride = 100
    d_os = [mv.DeviceBuffer(nv * out_stride * 4) for _, _, nv in shapes]
    segs = (_lib.OxhSegment * 2)(*[_lib.OxhSegment(d_ws[i].ptr, d_os[i].ptr, r, first, nv, None)
                                   for i, (r, first, nv) in enumerate(shapes)])
    mv.gemv_segments_f32(qt, segs, cols, d_x.ptr, stride, None, 1, out_stride)
    for i, (r, first, nv) in enumerate(shapes):
        got = d_os[i].download(np.float32, nv * out_stride).reshape(nv, out_stride)
        for v in range(nv):
            want, mag = want_rows(qt, ws[i], r, cols, np.ascontiguousarray(xs[first + v, :cols]))
            assert np.all(np.abs(got[v, :r].astype(np.float64) - want) <= TOL * mag)
    # a buffer for quantised activations makes no sense here, and neither does the integer entry point
    with pytest.raises(mv.OxhError) as e:
        mv.gemv_segments_f32(qt, segs, cols, d_x.ptr, stride, d_x.ptr, 1, out_stride)
    assert e.value.status == _lib.ERR_ARG
    assert oxh.oxh_gemv_segments(qt, segs, 2, cols, ctypes.c_void_p(d_x.ptr), 1, out_stride, None) == _lib.DECLINED
    for b in [d_x] + d_ws + d_os:
        b.free()


@pytest.mark.parametrize("qt", TYPES)
def test_get_rows_bits(oxh, qt):
    rows, cols = 50, 1280
    rb = synth.row_bytes(qt, cols)
    w = synth.weights(qt, rows, cols, seed=11, stream=qt)
    ids = np.array([0, 49, 7, 7, 23, 60], np.uint32)          # 60 is past the table: a row of zeros
    d_w, d_ids = mv.DeviceBuffer.from_host(w), mv.DeviceBuffer.from_host(ids)
    d_o = mv.DeviceBuffer(ids.size * cols * 4)
    mv.get_rows(qt, d_w.ptr, rows, cols, d_ids.ptr, ids.size, d_o.ptr, cols)
    got = d_o.download(np.float32, ids.size * cols).reshape(ids.size, cols)
    o = oxlibs.oracle()
    for k, i in enumerate(ids):
        want = np.zeros(cols, np.float32)
        if i < rows:
            assert o.oxo_dequant_row(qt, w[int(i) * rb:].ctypes.data, cols, want.ctypes.data) == 0
        assert np.array_equal(got[k].view(np.uint32), want.view(np.uint32)), k
    for b in (d_w, d_ids, d_o):
        b.free()


def test_golden_vectors_from_the_reference(oxh):
    g = np.load(os.path.join(oxlibs.ROOT, "tests", "golden", "iq4_types.npz"))
    for name, qt in (("iq4_nl", 26), ("iq4_xs", 27)):
        rows, cols, rb = (int(v) for v in g[name + "_api_shape"])
        w, x = np.ascontiguousarray(g[name + "_api_w"]), np.ascontiguousarray(g[name + "_api_x"])
        d_w, d_x, d_o = mv.DeviceBuffer.from_host(w), mv.DeviceBuffer.from_host(x), mv.DeviceBuffer(rows * 4)
        segs = (_lib.OxhSegment * 1)(_lib.OxhSegment(d_w.ptr, d_o.ptr, rows, 0, 0, None))
        mv.gemv_segments_f32(qt, segs, cols, d_x.ptr, cols, None, 1, rows)
        got = d_o.download(np.float32, rows)
        _, mag = want_rows(qt, w, rows, cols, x)
        # the compiled reference's own f32 result on its host: two f32 summation orders apart
        assert np.all(np.abs(got.astype(np.float64) - g[name + "_api_out"].astype(np.float64)) <= 2 * TOL * mag)
        for b in (d_w, d_x, d_o):
            b.free()


def test_host_entry_points_decline_by_default(oxh):
    for qt in TYPES:
        rows, cols = 16, 512
        w = synth.weights(qt, rows, cols, seed=1)
        x = synth.normal(cols, seed=1)
        out = np.full(rows, 5.0, np.float32)
        temp = np.zeros(cols, np.float32)
        assert mv.matvec_quantized(qt, w, rows, cols, synth.row_bytes(qt, cols), x, out, temp) == _lib.DECLINED
        assert np.all(out == 5.0)


OPT_IN = r"""
import sys
import numpy as np
sys.path.insert(0, %(root)r); sys.path.insert(0, %(root)r + "/tests")
import oxlibs
from oxidize_amd import _lib, synth
from oxidize_amd import matvec as mv
_lib.check(_lib.lib().oxh_init(0))
for qt in (26, 27):
    rows, cols = 700, 2048
    rb = synth.row_bytes(qt, cols)
    w = synth.weights(qt, rows, cols, seed=2, stream=qt)
    x = synth.normal(cols, seed=2)
    out = np.zeros(rows, np.float32)
    temp = np.full(cols, 3.0, np.float32)
    assert mv.matvec_quantized(qt, w, rows, cols, rb, x, out, temp) == 0
    want, mag = np.zeros(rows), np.zeros(rows)
    assert oxlibs.oracle().oxo_matvec_dequant(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, want.ctypes.data, mag.ctypes.data) == 0
    assert np.all(np.abs(out.astype(np.float64) - want) <= 4e-6 * mag)
    assert mv.matvec_quantized(qt, w, rows, cols, rb + 2, x, out, temp) == _lib.DECLINED      # padded stride
print("opt-in ok")
"""


def test_host_entry_point_when_opted_in(oxh):
    env = dict(os.environ, OXH_F32_PATH_TYPES="1")
    proc = subprocess.run([sys.executable, "-c", OPT_IN % {"root": oxlibs.ROOT}], env=env, stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=150)
    assert proc.returncode == 0 and "opt-in ok" in proc.stdout, proc.stdout
