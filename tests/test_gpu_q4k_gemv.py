"""GPU parity: Q8_K activation quantiser and Q4_K x Q8_K decode GEMV against
the CPU oracle, through the C ABI.  Bit-exact bars: activation bytes,
per-sub-block int32 sums and (for the K-quants) the final f32 bits."""
import numpy as np
import pytest

import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth

pytestmark = pytest.mark.gpu

Q4K = 13


def oracle_matvec(qtype, w, rows, cols, x):
    o = oxlibs.oracle()
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    rc = o.oxo_matvec_quantized(qtype, w.ctypes.data, rows, cols, synth.row_bytes(qtype, cols),
                                x.ctypes.data, out.ctypes.data, temp.ctypes.data)
    assert rc == 0
    return out, temp


@pytest.mark.parametrize("cols", [256, 512, 4096, 14336])
def test_quantize_q8_k_bytes_bit_exact(oxh, cols):
    n_vec = 3
    x = synth.normal(n_vec * cols, seed=3, stream=cols).reshape(n_vec, cols)
    x[1, :256] = 0.0                      # an all-zero block: d = 0, q = 0
    x[2, 5] = 1e-30                       # tiny values next to normal ones
    nbytes = mv.act_bytes(Q4K, cols)
    d_x = mv.DeviceBuffer.from_host(x)
    d_a = mv.DeviceBuffer(n_vec * nbytes)
    mv.quantize(Q4K, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    got = d_a.download(np.uint8, n_vec * nbytes).reshape(n_vec, nbytes)
    o = oxlibs.oracle()
    for v in range(n_vec):
        want = np.zeros(nbytes, np.uint8)
        o.oxo_quantize_q8_k(x[v].ctypes.data, cols, want.ctypes.data)
        assert np.array_equal(got[v], want), "vector %d" % v


@pytest.mark.parametrize("rows,cols", [(1, 256), (7, 256), (64, 512), (333, 4096),
                                       (40, 14336), (130, 2816)])
def test_matvec_quantized_q4k_bits(oxh, rows, cols):
    w = synth.weights(Q4K, rows, cols, seed=11, stream=rows)
    x = synth.normal(cols, seed=11, stream=7)
    out = np.full(rows, np.nan, np.float32)
    temp = np.zeros(cols, np.float32)
    rc = mv.matvec_quantized(Q4K, w, rows, cols, synth.row_bytes(Q4K, cols), x, out, temp)
    assert rc == 0
    want, want_temp = oracle_matvec(Q4K, w, rows, cols, x)
    nact = mv.act_bytes(Q4K, cols)
    assert np.array_equal(temp.view(np.uint8)[:nact], want_temp.view(np.uint8)[:nact])
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


def test_q4k_subblock_sums_bit_exact(oxh):
    rows, cols = 50, 4096
    w = synth.weights(Q4K, rows, cols, seed=5)
    x = synth.normal(cols, seed=5)
    o = oxlibs.oracle()
    nact = mv.act_bytes(Q4K, cols)
    act = np.zeros(nact, np.uint8)
    o.oxo_quantize_q8_k(x.ctypes.data, cols, act.ctypes.data)
    blocks = cols // 256
    want = np.zeros((rows, blocks, 8), np.int32)
    rb = synth.row_bytes(Q4K, cols)
    for r in range(rows):
        o.oxo_dot_q4_k_q8_k(w[r * rb:].ctypes.data, blocks, act.ctypes.data,
                            want[r].ctypes.data, None)
    d_w = mv.DeviceBuffer.from_host(w)
    d_a = mv.DeviceBuffer.from_host(act)
    d_s = mv.DeviceBuffer(want.nbytes)
    mv.debug_subblock_sums(Q4K, d_w.ptr, rows, cols, d_a.ptr, d_s.ptr)
    got = d_s.download(np.int32, want.size).reshape(want.shape)
    assert np.array_equal(got, want)
