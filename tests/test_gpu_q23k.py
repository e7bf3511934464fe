"""GPU parity for Q2_K (type id 8) and Q3_K (ids 9, 10, 11) weights through the
C ABI, against the CPU oracle and the committed vectors of the compiled
reference (tests/golden/q23_k.npz).

Bars: Q8_K activation bytes, the sixteen integer group sums per super-block and
the f32 outputs are bit-exact (the reference's scalar and dispatched kernels
for these types agree to the bit on the committed raw blocks, and so does its
batch path).
"""
import os
import zlib

import numpy as np
import pytest

import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "q23_k.npz")
Q2K, Q3KS, Q3K, Q3KL = 8, 9, 10, 11


def oracle_matvec(qtype, w, rows, cols, x):
    o = oxlibs.oracle()
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert o.oxo_matvec_quantized(qtype, w.ctypes.data, rows, cols, synth.row_bytes(qtype, cols),
                                  x.ctypes.data, out.ctypes.data, temp.ctypes.data) == 0
    return out, temp


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


@pytest.mark.parametrize("qtype,rows,cols", [
    (Q2K, 1, 256), (Q2K, 7, 256), (Q2K, 64, 512), (Q2K, 333, 4096), (Q2K, 4096, 4096), (Q2K, 100, 14336),
    (Q2K, 4100, 1024), (Q3K, 1, 256), (Q3KS, 7, 256), (Q3KL, 64, 512), (Q3K, 333, 4096), (Q3K, 4096, 4096),
    (Q3K, 100, 14336), (Q3KS, 33, 2816), (Q3K, 4100, 1024),
])
def test_matvec_quantized_bits(oxh, qtype, rows, cols):
    w = synth.weights(qtype, rows, cols, seed=26, stream=rows)
    x = synth.normal(cols, seed=26, stream=9)
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


@pytest.mark.parametrize("qtype,name", [(Q2K, "q2_k"), (Q3K, "q3_k")])
def test_group_sums_bit_exact(oxh, qtype, name):
    rows, cols = 37, 4096
    w = synth.weights(qtype, rows, cols, seed=6)
    x = synth.normal(cols, seed=6)
    o = oxlibs.oracle()
    act = np.zeros(mv.act_bytes(qtype, cols), np.uint8)
    o.oxo_quantize_q8_k(x.ctypes.data, cols, act.ctypes.data)
    blocks, rb = cols // 256, synth.row_bytes(qtype, cols)
    want = np.zeros((rows, blocks, 16), np.int32)
    fo = getattr(o, "oxo_dot_%s_q8_k" % name)
    for r in range(rows):
        fo(w[r * rb:].ctypes.data, blocks, act.ctypes.data, want[r].ctypes.data)
    d_w = mv.DeviceBuffer.from_host(w)
    d_a = mv.DeviceBuffer.from_host(act)
    d_s = mv.DeviceBuffer(want.nbytes)
    mv.debug_subblock_sums(qtype, d_w.ptr, rows, cols, d_a.ptr, d_s.ptr)
    got = d_s.download(np.int32, want.size).reshape(want.shape)
    assert np.array_equal(got, want)


def test_q2k_every_element_position(oxh):
    """One row per element: only that element's code is 3 and its group's scale
    is 1, so the row's output is 3 x d x that element's quantised activation."""
    cols = 256
    w = np.zeros((256, 84), np.uint8)
    w[:, 80:82] = np.array([0x00, 0x3C], np.uint8)                       # d = 1.0, dmin = 0
    for e in range(256):
        n, k, l = e >> 7, (e >> 5) & 3, e & 31
        w[e, e >> 4] = 1
        w[e, 16 + 32 * n + l] = 3 << (2 * k)
    w = np.ascontiguousarray(w.ravel())
    x = synth.normal(cols, seed=3)
    out = np.zeros(256, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(Q2K, w, 256, cols, 84, x, out, temp) == 0
    d = temp.view(np.float32)[0]
    q = temp.view(np.int8)[4:260].astype(np.float32)
    assert np.array_equal(out, d * (np.float32(1.0) * (3.0 * q)))
    want, _ = oracle_matvec(Q2K, w, 256, cols, x)
    assert np.array_equal(bits(out), bits(want))


def test_q3k_third_bit_of_every_element_position(oxh):
    """One row per element: every 2-bit code 0, only that element's third bit set,
    every scale 33 (i.e. +1): the row's output is d*dq*(4*q[e] - 4*sum(q))."""
    cols = 256
    w = np.zeros((256, 110), np.uint8)
    w[:, 108:110] = np.array([0x00, 0x3C], np.uint8)                     # d = 1.0
    w[:, 96:104] = 0x11                                                  # low nibbles: 1
    w[:, 104:108] = 0xAA                                                 # high pairs: 2 -> 33 - 32 = +1
    for e in range(256):
        n, k, l = e >> 7, (e >> 5) & 3, e & 31
        w[e, l] = 1 << (4 * n + k)
    w = np.ascontiguousarray(w.ravel())
    x = synth.normal(cols, seed=4)
    out = np.zeros(256, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(Q3K, w, 256, cols, 110, x, out, temp) == 0
    d = temp.view(np.float32)[0]
    q = temp.view(np.int8)[4:260].astype(np.int64)
    assert np.array_equal(out, (np.float32(1.0) * d) * (4 * q - 4 * q.sum()).astype(np.float32))
    want, _ = oracle_matvec(Q3K, w, 256, cols, x)
    assert np.array_equal(bits(out), bits(want))


@pytest.mark.parametrize("qt", [8, 9, 10, 11])
def test_api_goldens_from_the_compiled_reference(oxh, qt):
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
    # embedding lookup: the reference's dequantised rows
    d_w = mv.DeviceBuffer.from_host(w)
    ids = np.array([0, 1], np.uint32)
    d_ids = mv.DeviceBuffer.from_host(ids)
    d_o = mv.DeviceBuffer(2 * cols * 4)
    mv.get_rows(qt, d_w.ptr, rows, cols, d_ids.ptr, 2, d_o.ptr, cols)
    got = d_o.download(np.float32, 2 * cols).reshape(2, cols)
    assert np.array_equal(bits(got), g[key + "dequant_bits"])


@pytest.mark.parametrize("qt,name", [(8, "big_q2_k_4096x4096"), (10, "big_q3_k_4096x4096")])
def test_full_size_against_reference_checksums(oxh, qt, name):
    g = np.load(GOLD)
    w = synth.weights(qt, 4096, 4096, seed=0, stream=0)
    x = synth.normal(4096, seed=0, stream=1000)
    assert zlib.crc32(w.tobytes()) == int(g[name + "_crc_w"][0])
    out = np.zeros(4096, np.float32)
    temp = np.zeros(4096, np.float32)
    assert mv.matvec_quantized(qt, w, 4096, 4096, synth.row_bytes(qt, 4096), x, out, temp) == 0
    assert zlib.crc32(out.tobytes()) == int(g[name + "_crc_out"][0])
    assert np.array_equal(out, g[name + "_out"])


@pytest.mark.parametrize("qt", [Q2K, Q3K])
def test_fused_multi_input_and_batch(oxh, qt):
    cols, rows = 2048, [300, 0, 5, 64]
    rb = synth.row_bytes(qt, cols)
    ws = [synth.weights(qt, r, cols, seed=31, stream=i) if r else np.zeros(1, np.uint8)
          for i, r in enumerate(rows)]
    x = synth.normal(cols, seed=31, stream=99)
    outs = [np.full(max(r, 1), np.nan, np.float32) for r in rows]
    temp = np.zeros(cols, np.float32)
    oxh.oc_matvec_fused_test_reset()
    assert mv.matvec_quantized_fused([qt] * len(rows), ws, rows, cols, [rb] * len(rows), x, outs, temp) == 0
    st = oxh.oc_matvec_fused_test_stats()
    assert (st.activation_quantizations, st.parallel_dispatches, st.fallback_calls) == (1, 1, 0)
    for w, r, out in zip(ws, rows, outs):
        if r:
            want, _ = oracle_matvec(qt, w, r, cols, x)
            assert np.array_equal(bits(out[:r]), bits(want))
    xs = [synth.normal(cols, seed=41, stream=200 + i) for i in range(len(rows))]
    outs = [np.full(max(r, 1), np.nan, np.float32) for r in rows]
    assert mv.matvec_quantized_multi_input([qt] * len(rows), ws, rows, cols, [rb] * len(rows), xs, outs,
                                           temp) == 0
    for w, r, xv, out in zip(ws, rows, xs, outs):
        if r:
            want, _ = oracle_matvec(qt, w, r, cols, xv)
            assert np.array_equal(bits(out[:r]), bits(want))
    # batches of 1, 8 and 21 vectors with padded strides: every output equals the single-vector result
    w, r = ws[0], rows[0]
    for n_vec in (1, 8, 21):
        in_stride, out_stride = cols + 8, r + 3
        xb = synth.normal(n_vec * in_stride, seed=51, stream=n_vec).reshape(n_vec, in_stride)
        ob = np.full((n_vec, out_stride), -1.0, np.float32)
        scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
        assert mv.matvec_quantized_batch(qt, w, r, cols, rb, xb, in_stride, ob, out_stride, n_vec, temp,
                                         scratch) == 0
        assert np.all(ob[:, r:] == -1.0)
        for v in range(n_vec):
            want, _ = oracle_matvec(qt, w, r, cols, np.ascontiguousarray(xb[v, :cols]))
            assert np.array_equal(bits(ob[v, :r]), bits(want))


@pytest.mark.parametrize("qt", [Q2K, Q3K])
def test_device_segments_with_rmsnorm_prologue_and_pair(oxh, qt):
    """The fused float steps in front of these types too: RMSNorm prologue, then
    a paired segment writing silu(gate)*up; integers bit-exact on the device's
    own normalised vector."""
    o = oxlibs.oracle()
    cols, rows = 1024, 200
    rb = synth.row_bytes(qt, cols)
    wg = synth.weights(qt, rows, cols, seed=61, stream=1)
    wu = synth.weights(qt, rows, cols, seed=61, stream=2)
    x = synth.normal(cols, seed=61, stream=3)
    gamma = synth.normal(cols, seed=61, stream=4)
    d_wg, d_wu = mv.DeviceBuffer.from_host(wg), mv.DeviceBuffer.from_host(wu)
    d_x, d_g = mv.DeviceBuffer.from_host(x), mv.DeviceBuffer.from_host(gamma)
    d_n = mv.DeviceBuffer(cols * 4)
    d_o = mv.DeviceBuffer(rows * 4)
    d_act = mv.DeviceBuffer(mv.act_bytes(qt, cols))
    segs = mv.make_segments([(d_wg.ptr, d_o.ptr, rows, 0, 0, d_wu.ptr)])
    mv.gemv_segments_fused(qt, segs, cols, d_x.ptr, cols, mv.PRO_RMSNORM, d_g.ptr, eps=1e-5, d_pro_out=d_n.ptr,
                           d_act_out=d_act.ptr)
    mv.sync()
    normed = d_n.download(np.float32, cols)
    want_n = np.zeros(cols, np.float32)
    o.oxo_rms_norm_f32(x.ctypes.data, gamma.ctypes.data, want_n.ctypes.data, cols, 1e-5)
    assert np.allclose(normed, want_n, rtol=4e-6, atol=1e-30)
    g_out, temp = oracle_matvec(qt, wg, rows, cols, normed)
    u_out, _ = oracle_matvec(qt, wu, rows, cols, normed)
    assert np.array_equal(d_act.download(np.uint8, mv.act_bytes(qt, cols)), temp.view(np.uint8)[:mv.act_bytes(qt, cols)])
    h = np.zeros(rows, np.float32)
    o.oxo_swiglu_f32(g_out.ctypes.data, u_out.ctypes.data, h.ctypes.data, rows)
    got = d_o.download(np.float32, rows)
    assert np.allclose(got, h, rtol=4e-6, atol=1e-30)


def test_declines_what_the_reference_declines(oxh):
    w = np.zeros(84 * 4, np.uint8)
    x = np.zeros(300, np.float32)
    out, temp = np.zeros(4, np.float32), np.zeros(300, np.float32)
    assert mv.matvec_quantized(Q2K, w, 4, 300, 84, x, out, temp) == mv.DECLINED      # cols not in whole blocks
    x = np.zeros(256, np.float32)
    assert mv.matvec_quantized(Q3K, w, 3, 256, 112, x, out, temp) == mv.DECLINED     # padded row stride


def test_q3k_rewritten_as_q6k_bytes(oxh):
    """The device rewrite against the element-by-element numpy statement: raw random blocks (every
    scale value, every third-bit pattern) and generator blocks, block counts that do and do not fill
    the last workgroup."""
    from q3k_rewrite import q3k_as_q6k
    g = np.load(GOLD)
    raw = np.ascontiguousarray(g["q3_k_raw_w"]).reshape(-1)                 # 288 blocks
    rng = np.random.default_rng(3)
    rnd = rng.integers(0, 256, 110 * 1027, dtype=np.uint8)
    for w, rows, cols in ((raw, 24, 12 * 256), (rnd, 1027, 256), (rnd[:110], 1, 256),
                          (synth.weights(Q3K, 130, 2048, seed=8), 130, 2048)):
        d_w = mv.DeviceBuffer.from_host(w)
        d_o = mv.DeviceBuffer(rows * (cols // 256) * 210)
        mv.q3_k_as_q6_k(d_w.ptr, rows, cols, d_o.ptr)
        assert np.array_equal(d_o.download(np.uint8, rows * (cols // 256) * 210), q3k_as_q6k(w))
    with pytest.raises(Exception):
        mv.q3_k_as_q6_k(d_w.ptr, 1, 200, d_o.ptr)
    mv.q3_k_as_q6_k(0, 0, 256, 0)           # no rows: nothing to do


def test_q2k_widened_bytes(oxh):
    """The device widening of Q2_K blocks against the element-by-element numpy statement."""
    from q3k_rewrite import q2k_widen
    g = np.load(GOLD)
    raw = np.ascontiguousarray(g["q2_k_raw_w"]).reshape(-1)
    rnd = np.random.default_rng(4).integers(0, 256, 84 * 1027, dtype=np.uint8)
    for w, rows, cols in ((raw, 24, 12 * 256), (rnd, 1027, 256), (rnd[:84], 1, 256),
                          (synth.weights(Q2K, 130, 2048, seed=8), 130, 2048)):
        d_w = mv.DeviceBuffer.from_host(w)
        d_o = mv.DeviceBuffer(rows * (cols // 256) * 210)
        mv.q2_k_widen(d_w.ptr, rows, cols, d_o.ptr)
        assert np.array_equal(d_o.download(np.uint8, rows * (cols // 256) * 210), q2k_widen(w))
    with pytest.raises(Exception):
        mv.q2_k_widen(d_w.ptr, 1, 200, d_o.ptr)


@pytest.mark.parametrize("n_vec", [1, 16, 17, 40, 130])
def test_q2k_wide_tile_kernel_on_raw_blocks(oxh, n_vec):
    """oxh_mmq on widened raw random Q2_K blocks (every scale, minimum and code value, arbitrary f16 d and
    dmin as far as they are finite) against the oracle's Q2_K dot of the original blocks, bit for bit,
    through every tile shape."""
    rows, cols = 203, 1024
    rng = np.random.default_rng(n_vec)
    w = rng.integers(0, 256, rows * 4 * 84, dtype=np.uint8).reshape(-1, 84)
    w[:, 81] &= 0x3B          # |d|, |dmin| below 2: finite, products stay finite
    w[:, 83] &= 0x3B
    w = w.reshape(-1)
    x = synth.normal(n_vec * cols, seed=5, stream=n_vec)
    o = oxlibs.oracle()
    act = np.zeros(n_vec * 4 * 292, np.uint8)
    for v in range(n_vec):
        o.oxo_quantize_q8_k(x[v * cols:].ctypes.data, cols, act[v * 4 * 292:].ctypes.data)
    want = np.zeros((n_vec, rows), np.float32)
    for v in range(n_vec):
        for r in range(rows):
            want[v, r] = o.oxo_dot_q2_k_q8_k(w[r * 4 * 84:].ctypes.data, 4, act[v * 4 * 292:].ctypes.data, None)
    d_w = mv.DeviceBuffer.from_host(w)
    d_wide = mv.DeviceBuffer(rows * 4 * 210)
    mv.q2_k_widen(d_w.ptr, rows, cols, d_wide.ptr)
    d_a = mv.DeviceBuffer.from_host(act)
    d_o = mv.DeviceBuffer(n_vec * rows * 4)
    mv.mmq(mv.Q2_K_WIDE, d_wide.ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows)
    got = d_o.download(np.float32, n_vec * rows).reshape(n_vec, rows)
    assert np.array_equal(bits(got), bits(want))
    # the widened blocks with a tile's columns shared between workgroups (four super-blocks are too few
    # to split: a wider matrix of the same blocks against the unsplit launch)
    wide_rows = rows // 14
    need = mv.mmq_split_workspace(mv.Q2_K_WIDE, wide_rows, 14 * cols, n_vec, wide_rows)
    if n_vec <= 64:
        assert need == 56 * n_vec * wide_rows * 4
        d_a14 = mv.DeviceBuffer.from_host(np.tile(act.reshape(n_vec, -1), (1, 14)).reshape(-1))
        d_ws = mv.DeviceBuffer(need)
        d_o1, d_o2 = mv.DeviceBuffer(n_vec * wide_rows * 4), mv.DeviceBuffer(n_vec * wide_rows * 4)
        mv.mmq(mv.Q2_K_WIDE, d_wide.ptr, wide_rows, 14 * cols, d_a14.ptr, n_vec, d_o1.ptr, wide_rows)
        mv.mmq_split(mv.Q2_K_WIDE, d_wide.ptr, wide_rows, 14 * cols, d_a14.ptr, n_vec, d_o2.ptr, wide_rows,
                     d_ws.ptr, need)
        assert np.array_equal(d_o1.download(np.uint32, n_vec * wide_rows), d_o2.download(np.uint32, n_vec * wide_rows))
    else:
        assert need == 0
    # the widened blocks are no GGUF type: every other entry point refuses the id
    seg = mv.make_segments([(d_wide.ptr, d_o.ptr, rows, 0)])
    with pytest.raises(Exception):
        mv.gemv_segments(mv.Q2_K_WIDE, seg, cols, d_a.ptr, 1, rows)


@pytest.mark.parametrize("qt,rows,cols,n_vec", [(Q3K, 300, 2048, 9), (Q3KS, 65, 256, 16), (Q3KL, 1, 512, 33),
                                                (Q3K, 1000, 4096, 100), (Q3K, 4096, 4096, 512),
                                                (Q2K, 300, 2048, 9), (Q2K, 65, 256, 16), (Q2K, 1, 512, 33),
                                                (Q2K, 1000, 4096, 100), (Q2K, 4096, 4096, 512)])
def test_q23k_prefill_batches_on_the_matrix_cores(oxh, qt, rows, cols, n_vec):
    """More than eight vectors of Q2_K / Q3_K weights go through the rewrite and the Q6_K tile kernel:
    every output still has the bits of the single-vector dot."""
    rb = synth.row_bytes(qt, cols)
    w = synth.weights(qt, rows, cols, seed=61, stream=n_vec)
    in_stride, out_stride = cols + 8, rows + 3
    xb = synth.normal(n_vec * in_stride, seed=62, stream=n_vec).reshape(n_vec, in_stride)
    ob = np.full((n_vec, out_stride), -1.0, np.float32)
    temp = np.zeros(cols, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    assert mv.matvec_quantized_batch(qt, w, rows, cols, rb, xb, in_stride, ob, out_stride, n_vec, temp,
                                     scratch) == 0
    assert np.all(ob[:, rows:] == -1.0)
    o = oxlibs.oracle()
    want = np.zeros((n_vec, out_stride), np.float32)
    act = np.zeros(scratch.size, np.uint8)
    assert o.oxo_matvec_quantized_batch(qt, w.ctypes.data, rows, cols, rb, xb.ctypes.data, in_stride,
                                        want.ctypes.data, out_stride, n_vec, act.ctypes.data, act.size) == 0
    assert np.array_equal(bits(ob[:, :rows]), bits(want[:, :rows]))
