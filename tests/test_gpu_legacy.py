"""GPU parity for the 32-value formats Q4_0, Q4_1, Q5_0, Q5_1 (type ids 3-6) and
AL5_XS (id 18; 3-bit codes), Q8_0 activations, through the C ABI.

Bars: Q8_0 activation bytes and the per-block integers bit-exact; f32 outputs
bit-exact against the oracle's block-sequential chain (oxk.c:88-191) and within
|a-b| <= 1e-4 + 1e-5*|ref| of the compiled reference's entry points, whose x86
row kernels add the same per-block terms in f32 lanes."""
import os

import numpy as np
import pytest

import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "legacy_formats.npz")
LEGACY = (("q4_0", 3), ("q4_1", 4), ("q5_0", 5), ("q5_1", 6), ("al5_xs", 18))
FLOAT_RTOL = 4e-6


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def oracle_matvec(qtype, w, rows, cols, x):
    o = oxlibs.oracle()
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert o.oxo_matvec_quantized(qtype, w.ctypes.data, rows, cols, synth.row_bytes(qtype, cols),
                                  x.ctypes.data, out.ctypes.data, temp.ctypes.data) == 0
    return out, temp


@pytest.mark.parametrize("name,qtype", LEGACY)
@pytest.mark.parametrize("rows,cols", [(1, 32), (5, 96), (1000, 896), (300, 4864), (4096, 4096), (77, 14336)])
def test_matvec_quantized_bits(oxh, name, qtype, rows, cols):
    w = synth.weights(qtype, rows, cols, seed=41, stream=rows)
    x = synth.normal(cols, seed=41, stream=9)
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
        ref.oc_matvec_quantized(qtype, w.ctypes.data, rows, cols, rb, x.ctypes.data, r_out.ctypes.data,
                                r_tmp.ctypes.data)
        assert np.array_equal(temp.view(np.uint8)[:nact], r_tmp.view(np.uint8)[:nact])
        assert np.all(np.abs(out - r_out) <= 1e-4 + 1e-5 * np.abs(r_out))


@pytest.mark.parametrize("qtype", [3, 17])
@pytest.mark.parametrize("rows,cols", [(5, 96), (64, 4096)])
def test_block_sums_left_behind_the_activation(oxh, qtype, rows, cols):
    """Q4_0 and AL5: the int32 sum of every activation block follows the blocks in temp, from the next
    multiple of four bytes on (matvec.c:198-227, :866-877)."""
    w = synth.weights(3, rows, cols, seed=43, stream=rows)        # AL5 is the Q4_0 layout under its own id
    x = synth.normal(cols, seed=43, stream=9)
    out = np.zeros(rows, np.float32)
    temp = np.full(cols, np.nan, np.float32)
    rb = synth.row_bytes(3, cols)
    assert mv.matvec_quantized(qtype, w, rows, cols, rb, x, out, temp) == 0
    nact, blocks = mv.act_bytes(qtype, cols), cols // 32
    raw = temp.view(np.uint8)
    q = raw[:nact].reshape(blocks, 34)[:, 2:].view(np.int8).astype(np.int32)
    at = (nact + 3) & ~3
    got = raw[at:at + 4 * blocks].view(np.int32)
    assert np.array_equal(got, q.sum(axis=1))
    ref = oxlibs.ref()
    if ref is not None:
        r_out = np.zeros(rows, np.float32)
        r_tmp = np.full(cols, np.nan, np.float32)
        ref.oc_matvec_quantized(qtype, w.ctypes.data, rows, cols, rb, x.ctypes.data, r_out.ctypes.data,
                                r_tmp.ctypes.data)
        assert np.array_equal(raw[:at + 4 * blocks], r_tmp.view(np.uint8)[:at + 4 * blocks])


@pytest.mark.parametrize("name,qtype", LEGACY)
def test_api_goldens_from_the_compiled_reference(oxh, name, qtype):
    g = np.load(GOLD)
    rows, cols, rb = (int(v) for v in g[name + "_api_shape"])
    w, x = g[name + "_api_w"], g[name + "_api_x"]
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(qtype, w, rows, cols, rb, x, out, temp) == 0
    a = g[name + "_api_act"]
    assert np.array_equal(temp.view(np.uint8)[:a.size], a)
    want = g[name + "_api_out"]
    assert np.all(np.abs(out - want) <= 1e-4 + 1e-5 * np.abs(want))


@pytest.mark.parametrize("name,qtype", LEGACY)
def test_block_integers_bit_exact(oxh, name, qtype):
    rows, cols = 37, 896
    w = synth.weights(qtype, rows, cols, seed=6)
    x = synth.normal(cols, seed=6)
    o = oxlibs.oracle()
    act = np.zeros(mv.act_bytes(qtype, cols), np.uint8)
    o.oxo_quantize_q8_0(x.ctypes.data, cols, act.ctypes.data)
    blocks, rb = cols // 32, synth.row_bytes(qtype, cols)
    want = np.zeros((rows, blocks), np.int32)
    fo = getattr(o, "oxo_dot_%s_q8_0" % name)
    for r in range(rows):
        fo(w[r * rb:].ctypes.data, blocks, act.ctypes.data, want[r].ctypes.data)
    d_w, d_a = mv.DeviceBuffer.from_host(w), mv.DeviceBuffer.from_host(act)
    d_s = mv.DeviceBuffer(want.nbytes)
    mv.debug_subblock_sums(qtype, d_w.ptr, rows, cols, d_a.ptr, d_s.ptr)
    assert np.array_equal(d_s.download(np.int32, want.size).reshape(want.shape), want)


@pytest.mark.parametrize("name,qtype", LEGACY)
def test_grouped_and_batched_entry_points(oxh, name, qtype):
    cols, rows = 896, [896, 128, 0, 128]
    rb = synth.row_bytes(qtype, cols)
    ws = [synth.weights(qtype, r, cols, seed=31, stream=i) if r else np.zeros(1, np.uint8)
          for i, r in enumerate(rows)]
    x = synth.normal(cols, seed=31, stream=99)
    outs = [np.full(max(r, 1), np.nan, np.float32) for r in rows]
    temp = np.zeros(cols, np.float32)
    oxh.oc_matvec_fused_test_reset()
    assert mv.matvec_quantized_fused([qtype] * len(rows), ws, rows, cols, [rb] * len(rows), x, outs, temp) == 0
    st = oxh.oc_matvec_fused_test_stats()
    assert (st.activation_quantizations, st.parallel_dispatches, st.fallback_calls) == (1, 1, 0)
    for w, r, out in zip(ws, rows, outs):
        if r:
            want, _ = oracle_matvec(qtype, w, r, cols, x)
            assert np.array_equal(bits(out[:r]), bits(want))
    # batch of 11 vectors with padded strides (more than one GEMV slice)
    n_vec, r = 11, 70
    w = synth.weights(qtype, r, cols, seed=51)
    xs = synth.normal(n_vec * (cols + 4), seed=51, stream=3).reshape(n_vec, cols + 4)
    bo = np.full((n_vec, r + 5), -7.25, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    assert mv.matvec_quantized_batch(qtype, w, r, cols, rb, xs, cols + 4, bo, r + 5, n_vec, temp, scratch) == 0
    for v in range(n_vec):
        want, _ = oracle_matvec(qtype, w, r, cols, np.ascontiguousarray(xs[v, :cols]))
        assert np.array_equal(bits(bo[v, :r]), bits(want))
        assert np.all(bo[v, r:] == -7.25)


@pytest.mark.parametrize("name,qtype", LEGACY)
def test_fused_prologue_and_paired_segments(oxh, name, qtype):
    rows, cols = 500, 1024
    wg = synth.weights(qtype, rows, cols, seed=21, stream=1)
    wu = synth.weights(qtype, rows, cols, seed=21, stream=2)
    x = (synth.normal(cols, seed=21, stream=3) * np.float32(2.0)).reshape(1, cols)
    gamma = (synth.normal(cols, seed=22) * np.float32(0.1) + np.float32(1.0)).astype(np.float32)
    d_g, d_u, d_x, d_gm = (mv.DeviceBuffer.from_host(a) for a in (wg, wu, x, gamma))
    d_h, d_y = mv.DeviceBuffer(rows * 4), mv.DeviceBuffer(cols * 4)
    segs = mv.make_segments([(d_g.ptr, d_h.ptr, rows, 0, 0, d_u.ptr)])
    mv.gemv_segments_fused(qtype, segs, cols, d_x.ptr, cols, mv.PRO_RMSNORM, d_gm.ptr, 1e-5, d_y.ptr, None, 1, rows)
    y = d_y.download(np.float32, cols)
    o = oxlibs.oracle()
    want_y = np.zeros(cols, np.float32)
    o.oxo_rms_norm_f32(x.ctypes.data, gamma.ctypes.data, want_y.ctypes.data, cols, 1e-5)
    assert np.all(np.abs(y - want_y) <= FLOAT_RTOL * np.abs(want_y))
    gate, _ = oracle_matvec(qtype, wg, rows, cols, y)
    up, _ = oracle_matvec(qtype, wu, rows, cols, y)
    want = np.zeros(rows, np.float32)
    o.oxo_swiglu_f32(gate.ctypes.data, up.ctypes.data, want.ctypes.data, rows)
    h = d_h.download(np.float32, rows)
    assert np.all(np.abs(h - want) <= FLOAT_RTOL * np.abs(want) + 1e-30)


@pytest.mark.parametrize("alias,base", [(17, 3), (19, 5), (20, 7)])
def test_alias_type_ids_run_the_base_layout(oxh, alias, base):
    """AL5 / AL6 / AL8 (oxidize-c/src/compute/quantization.c:207-214): same
    bytes, same dot, another id -- host entry point, device segments and the
    embedding lookup give the base type's bits."""
    rows, cols = 300, 896
    rb = synth.row_bytes(base, cols)
    w = synth.weights(base, rows, cols, seed=21, stream=alias)
    x = synth.normal(cols, seed=21, stream=alias + 50)
    outs = []
    for t in (alias, base):
        out, temp = np.zeros(rows, np.float32), np.zeros(cols, np.float32)
        assert mv.matvec_quantized(t, w, rows, cols, rb, x, out, temp) == 0
        outs.append((out, temp.copy()))
    assert np.array_equal(bits(outs[0][0]), bits(outs[1][0]))
    assert np.array_equal(outs[0][1].view(np.uint8), outs[1][1].view(np.uint8))
    o = oxlibs.oracle()
    want, t2 = np.zeros(rows, np.float32), np.zeros(cols, np.float32)
    assert o.oxo_matvec_quantized(alias, w.ctypes.data, rows, cols, rb, x.ctypes.data, want.ctypes.data,
                                  t2.ctypes.data) == 0
    assert np.array_equal(bits(outs[0][0]), bits(want))
    d_w = mv.DeviceBuffer.from_host(w)
    ids = np.array([0, rows - 1, 7], np.uint32)
    d_ids = mv.DeviceBuffer.from_host(ids)
    d_o = mv.DeviceBuffer(ids.size * cols * 4)
    mv.get_rows(alias, d_w.ptr, rows, cols, d_ids.ptr, ids.size, d_o.ptr, cols)
    got = d_o.download(np.float32, ids.size * cols).reshape(ids.size, cols)
    for k, i in enumerate(ids):
        deq = np.zeros(cols, np.float32)
        assert o.oxo_dequant_row(alias, w[int(i) * rb:].ctypes.data, cols, deq.ctypes.data) == 0
        assert np.array_equal(bits(got[k]), bits(deq))


@pytest.mark.parametrize("name,qtype", (("q8_0", 7), ("q4_0", 3), ("q5_0", 5), ("al5_xs", 18)))
@pytest.mark.parametrize("cols", [32, 96, 416])
def test_segment_that_starts_two_bytes_past_a_multiple_of_four(oxh, name, qtype, cols):
    """Rows of an odd number of these blocks are 2 (mod 4) bytes long, so a segment that starts at an odd
    row has every other block, the first one included, two bytes past a multiple of four; the kernels
    fetch such a block from the multiple of four ahead of it or behind its first two bytes (inside the
    matrix either way).  Rows 1.. and 3.. of a matrix as segments of their own, one and three activations."""
    rows = 9
    rb = synth.row_bytes(qtype, cols)
    assert rb % 4 == 2
    w = synth.weights(qtype, rows, cols, seed=61, stream=cols)
    d_w = mv.DeviceBuffer.from_host(w)
    for nv in (1, 3):
        xs = synth.normal(nv * cols, seed=62, stream=nv).reshape(nv, cols)
        d_x = mv.DeviceBuffer.from_host(xs)
        d_o = mv.DeviceBuffer(2 * nv * rows * 4)
        first = [(1, rows - 1), (3, rows - 3)]
        segs = mv.make_segments([(d_w.ptr + r0 * rb, d_o.ptr + k * nv * rows * 4, n, 0)
                                 for k, (r0, n) in enumerate(first)])
        mv.gemv_segments_f32(qtype, segs, cols, d_x.ptr, cols, None, nv, rows)
        got = d_o.download(np.float32, 2 * nv * rows).reshape(2, nv, rows)
        for v in range(nv):
            want, _ = oracle_matvec(qtype, w, rows, cols, xs[v])
            for k, (r0, n) in enumerate(first):
                assert np.array_equal(bits(got[k, v, :n]), bits(want[r0:r0 + n])), (name, cols, nv, k)
        d_x.free()
        d_o.free()
    d_w.free()
