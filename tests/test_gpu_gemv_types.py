"""GPU parity for the Q6_K and Q8_0 decode GEMVs, the Q8_0 activation
quantiser and the grouped entry points (fused / multi-input / batch), through
the C ABI, against the CPU oracle.

Bars: activation bytes and integer sub-block sums bit-exact for every type;
f32 outputs bit-exact for Q4_K and Q6_K; Q8_0 f32 outputs bit-exact against the
oracle's block-sequential chain and within |a-b| <= 1e-4 + 1e-5*|ref| of the
compiled reference (whose x86 decode kernel sums the same terms in f32 lanes).
"""
import numpy as np
import pytest

import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth

pytestmark = pytest.mark.gpu

Q80, Q4K, Q6K = 7, 13, 16


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


@pytest.mark.parametrize("cols", [32, 896, 4864, 4096])
def test_quantize_q8_0_bytes_bit_exact(oxh, cols):
    n_vec = 3
    x = synth.normal(n_vec * cols, seed=4, stream=cols).reshape(n_vec, cols)
    x[1, :32] = 0.0
    x[2, :32] *= 1e-7          # f16 scale lands in the subnormal range
    x[0, :32] *= 3e4           # large scale
    nbytes = mv.act_bytes(Q80, cols)
    d_x = mv.DeviceBuffer.from_host(x)
    d_a = mv.DeviceBuffer(n_vec * nbytes)
    mv.quantize(Q80, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    got = d_a.download(np.uint8, n_vec * nbytes).reshape(n_vec, nbytes)
    o = oxlibs.oracle()
    for v in range(n_vec):
        want = np.zeros(nbytes, np.uint8)
        o.oxo_quantize_q8_0(x[v].ctypes.data, cols, want.ctypes.data)
        assert np.array_equal(got[v], want), "vector %d" % v


@pytest.mark.parametrize("qtype,rows,cols", [
    (Q6K, 1, 256), (Q6K, 9, 768), (Q6K, 100, 14336), (Q6K, 257, 4096), (Q6K, 33, 2816),
    (Q80, 1, 32), (Q80, 5, 96), (Q80, 1000, 896), (Q80, 300, 4864), (Q80, 77, 4096),
])
def test_matvec_quantized_bits(oxh, qtype, rows, cols):
    w = synth.weights(qtype, rows, cols, seed=21, stream=rows)
    x = synth.normal(cols, seed=21, stream=9)
    out = np.full(rows, np.nan, np.float32)
    temp = np.zeros(cols, np.float32)
    rc = mv.matvec_quantized(qtype, w, rows, cols, synth.row_bytes(qtype, cols), x, out, temp)
    assert rc == 0
    want, want_temp = oracle_matvec(qtype, w, rows, cols, x)
    nact = mv.act_bytes(qtype, cols)
    assert np.array_equal(temp.view(np.uint8)[:nact], want_temp.view(np.uint8)[:nact])
    assert np.array_equal(bits(out), bits(want))
    ref = oxlibs.ref()
    if ref is not None:
        r_out = np.zeros(rows, np.float32)
        r_tmp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qtype, w.ctypes.data, rows, cols, synth.row_bytes(qtype, cols),
                                x.ctypes.data, r_out.ctypes.data, r_tmp.ctypes.data)
        assert np.array_equal(temp.view(np.uint8)[:nact], r_tmp.view(np.uint8)[:nact])
        if qtype == Q80:
            assert np.all(np.abs(out - r_out) <= 1e-4 + 1e-5 * np.abs(r_out))
        else:
            assert np.array_equal(bits(out), bits(r_out))


@pytest.mark.parametrize("qtype,cols,per_block", [(Q6K, 4096, 16), (Q80, 896, 1)])
def test_subblock_sums_bit_exact(oxh, qtype, cols, per_block):
    rows = 37
    w = synth.weights(qtype, rows, cols, seed=6)
    x = synth.normal(cols, seed=6)
    o = oxlibs.oracle()
    nact = mv.act_bytes(qtype, cols)
    act = np.zeros(nact, np.uint8)
    blocks = cols // synth.BLOCK_ELEMS[qtype]
    rb = synth.row_bytes(qtype, cols)
    want = np.zeros((rows, blocks, per_block), np.int32)
    if qtype == Q6K:
        o.oxo_quantize_q8_k(x.ctypes.data, cols, act.ctypes.data)
        for r in range(rows):
            o.oxo_dot_q6_k_q8_k(w[r * rb:].ctypes.data, blocks, act.ctypes.data, want[r].ctypes.data)
    else:
        o.oxo_quantize_q8_0(x.ctypes.data, cols, act.ctypes.data)
        for r in range(rows):
            o.oxo_dot_q8_0_q8_0(w[r * rb:].ctypes.data, blocks, act.ctypes.data, want[r].ctypes.data)
    d_w = mv.DeviceBuffer.from_host(w)
    d_a = mv.DeviceBuffer.from_host(act)
    d_s = mv.DeviceBuffer(want.nbytes)
    mv.debug_subblock_sums(qtype, d_w.ptr, rows, cols, d_a.ptr, d_s.ptr)
    got = d_s.download(np.int32, want.size).reshape(want.shape)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("qtype,cols,rows", [(Q4K, 4096, [4096, 1024, 1024]),
                                             (Q4K, 2048, [300, 0, 5]),
                                             (Q6K, 1024, [64, 64]),
                                             (Q80, 896, [896, 128, 128])])
def test_fused_equals_separate(oxh, qtype, cols, rows):
    """oc_matvec_quantized_fused: bit-identical to one call per matrix, one
    activation quantisation and one dispatch (tests/test_matvec_fused.c:88-136)."""
    rb = synth.row_bytes(qtype, cols)
    ws = [synth.weights(qtype, r, cols, seed=31, stream=i) if r else np.zeros(1, np.uint8)
          for i, r in enumerate(rows)]
    x = synth.normal(cols, seed=31, stream=99)
    outs = [np.full(max(r, 1), np.nan, np.float32) for r in rows]
    temp = np.zeros(cols, np.float32)
    oxh.oc_matvec_fused_test_reset()
    rc = mv.matvec_quantized_fused([qtype] * len(rows), ws, rows, cols, [rb] * len(rows), x, outs, temp)
    assert rc == 0
    st = oxh.oc_matvec_fused_test_stats()
    assert (st.activation_quantizations, st.parallel_dispatches, st.fallback_calls) == (1, 1, 0)
    for w, r, out in zip(ws, rows, outs):
        if r == 0:
            continue
        want, _ = oracle_matvec(qtype, w, r, cols, x)
        assert np.array_equal(bits(out[:r]), bits(want))


def test_fused_mixed_types_falls_back_per_matrix(oxh):
    cols = 1024
    rows = [40, 24]
    qts = [Q4K, Q6K]
    ws = [synth.weights(q, r, cols, seed=32, stream=i) for i, (q, r) in enumerate(zip(qts, rows))]
    x = synth.normal(cols, seed=32)
    outs = [np.zeros(r, np.float32) for r in rows]
    temp = np.zeros(cols, np.float32)
    oxh.oc_matvec_fused_test_reset()
    rc = mv.matvec_quantized_fused(qts, ws, rows, cols, [synth.row_bytes(q, cols) for q in qts],
                                   x, outs, temp)
    assert rc == 0
    st = oxh.oc_matvec_fused_test_stats()
    assert (st.activation_quantizations, st.parallel_dispatches, st.fallback_calls) == (2, 2, 2)
    for q, w, r, out in zip(qts, ws, rows, outs):
        want, _ = oracle_matvec(q, w, r, cols, x)
        assert np.array_equal(bits(out), bits(want))


@pytest.mark.parametrize("qtype,cols,rows", [(Q4K, 14336, [4096, 4096]), (Q4K, 768, [3, 17, 1, 40]),
                                             (Q6K, 512, [10, 20]), (Q80, 64, [5, 6, 7])])
def test_multi_input_equals_separate(oxh, qtype, cols, rows):
    rb = synth.row_bytes(qtype, cols)
    ws = [synth.weights(qtype, r, cols, seed=41, stream=i) for i, r in enumerate(rows)]
    xs = [synth.normal(cols, seed=41, stream=200 + i) for i in range(len(rows))]
    outs = [np.full(r, np.nan, np.float32) for r in rows]
    temp = np.zeros(cols, np.float32)
    oxh.oc_matvec_fused_test_reset()
    rc = mv.matvec_quantized_multi_input([qtype] * len(rows), ws, rows, cols, [rb] * len(rows),
                                         xs, outs, temp)
    assert rc == 0
    st = oxh.oc_matvec_fused_test_stats()
    assert (st.activation_quantizations, st.parallel_dispatches, st.fallback_calls) == (len(rows), 1, 0)
    for w, r, x, out in zip(ws, rows, xs, outs):
        want, _ = oracle_matvec(qtype, w, r, cols, x)
        assert np.array_equal(bits(out), bits(want))


@pytest.mark.parametrize("qtype,rows,cols,n_vec,in_pad,out_pad", [
    (Q4K, 96, 1024, 1, 0, 0), (Q4K, 96, 1024, 5, 3, 7), (Q4K, 64, 14336, 8, 0, 0),
    (Q6K, 50, 512, 3, 16, 1), (Q80, 70, 896, 8, 0, 5), (Q80, 70, 896, 2, 4, 0),
    (Q4K, 40, 512, 13, 0, 3), (Q6K, 24, 768, 11, 0, 0),
])
def test_batch_equals_single(oxh, qtype, rows, cols, n_vec, in_pad, out_pad):
    """oc_matvec_quantized_batch: every output equals the single-vector call;
    padded strides honoured and the padding left untouched
    (tests/test_matvec_batch.c:86-99, :188-234)."""
    in_stride, out_stride = cols + in_pad, rows + out_pad
    w = synth.weights(qtype, rows, cols, seed=51)
    xs = synth.normal(n_vec * in_stride, seed=51, stream=3).reshape(n_vec, in_stride)
    outs = np.full((n_vec, out_stride), -7.25, np.float32)
    temp = np.zeros(cols, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    rc = mv.matvec_quantized_batch(qtype, w, rows, cols, synth.row_bytes(qtype, cols), xs,
                                   in_stride, outs, out_stride, n_vec, temp, scratch)
    assert rc == 0
    for v in range(n_vec):
        want, _ = oracle_matvec(qtype, w, rows, cols, np.ascontiguousarray(xs[v, :cols]))
        assert np.array_equal(bits(outs[v, :rows]), bits(want)), "vector %d" % v
        assert np.all(outs[v, rows:] == -7.25)


def test_declines_like_the_reference(oxh):
    """Shapes the reference's integer path refuses come back OXH_DECLINED with
    the outputs untouched (matvec.c:99-127, :961-985, :1290-1292)."""
    out = np.full(8, 3.5, np.float32)
    temp = np.zeros(4096, np.float32)
    x = synth.normal(4096, seed=1)
    w = synth.weights(Q4K, 8, 4096, seed=1)
    rb = synth.row_bytes(Q4K, 4096)
    # K-quant with cols not a multiple of 256 (e.g. n_embd = 896)
    assert mv.matvec_quantized(Q4K, w, 8, 896, 504, x, out, temp) == mv.DECLINED
    # padded row stride
    assert mv.matvec_quantized(Q4K, w, 4, 4096, rb + 16, x, out, temp) == mv.DECLINED
    # a type with no kernel here (F16 = 1)
    assert mv.matvec_quantized(1, w, 8, 4096, 8192, x, out, temp) == mv.DECLINED
    # global switch off
    oxh.oc_matvec_set_fused(False)
    try:
        assert mv.matvec_quantized(Q4K, w, 8, 4096, rb, x, out, temp) == mv.DECLINED
    finally:
        oxh.oc_matvec_set_fused(True)
    # batch without scratch / with scratch smaller than one activation
    outs = np.full((2, 8), 3.5, np.float32)
    xs = np.stack([x, x])
    assert mv.matvec_quantized_batch(Q4K, w, 8, 4096, rb, xs, 4096, outs, 8, 2, temp, None) == mv.DECLINED
    small = np.zeros(100, np.uint8)
    assert mv.matvec_quantized_batch(Q4K, w, 8, 4096, rb, xs, 4096, outs, 8, 2, temp, small) == mv.DECLINED
    assert np.all(out == 3.5) and np.all(outs == 3.5)
    # and the same call with everything in order is handled
    assert mv.matvec_quantized(Q4K, w, 8, 4096, rb, x, out, temp) == mv.OK


def test_empty_inputs_are_no_ops(oxh):
    x = synth.normal(256, seed=1)
    w = synth.weights(Q4K, 1, 256, seed=1)
    out = np.full(4, 1.5, np.float32)
    temp = np.zeros(256, np.float32)
    assert mv.matvec_quantized(Q4K, w, 0, 256, 144, x, out, temp) == mv.OK
    assert mv.matvec_quantized_fused([], [], [], 256, [], x, [], temp) == mv.OK
    scratch = np.zeros(4096, np.uint8)
    assert mv.matvec_quantized_batch(Q4K, w, 1, 256, 144, x, 256, out, 1, 0, temp, scratch) == mv.OK
    assert np.all(out == 1.5)


def test_expert_slices_resolve_inside_a_registered_tensor(oxh):
    """A stacked expert tensor registered once; calls pass slice pointers
    (llama.c:4248-4251 stacks expert e at rows [e*rows, (e+1)*rows))."""
    n_exp, rows, cols = 4, 48, 1024
    rb = synth.row_bytes(Q4K, cols)
    w = synth.weights(Q4K, n_exp * rows, cols, seed=61)
    from oxidize_amd import _lib
    _lib.check(oxh.oxh_weight_register(w.ctypes.data, w.nbytes))
    base = oxh.oxh_weight_device_ptr(w.ctypes.data)
    x = synth.normal(cols, seed=61)
    temp = np.zeros(cols, np.float32)
    for e in (2, 0, 3):
        sl = w[e * rows * rb:(e + 1) * rows * rb]
        assert oxh.oxh_weight_device_ptr(sl.ctypes.data) == base + e * rows * rb
        out = np.zeros(rows, np.float32)
        assert mv.matvec_quantized(Q4K, sl, rows, cols, rb, x, out, temp) == mv.OK
        want, _ = oracle_matvec(Q4K, np.ascontiguousarray(sl), rows, cols, x)
        assert np.array_equal(bits(out), bits(want))
    # registered ranges are the caller's promise that the bytes stay put: give it back before w is freed
    assert oxh.oxh_weight_unregister(w.ctypes.data) == 0
    assert oxh.oxh_weight_device_ptr(w.ctypes.data) is None


@pytest.mark.parametrize("qtype", [Q4K, Q6K])
@pytest.mark.parametrize("rows,cols,n_vec,out_pad", [
    (32, 256, 32, 0), (130, 1024, 9, 0), (128, 4096, 64, 0), (200, 2816, 100, 5),
    (257, 512, 65, 1), (64, 14336, 40, 0),
])
def test_mmq_batch_bit_identical_to_single_vector(oxh, qtype, rows, cols, n_vec, out_pad):
    """More than 8 vectors of Q4_K or Q6_K go through the int8-MFMA kernels;
    the reference promises batch == single-vector to the bit for K-quants
    (matvec.h:115-117, tests/test_matvec_batch.c:86-99)."""
    Q4K_ = qtype
    out_stride = rows + out_pad
    w = synth.weights(Q4K_, rows, cols, seed=71, stream=rows)
    xs = synth.normal(n_vec * cols, seed=71, stream=n_vec).reshape(n_vec, cols)
    xs[3, :256] = 0.0
    outs = np.full((n_vec, out_stride), -7.25, np.float32)
    temp = np.zeros(cols, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    rc = mv.matvec_quantized_batch(qtype, w, rows, cols, synth.row_bytes(qtype, cols), xs, cols, outs,
                                   out_stride, n_vec, temp, scratch)
    assert rc == 0
    o = oxlibs.oracle()
    want = np.zeros((n_vec, rows), np.float32)
    sc2 = np.zeros(o.oxo_matvec_batch_scratch_bytes(cols), np.uint8)
    assert o.oxo_matvec_quantized_batch(qtype, w.ctypes.data, rows, cols, synth.row_bytes(qtype, cols),
                                        xs.ctypes.data, cols, want.ctypes.data, rows, n_vec,
                                        sc2.ctypes.data, sc2.nbytes) == 0
    assert np.array_equal(bits(outs[:, :rows]), bits(want))
    assert np.all(outs[:, rows:] == -7.25)


@pytest.mark.parametrize("qtype,cols,d_off", [(Q4K, 1024, 0), (Q6K, 1024, 208), (Q80, 256, 0)])
def test_subnormal_and_extreme_f16_weight_scales(oxh, qtype, cols, d_off):
    """f16 block scales in the subnormal range, at the largest finite value and
    negative: the f16 -> f32 step must be exact for every bit pattern."""
    rows = 64
    w = synth.weights(qtype, rows, cols, seed=81)
    bsz = synth.BLOCK_BYTES[qtype]
    blk = w.reshape(-1, bsz)
    pats = np.array([0x0001, 0x0002, 0x03FF, 0x0400, 0x7BFF, 0x8001, 0x83FF, 0xBC00, 0x0000, 0x8000,
                     0x0155, 0x3555], np.uint16)
    sel = pats[np.arange(blk.shape[0]) % pats.size]
    blk[:, d_off] = sel & 0xFF
    blk[:, d_off + 1] = sel >> 8
    if qtype == Q4K:
        sel2 = pats[(np.arange(blk.shape[0]) * 5 + 3) % pats.size]
        blk[:, 2] = sel2 & 0xFF
        blk[:, 3] = sel2 >> 8
    x = synth.normal(cols, seed=81)
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(qtype, w, rows, cols, synth.row_bytes(qtype, cols), x, out, temp) == 0
    want, _ = oracle_matvec(qtype, w, rows, cols, x)
    assert np.array_equal(bits(out), bits(want))


@pytest.mark.parametrize("qtype,rows,cols,n_vec", [(Q4K, 100, 4096, 1), (Q6K, 60, 2048, 3), (Q80, 90, 896, 8)])
def test_prequantised_and_fused_paths_agree(oxh, qtype, rows, cols, n_vec):
    """Layer 2: quantiser kernel + GEMV over stored Q8 bytes gives the same
    outputs and the same activation bytes as the single fused launch."""
    w = synth.weights(qtype, rows, cols, seed=91)
    xs = synth.normal(n_vec * cols, seed=91).reshape(n_vec, cols)
    d_w = mv.DeviceBuffer.from_host(w)
    d_x = mv.DeviceBuffer.from_host(xs)
    nact = mv.act_bytes(qtype, cols)
    d_a1, d_a2 = mv.DeviceBuffer(n_vec * nact), mv.DeviceBuffer(n_vec * nact)
    d_o1, d_o2 = mv.DeviceBuffer(n_vec * rows * 4), mv.DeviceBuffer(n_vec * rows * 4)
    mv.quantize(qtype, d_x.ptr, cols, n_vec, cols, d_a1.ptr)
    mv.gemv_segments(qtype, mv.make_segments([(d_w.ptr, d_o1.ptr, rows, 0)]), cols, d_a1.ptr, n_vec, rows)
    mv.gemv_segments_f32(qtype, mv.make_segments([(d_w.ptr, d_o2.ptr, rows, 0)]), cols, d_x.ptr, cols,
                         d_a2.ptr, n_vec, rows)
    a1 = d_a1.download(np.uint8, n_vec * nact)
    a2 = d_a2.download(np.uint8, n_vec * nact)
    o1 = d_o1.download(np.float32, n_vec * rows)
    o2 = d_o2.download(np.float32, n_vec * rows)
    assert np.array_equal(a1, a2)
    assert np.array_equal(bits(o1), bits(o2))
    o = oxlibs.oracle()
    for v in range(n_vec):
        want, _ = oracle_matvec(qtype, w, rows, cols, np.ascontiguousarray(xs[v]))
        assert np.array_equal(bits(o1[v * rows:(v + 1) * rows]), bits(want))


@pytest.mark.parametrize("qtype,rows,cols", [(Q4K, 1000, 4096), (15, 300, 1024), (Q6K, 500, 2816), (Q80, 2000, 896),
                                             (Q80, 64, 32), (Q4K, 7, 256), (3, 300, 896), (4, 300, 896),
                                             (5, 300, 896), (6, 300, 896), (5, 9, 32), (6, 9, 1056), (18, 200, 896),
                                             (18, 3, 32)])
def test_embedding_rows_bit_identical_to_the_cpu_dequantisation(oxh, qtype, rows, cols):
    """oxh_get_rows against the oracle's dequantisation (itself bit-identical
    to the compiled reference's oc_quant_dequant_row): ids on the device, first
    and last row, repeats, padded output stride, and an id beyond the matrix,
    which must give zeros."""
    w = synth.weights(qtype, rows, cols, seed=33, stream=rows)
    rb = synth.row_bytes(qtype, cols)
    ids = np.array([0, rows - 1, rows // 2, 0, rows, 0xFFFFFFFF, 1 % rows], np.uint32)
    stride = cols + 8
    d_w = mv.DeviceBuffer.from_host(w)
    d_ids = mv.DeviceBuffer.from_host(ids)
    d_o = mv.DeviceBuffer(ids.size * stride * 4)
    d_o.upload(np.full(ids.size * stride, -7.25, np.float32))
    mv.get_rows(qtype, d_w.ptr, rows, cols, d_ids.ptr, ids.size, d_o.ptr, stride)
    got = d_o.download(np.float32, ids.size * stride).reshape(ids.size, stride)
    o = oxlibs.oracle()
    for t, i in enumerate(ids):
        want = np.zeros(cols, np.float32)
        if i < rows:
            assert o.oxo_dequant_row(qtype, w[int(i) * rb:].ctypes.data, cols, want.ctypes.data) == 0
        assert np.array_equal(bits(got[t, :cols]), bits(want)), "id %d" % i
    assert np.all(got[:, cols:] == -7.25)
    # a type without a kernel here declines
    with pytest.raises(mv.OxhError) as e:
        mv.get_rows(1, d_w.ptr, rows, cols, d_ids.ptr, ids.size, d_o.ptr, stride)
    assert e.value.status == mv.DECLINED


@pytest.mark.parametrize("fmt", [Q80, 3, 4, 5, 6, 18])
@pytest.mark.parametrize("rows,cols,nvs", [(151, 896, (5, 8)), (64, 32, (8,)), (1000, 4864, (6, 8)), (33, 2048, (7, 5)),
                                           (4864, 896, (8, 8, 5)), (70, 2336, (16, 9)), (20, 64, (12,))])
def test_q8_0_small_batches_on_the_matrix_cores(oxh, fmt, rows, cols, nvs):
    """Launches over a 32-value format with five or more activations per weight and a buffer for
    their quantised form run on the int8 MFMA kernel: per-block integers exact,
    f32 the block-sequential chain, so every output carries the oracle's bits.
    One segment per entry of `nvs`, each with its own run of activations and
    its own count; ragged rows; the same launch with fewer than five
    activations (dot-instruction kernel) as a cross-check of the segment logic."""
    rb = synth.row_bytes(fmt, cols)
    n_act = sum(nvs)
    ws = [synth.weights(fmt, rows, cols, seed=71, stream=i) for i in range(len(nvs))]
    xs = synth.normal(n_act * cols, seed=71, stream=9).reshape(n_act, cols)
    d_ws = [mv.DeviceBuffer.from_host(w) for w in ws]
    d_x = mv.DeviceBuffer.from_host(xs)
    d_act = mv.DeviceBuffer(n_act * mv.act_bytes(fmt, cols))
    d_out = mv.DeviceBuffer(n_act * rows * 4)
    d_out.upload(np.full(n_act * rows, np.nan, np.float32))
    items, first = [], 0
    for d_w, nv in zip(d_ws, nvs):
        items.append((d_w.ptr, d_out.ptr + first * rows * 4, rows, first, nv))
        first += nv
    mv.gemv_segments_f32(fmt, mv.make_segments(items), cols, d_x.ptr, cols, d_act.ptr, max(nvs), rows)
    mv.sync()
    got = d_out.download(np.float32, n_act * rows).reshape(n_act, rows)
    o = oxlibs.oracle()
    acts = d_act.download(np.uint8, n_act * mv.act_bytes(fmt, cols)).reshape(n_act, -1)
    first = 0
    for w, nv in zip(ws, nvs):
        for v in range(first, first + nv):
            want, temp = oracle_matvec(fmt, w, rows, cols, np.ascontiguousarray(xs[v]))
            assert np.array_equal(acts[v], temp.view(np.uint8)[:acts.shape[1]])
            assert np.array_equal(bits(got[v]), bits(want)), (nv, v)
        first += nv
    assert rb * rows == ws[0].nbytes


@pytest.mark.parametrize("qtype,size", [(Q4K, 144), (15, 176), (Q6K, 210), (Q80, 34), (8, 84), (10, 110), (3, 18),
                                        (4, 20), (5, 22), (6, 24), (18, 14)])
def test_every_weight_byte_influences_its_row(oxh, qtype, size):
    """oxidize-c/tests/test_quant.c:569-583 as a kernel test: one row per byte of
    a block, that byte altered; every row must differ from the unaltered one
    (no byte of any layout is ignored or read from the wrong place) and carry
    the oracle's bits."""
    group = 256 if size > 34 else 32
    base = synth.weights(qtype, 1, group, seed=13, stream=qtype)
    masks = (0x15, 0x6A)             # two alterations per byte: an integer change can cancel by chance
    w = np.tile(base, 2 * size + 1).reshape(2 * size + 1, size)
    for i in range(size):
        for m, mask in enumerate(masks):
            w[1 + 2 * i + m, i] ^= mask
    w = np.ascontiguousarray(w.ravel())
    x = (synth.normal(group, seed=13, stream=1) ** 2 + 0.25).astype(np.float32)      # all positive
    rows = 2 * size + 1
    out = np.zeros(rows, np.float32)
    temp = np.zeros(group, np.float32)
    assert mv.matvec_quantized(qtype, w, rows, group, size, x, out, temp) == 0
    want, _ = oracle_matvec(qtype, w, rows, group, x)
    assert np.array_equal(bits(out), bits(want))
    ob = bits(out)
    same = [i for i in range(size) if ob[1 + 2 * i] == ob[0] and ob[2 + 2 * i] == ob[0]]
    assert not same, "bytes without influence: %s" % same


@pytest.mark.parametrize("qtype,cols,n_vec", [(Q80, 896, 600), (Q80, 4096, 33), (25, 512, 300), (3, 1024, 530)])
def test_long_batches_of_types_without_a_tile_kernel(oxh, qtype, cols, n_vec):
    """Batches over the 32-value and codebook formats run as slices of a few activations, up to 32 slices
    per launch: lengths that need several launches, a last launch with one slice, a ragged last slice."""
    rows = 70
    rb = synth.row_bytes(qtype, cols)
    w = synth.weights(qtype, rows, cols, seed=61, stream=cols)
    xs = synth.normal(n_vec * (cols + 8), seed=61, stream=n_vec).reshape(n_vec, cols + 8)
    outs = np.full((n_vec, rows + 3), -7.25, np.float32)
    temp = np.zeros(cols, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    assert mv.matvec_quantized_batch(qtype, w, rows, cols, rb, xs, cols + 8, outs, rows + 3, n_vec, temp, scratch) == 0
    assert np.all(outs[:, rows:] == -7.25)
    for v in list(range(0, n_vec, 37)) + [n_vec - 1]:
        want, _ = oracle_matvec(qtype, w, rows, cols, np.ascontiguousarray(xs[v, :cols]))
        assert np.array_equal(bits(outs[v, :rows]), bits(want)), v


@pytest.mark.parametrize("qtype,rows,cols,n_vec", [
    (Q80, 70, 896, 600),        # 28 blocks: a full step and a short one; ragged row and token tiles
    (Q80, 130, 4096, 65),       # a second row tile of two rows, a second token tile of one token
    (Q80, 16, 32, 64),          # one block per row
    (3, 257, 1024, 64),         # Q4_0
    (4, 128, 544, 100),         # Q4_1, 17 blocks: the last step is a single block
    (5, 17, 992, 33),           # Q5_0, 31 blocks: an odd last step
    (6, 300, 2048, 129),        # Q5_1
    (18, 129, 1056, 70),        # AL5_XS, 33 blocks of 14 bytes: a last step shorter than one 16-byte piece
    (20, 64, 512, 17),          # AL8: the Q8_0 layout under its own id
])
def test_token_tiled_kernel_of_the_32_value_formats(oxh, qtype, rows, cols, n_vec):
    """oxh_mmq over the 32-value formats (128 rows x 64 tokens per workgroup, activations staged sixteen
    blocks at a time): every output is the single-vector dot, bit for bit, and nothing outside the
    rows x n_vec outputs is written."""
    canon = {17: 3, 19: 5, 20: 7}.get(qtype, qtype)
    w = synth.weights(canon, rows, cols, seed=83, stream=rows + cols)
    xs = synth.normal(n_vec * cols, seed=83, stream=n_vec).reshape(n_vec, cols)
    xs[n_vec // 2, :64] = 0.0
    d_w = mv.DeviceBuffer.from_host(w)
    d_x = mv.DeviceBuffer.from_host(xs)
    d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(qtype, cols))
    mv.quantize(qtype, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    stride = rows + 3
    d_out = mv.DeviceBuffer.from_host(np.full((n_vec, stride), -7.25, np.float32))
    assert mv.mmq_tile(qtype, rows, n_vec, 256) == (128, 64)
    mv.mmq(qtype, d_w.ptr, rows, cols, d_a.ptr, n_vec, d_out.ptr, stride)
    mv.sync()
    outs = d_out.download(np.float32, n_vec * stride).reshape(n_vec, stride)
    assert np.all(outs[:, rows:] == -7.25)
    for v in sorted(set(list(range(0, n_vec, 13)) + [n_vec // 2, 63 % n_vec, 64 % n_vec, n_vec - 1])):
        want, _ = oracle_matvec(canon, w, rows, cols, np.ascontiguousarray(xs[v]))
        assert np.array_equal(bits(outs[v, :rows]), bits(want)), v


@pytest.mark.parametrize("qtype,rows,cols,n_vec", [(Q4K, 40, 512, 3), (Q80, 33, 256, 1), (Q6K, 70, 256, 8)])
def test_a_call_with_more_than_32_segments_runs_as_launches_of_32(oxh, qtype, rows, cols, n_vec):
    """Seventy segments, each its own matrix and run of activations, in one call: the bits of the same
    segments in calls of at most 32, over quantised activations and over f32 inputs with a buffer for the
    quantised bytes; f32 inputs without one are refused."""
    from oxidize_amd import _lib
    n_seg = 70
    rb = synth.row_bytes(qtype, cols)
    w = synth.weights(qtype, n_seg * rows, cols, seed=97)
    d_w = mv.DeviceBuffer.from_host(w)
    n_act = n_seg * n_vec
    d_x = mv.DeviceBuffer.from_host(synth.normal(n_act * cols, seed=97, stream=1))
    nact = mv.act_bytes(qtype, cols)
    a_ref, a_all = mv.DeviceBuffer(n_act * nact), mv.DeviceBuffer(n_act * nact)
    outs = [mv.DeviceBuffer(n_act * rows * 4) for _ in range(3)]
    for o in outs:
        o.upload(np.full(n_act * rows, np.float32(-3.0)))

    def items(o):
        return [(d_w.ptr + s * rows * rb, o.ptr + s * n_vec * rows * 4, rows, s * n_vec, n_vec) for s in range(n_seg)]

    mv.quantize(qtype, d_x.ptr, cols, n_act, cols, a_ref.ptr)
    it = items(outs[0])
    for k in range(0, n_seg, 32):
        mv.gemv_segments(qtype, mv.make_segments(it[k:k + 32]), cols, a_ref.ptr, 1, rows)
    mv.gemv_segments(qtype, mv.make_segments(items(outs[1])), cols, a_ref.ptr, 1, rows)
    mv.gemv_segments_f32(qtype, mv.make_segments(items(outs[2])), cols, d_x.ptr, cols, a_all.ptr, 1, rows)
    mv.sync()
    want = outs[0].download(np.float32, n_act * rows)
    assert not np.any(want == np.float32(-3.0))
    assert np.array_equal(bits(outs[1].download(np.float32, n_act * rows)), bits(want))
    assert np.array_equal(bits(outs[2].download(np.float32, n_act * rows)), bits(want))
    assert np.array_equal(a_all.download(np.uint8, n_act * nact), a_ref.download(np.uint8, n_act * nact))
    with pytest.raises(mv.OxhError) as e:
        mv.gemv_segments_f32(qtype, mv.make_segments(items(outs[2])), cols, d_x.ptr, cols, None, 1, rows)
    assert e.value.status == _lib.ERR_ARG
