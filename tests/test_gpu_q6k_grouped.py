"""Q6_K regrouped in runs of eight blocks (oxh_q6_k_group, OXH_Q6_K_G8): the decode kernels must give the
bits of the file layout, which other tests hold to the oracle; the permutation itself is checked against a
numpy statement of the layout the header documents; the host layer must use the regrouped copy without a
caller noticing anything but the time."""
import ctypes

import numpy as np
import pytest

import oxlibs
from oxidize_amd import _lib, synth
from oxidize_amd import matvec as mv

pytestmark = pytest.mark.gpu
Q4K, Q6K, G8 = 13, 16, mv.Q6_K_G8


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def regroup(w, n_blocks):
    """The documented layout: per eight blocks, pieces la / lb / hh of (block j, lane u) at 16*(4j+u) in
    three 512-byte planes, then the scales of block j at 1536 + 16j and its d at 1664 + 2j."""
    b = w.reshape(n_blocks // 8, 8, 210)
    out = np.zeros((n_blocks // 8, 1680), np.uint8)
    for j in range(8):
        for u in range(4):
            n, lh = u >> 1, u & 1
            at = 16 * (4 * j + u)
            out[:, at:at + 16] = b[:, j, 64 * n + 16 * lh:64 * n + 16 * lh + 16]
            out[:, 512 + at:528 + at] = b[:, j, 64 * n + 32 + 16 * lh:64 * n + 48 + 16 * lh]
            out[:, 1024 + at:1040 + at] = b[:, j, 128 + 32 * n + 16 * lh:144 + 32 * n + 16 * lh]
        out[:, 1536 + 16 * j:1552 + 16 * j] = b[:, j, 192:208]
        out[:, 1664 + 2 * j:1666 + 2 * j] = b[:, j, 208:210]
    return out.reshape(-1)


def grouped_copy(w, rows, cols):
    d_w = mv.DeviceBuffer.from_host(w)
    d_g = mv.DeviceBuffer(w.nbytes)
    mv.q6_k_group(d_w.ptr, rows, cols, d_g.ptr)
    mv.sync()
    return d_w, d_g


@pytest.mark.parametrize("rows,cols", [(1, 2048), (7, 4096), (333, 14336), (4096, 2048)])
def test_regrouping_is_the_documented_permutation(oxh, rows, cols):
    w = synth.weights(Q6K, rows, cols, seed=31, stream=rows)
    d_w, d_g = grouped_copy(w, rows, cols)
    got = d_g.download(np.uint8, w.nbytes)
    assert np.array_equal(got, regroup(w, rows * cols // 256))
    assert np.array_equal(np.sort(got), np.sort(w))          # the same bytes


@pytest.mark.parametrize("rows,cols,n_vec", [(1, 2048, 1), (100, 14336, 1), (4096, 14336, 1), (257, 4096, 1),
                                             (1025, 2048, 3), (300, 6144, 8), (4097, 4096, 2)])
def test_gemv_bits_equal_the_file_layout_and_the_oracle(oxh, rows, cols, n_vec):
    w = synth.weights(Q6K, rows, cols, seed=32, stream=rows + n_vec)
    d_w, d_g = grouped_copy(w, rows, cols)
    x = synth.normal(n_vec * cols, seed=32, stream=9000 + rows)
    d_x = mv.DeviceBuffer.from_host(x)
    o1, o2 = mv.DeviceBuffer(n_vec * rows * 4), mv.DeviceBuffer(n_vec * rows * 4)
    a1, a2 = mv.DeviceBuffer(n_vec * mv.act_bytes(Q6K, cols)), mv.DeviceBuffer(n_vec * mv.act_bytes(Q6K, cols))
    mv.gemv_segments_f32(Q6K, mv.make_segments([(d_w.ptr, o1.ptr, rows, 0)]), cols, d_x.ptr, cols, a1.ptr, n_vec, rows)
    mv.gemv_segments_f32(G8, mv.make_segments([(d_g.ptr, o2.ptr, rows, 0)]), cols, d_x.ptr, cols, a2.ptr, n_vec, rows)
    mv.sync()
    want, got = o1.download(np.float32, n_vec * rows), o2.download(np.float32, n_vec * rows)
    assert np.array_equal(bits(want), bits(got))
    assert np.array_equal(a1.download(np.uint8, a1.nbytes), a2.download(np.uint8, a2.nbytes))
    # vector 0 against the oracle directly
    o = oxlibs.oracle()
    ref = np.zeros(rows, np.float32)
    tmp = np.zeros(cols, np.float32)
    x0 = np.ascontiguousarray(x[:cols])
    assert o.oxo_matvec_quantized(Q6K, w.ctypes.data, rows, cols, synth.row_bytes(Q6K, cols), x0.ctypes.data,
                                  ref.ctypes.data, tmp.ctypes.data) == 0
    assert np.array_equal(bits(got[:rows]), bits(ref))
    # stored activations from a separate quantiser launch
    mv.quantize(Q6K, d_x.ptr, cols, n_vec, cols, a1.ptr)
    mv.gemv_segments(G8, mv.make_segments([(d_g.ptr, o2.ptr, rows, 0)]), cols, a1.ptr, n_vec, rows)
    mv.sync()
    assert np.array_equal(bits(o2.download(np.float32, n_vec * rows)), bits(want))


def test_pairs_prologues_and_several_segments(oxh):
    cols, rows = 4096, 1536
    w = synth.weights(Q6K, 2 * rows, cols, seed=33, stream=1)
    d_w, d_g = grouped_copy(w, 2 * rows, cols)
    half = rows * synth.row_bytes(Q6K, cols)
    x = mv.DeviceBuffer.from_host(synth.normal(cols, seed=33, stream=2))
    g = mv.DeviceBuffer.from_host((synth.normal(cols, seed=33, stream=3) * np.float32(0.1) + np.float32(1)).astype(np.float32))
    add = mv.DeviceBuffer.from_host(synth.normal(cols, seed=33, stream=4))
    res = []
    for qt, base in ((Q6K, d_w.ptr), (G8, d_g.ptr)):
        out = mv.DeviceBuffer(2 * rows * 4)
        s_out = mv.DeviceBuffer(cols * 4)
        got = []
        # a gate/up pair behind residual add + RMSNorm
        mv.gemv_segments_fused(qt, mv.make_segments([(base, out.ptr, rows, 0, 0, base + half)]), cols, x.ptr, cols,
                               mv.PRO_RMSNORM, g.ptr, 1e-5, None, None, 1, 0, None, d_add=add.ptr, d_sum_out=s_out.ptr)
        mv.sync()
        got.append(out.download(np.float32, rows))
        got.append(s_out.download(np.float32, cols))
        # two segments of unequal size behind SwiGLU
        mv.gemv_segments_fused(qt, mv.make_segments([(base, out.ptr, 1000, 0), (base + half, out.ptr + 4000, rows, 0)]),
                               cols, x.ptr, cols, mv.PRO_SWIGLU, add.ptr)
        mv.sync()
        got.append(out.download(np.float32, 1000 + rows))
        res.append(got)
    for a, b in zip(*res):
        assert np.array_equal(bits(a), bits(b))


def test_plan_takes_the_regrouped_type(oxh):
    hidden, ffn = 2048, 4096
    ops, want, outs = [], [], []
    for i, (rows, cols) in enumerate(((hidden, ffn), (1500, hidden), (hidden, ffn))):
        w = synth.weights(Q6K, rows, cols, seed=34, stream=i)
        d_w, d_g = grouped_copy(w, rows, cols)
        x = mv.DeviceBuffer.from_host(synth.normal(cols, seed=34, stream=10 + i))
        o1, o2 = mv.DeviceBuffer(rows * 4), mv.DeviceBuffer(rows * 4)
        mv.gemv_segments_f32(Q6K, mv.make_segments([(d_w.ptr, o1.ptr, rows, 0)]), cols, x.ptr, cols)
        mv.sync()
        want.append(o1.download(np.float32, rows))
        outs.append((o2, rows, d_g, x))
        ops.append(dict(qtype=G8, segs=mv.make_segments([(d_g.ptr, o2.ptr, rows, 0)]), cols=cols, d_x=x.ptr))
    for env in (None, "0"):
        plan = mv.Plan(ops) if env is None else None
        if env is not None:
            import os
            os.environ["OXH_PLAN_PRESTAGE"] = env
            try:
                plan = mv.Plan(ops)
            finally:
                del os.environ["OXH_PLAN_PRESTAGE"]
        assert plan.info()["prestaged"] == (env is None)
        for o2, rows, _, _ in outs:
            mv.lib().oxh_memset(ctypes.c_void_p(o2.ptr), 0xFF, rows * 4, None)
        plan.launch()
        assert plan.status() == 0
        for (o2, rows, _, _), w_ in zip(outs, want):
            assert np.array_equal(bits(o2.download(np.float32, rows)), bits(w_))
        plan.destroy()


def test_what_declines_the_regrouped_type(oxh):
    lib = mv.lib()
    buf = mv.DeviceBuffer(1 << 20)
    # cols must be whole groups of eight blocks
    assert lib.oxh_q6_k_group(ctypes.c_void_p(buf.ptr), 4, 1024, ctypes.c_void_p(buf.ptr + (1 << 19)), None) == _lib.DECLINED
    assert lib.oxh_act_kind(G8, 1024) == 0 and lib.oxh_act_kind(G8, 2048) == 2
    assert lib.oxh_row_bytes(G8, 4096) == 16 * 210
    # the matrix-core kernel and the row lookup read the file layout only
    assert lib.oxh_mmq(G8, ctypes.c_void_p(buf.ptr), 16, 2048, ctypes.c_void_p(buf.ptr), 16, ctypes.c_void_p(buf.ptr), 16, None) == _lib.DECLINED
    ids = mv.DeviceBuffer.from_host(np.zeros(1, np.uint32))
    assert lib.oxh_get_rows(G8, ctypes.c_void_p(buf.ptr), 16, 2048, ctypes.c_void_p(ids.ptr), 1, ctypes.c_void_p(buf.ptr), 2048, None) == _lib.DECLINED
    with pytest.raises(_lib.OxhError):
        mv.Plan([dict(qtype=G8, segs=mv.make_segments([(buf.ptr, buf.ptr + 4096, 8, 0)]), cols=1024, d_x=buf.ptr)])


def test_host_layer_keeps_a_regrouped_copy_of_registered_q6k(oxh):
    """oc_matvec_quantized over a Q6_K matrix with cols % 2048 == 0 runs on the regrouped copy (one more
    resident form next to the file layout); results and stored activations do not change, and a batch of
    more than eight vectors (matrix cores, file layout) still agrees with the single-vector results."""
    rows, cols = 600, 4096
    w = synth.weights(Q6K, rows, cols, seed=35, stream=0)
    rb = synth.row_bytes(Q6K, cols)
    o = oxlibs.oracle()
    x = synth.normal(12 * cols, seed=35, stream=1).reshape(12, cols)
    want = np.zeros((12, rows), np.float32)
    tmp = np.zeros(cols, np.float32)
    for v in range(12):
        assert o.oxo_matvec_quantized(Q6K, w.ctypes.data, rows, cols, rb, x[v].ctypes.data, want[v].ctypes.data,
                                      tmp.ctypes.data) == 0
    assert oxh.oxh_weight_register(w.ctypes.data, w.nbytes) == 0
    try:
        for v in range(3):
            out = np.zeros(rows, np.float32)
            t = np.zeros(cols, np.float32)
            assert mv.matvec_quantized(Q6K, w, rows, cols, rb, x[v], out, t) == 0
            assert np.array_equal(bits(out), bits(want[v]))
        # fused launch of two row ranges of the same registered matrix
        a, b = np.zeros(400, np.float32), np.zeros(200, np.float32)
        t = np.zeros(cols, np.float32)
        assert mv.matvec_quantized_fused([Q6K, Q6K], [w[:400 * rb], w[400 * rb:]], [400, 200], cols, [rb, rb], x[0],
                                         [a, b], t) == 0
        assert np.array_equal(bits(np.concatenate([a, b])), bits(want[0]))
        outs = np.zeros((12, rows), np.float32)
        t = np.zeros(cols, np.float32)
        scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
        assert mv.matvec_quantized_batch(Q6K, w, rows, cols, rb, x, cols, outs, rows, 12, t, scratch) == 0
        assert np.array_equal(bits(outs), bits(want))
    finally:
        assert oxh.oxh_weight_unregister(w.ctypes.data) == 0
