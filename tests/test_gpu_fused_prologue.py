"""GPU parity for the GEMV launches with a fused prologue (RMSNorm or SwiGLU in
front of the activation quantiser), through the C ABI.

Two bars, because the prologue is float arithmetic and everything after it is
the integer path:
  * the prologue's f32 result (stored on request) agrees with the oracle's
    scalar restatement of the reference within FLOAT_RTOL relative -- the
    reference's own SIMD variants differ from its scalar form by as much;
  * given exactly those f32 values, the quantised activation bytes and the
    outputs are bit-identical to the oracle's quantise + block dot, and to the
    library's own launch without a prologue over the same values.
"""
import numpy as np
import pytest

import oxlibs
from oxidize_amd import _lib
from oxidize_amd import matvec as mv
from oxidize_amd import synth

pytestmark = pytest.mark.gpu

Q80, Q4K, Q5K, Q6K = 7, 13, 15, 16
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


def run_fused(qtype, w, rows, cols, xs, kind, b, eps=0.0):
    """-> (prologue f32 result, activation bytes, outputs), all from the device."""
    n_vec = xs.shape[0]
    d_w = mv.DeviceBuffer.from_host(w)
    d_x = mv.DeviceBuffer.from_host(xs)
    d_b = mv.DeviceBuffer.from_host(b)
    nact = mv.act_bytes(qtype, cols)
    d_y = mv.DeviceBuffer(n_vec * cols * 4)
    d_a = mv.DeviceBuffer(n_vec * nact)
    d_o = mv.DeviceBuffer(n_vec * rows * 4)
    segs = mv.make_segments([(d_w.ptr, d_o.ptr, rows, 0)])
    mv.gemv_segments_fused(qtype, segs, cols, d_x.ptr, cols, kind, d_b.ptr, eps, d_y.ptr, d_a.ptr,
                           n_vec, rows)
    y = d_y.download(np.float32, n_vec * cols).reshape(n_vec, cols)
    acts = d_a.download(np.uint8, n_vec * nact).reshape(n_vec, nact)
    out = d_o.download(np.float32, n_vec * rows).reshape(n_vec, rows)
    # the same values through the launch without a prologue
    d_o2 = mv.DeviceBuffer(n_vec * rows * 4)
    segs2 = mv.make_segments([(d_w.ptr, d_o2.ptr, rows, 0)])
    mv.gemv_segments_f32(qtype, segs2, cols, d_y.ptr, cols, None, n_vec, rows)
    out2 = d_o2.download(np.float32, n_vec * rows).reshape(n_vec, rows)
    assert np.array_equal(bits(out), bits(out2))
    return y, acts, out


def check_integer_path(qtype, w, rows, cols, y, acts, out):
    nact = acts.shape[1]
    for v in range(y.shape[0]):
        want, wtemp = oracle_matvec(qtype, w, rows, cols, np.ascontiguousarray(y[v]))
        assert np.array_equal(acts[v], wtemp.view(np.uint8)[:nact]), "activation bytes, vector %d" % v
        assert np.array_equal(bits(out[v]), bits(want)), "outputs, vector %d" % v


CASES = [
    (Q4K, 300, 256, 1), (Q4K, 4096, 4096, 1), (Q4K, 700, 14336, 1), (Q4K, 64, 18432, 1),
    (Q4K, 200, 4096, 3), (Q4K, 64, 18432, 2), (Q5K, 333, 4096, 1), (Q5K, 100, 2048, 8),
    (Q6K, 4096, 14336, 1), (Q6K, 50, 512, 5), (Q80, 1000, 896, 1), (Q80, 300, 4864, 1),
    (Q80, 90, 96, 4), (Q80, 5, 32, 1),
]


@pytest.mark.parametrize("qtype,rows,cols,n_vec", CASES)
def test_rmsnorm_prologue(oxh, qtype, rows, cols, n_vec):
    w = synth.weights(qtype, rows, cols, seed=3, stream=rows)
    xs = (synth.normal(n_vec * cols, seed=3, stream=cols) * np.float32(2.5)).reshape(n_vec, cols)
    if n_vec > 1:
        xs[1] *= np.float32(1e-3)
    gamma = (synth.normal(cols, seed=4, stream=cols) * np.float32(0.2) + np.float32(1.0)).astype(np.float32)
    eps = 1e-5
    y, acts, out = run_fused(qtype, w, rows, cols, xs, mv.PRO_RMSNORM, gamma, eps)
    o = oxlibs.oracle()
    for v in range(n_vec):
        want = np.zeros(cols, np.float32)
        o.oxo_rms_norm_f32(xs[v].ctypes.data, gamma.ctypes.data, want.ctypes.data, cols, eps)
        assert np.all(np.abs(y[v] - want) <= FLOAT_RTOL * np.abs(want)), "vector %d" % v
        xd = xs[v].astype(np.float64)
        exact = xd / np.sqrt((xd * xd).mean() + eps) * gamma
        assert np.all(np.abs(y[v] - exact) <= FLOAT_RTOL * np.abs(exact))
    check_integer_path(qtype, w, rows, cols, y, acts, out)


@pytest.mark.parametrize("qtype,rows,cols,n_vec", CASES)
def test_swiglu_prologue(oxh, qtype, rows, cols, n_vec):
    w = synth.weights(qtype, rows, cols, seed=5, stream=rows)
    gate = (synth.normal(n_vec * cols, seed=5, stream=cols) * np.float32(3.0)).reshape(n_vec, cols)
    up = synth.normal(n_vec * cols, seed=6, stream=cols).reshape(n_vec, cols)
    gate[0, :8] = np.array([0.0, -0.0, 30.0, -30.0, 88.5, -88.5, 1e-9, -100.0], np.float32)[:min(8, cols)]
    y, acts, out = run_fused(qtype, w, rows, cols, gate, mv.PRO_SWIGLU, up)
    o = oxlibs.oracle()
    for v in range(n_vec):
        want = np.zeros(cols, np.float32)
        o.oxo_swiglu_f32(gate[v].ctypes.data, up[v].ctypes.data, want.ctypes.data, cols)
        assert np.all(np.abs(y[v] - want) <= FLOAT_RTOL * np.abs(want) + 1e-30), "vector %d" % v
    check_integer_path(qtype, w, rows, cols, y, acts, out)


@pytest.mark.parametrize("qtype,rows,cols,n_vec", [(Q4K, 4096, 4096, 1), (Q4K, 64, 18432, 2), (Q6K, 50, 512, 5),
                                                  (Q5K, 333, 4096, 1), (Q80, 300, 4864, 1), (Q80, 90, 96, 4)])
def test_residual_add_rmsnorm_prologue(oxh, qtype, rows, cols, n_vec):
    """x + add is stored bit-exactly (one f32 addition per element), normalised
    like the oracle normalises that sum, and quantised / multiplied exactly."""
    w = synth.weights(qtype, rows, cols, seed=13, stream=rows)
    xs = (synth.normal(n_vec * cols, seed=13, stream=cols) * np.float32(2.0)).reshape(n_vec, cols)
    add = synth.normal(n_vec * cols, seed=14, stream=cols).reshape(n_vec, cols)
    gamma = (synth.normal(cols, seed=15, stream=cols) * np.float32(0.2) + np.float32(1.0)).astype(np.float32)
    eps = 1e-5
    d_w = mv.DeviceBuffer.from_host(w)
    d_x, d_add, d_g = (mv.DeviceBuffer.from_host(a) for a in (xs, add, gamma))
    nact = mv.act_bytes(qtype, cols)
    d_y, d_s = mv.DeviceBuffer(n_vec * cols * 4), mv.DeviceBuffer(n_vec * cols * 4)
    d_a, d_o = mv.DeviceBuffer(n_vec * nact), mv.DeviceBuffer(n_vec * rows * 4)
    segs = mv.make_segments([(d_w.ptr, d_o.ptr, rows, 0)])
    mv.gemv_segments_fused(qtype, segs, cols, d_x.ptr, cols, mv.PRO_RMSNORM, d_g.ptr, eps, d_y.ptr, d_a.ptr,
                           n_vec, rows, d_add=d_add.ptr, d_sum_out=d_s.ptr)
    total = d_s.download(np.float32, n_vec * cols).reshape(n_vec, cols)
    assert np.array_equal(bits(total), bits(xs + add))
    y = d_y.download(np.float32, n_vec * cols).reshape(n_vec, cols)
    o = oxlibs.oracle()
    for v in range(n_vec):
        want = np.zeros(cols, np.float32)
        o.oxo_rms_norm_f32(total[v].ctypes.data, gamma.ctypes.data, want.ctypes.data, cols, eps)
        assert np.all(np.abs(y[v] - want) <= FLOAT_RTOL * np.abs(want)), "vector %d" % v
    acts = d_a.download(np.uint8, n_vec * nact).reshape(n_vec, nact)
    out = d_o.download(np.float32, n_vec * rows).reshape(n_vec, rows)
    check_integer_path(qtype, w, rows, cols, y, acts, out)


def test_rmsnorm_prologue_with_several_segments(oxh):
    """q, k and v share one normalised input (one launch); and a launch whose
    segments each take their own vector (the multi-input form)."""
    cols, rows = 4096, [4096, 1024, 1024]
    ws = [synth.weights(Q4K, r, cols, seed=7, stream=i) for i, r in enumerate(rows)]
    xs = synth.normal(3 * cols, seed=7, stream=50).reshape(3, cols)
    gamma = (synth.normal(cols, seed=8) * np.float32(0.1) + np.float32(1.0)).astype(np.float32)
    d_ws = [mv.DeviceBuffer.from_host(w) for w in ws]
    d_os = [mv.DeviceBuffer(r * 4) for r in rows]
    d_x = mv.DeviceBuffer.from_host(xs)
    d_g = mv.DeviceBuffer.from_host(gamma)
    d_y = mv.DeviceBuffer(3 * cols * 4)
    for shared in (True, False):
        segs = mv.make_segments([(d_ws[i].ptr, d_os[i].ptr, rows[i], 0 if shared else i) for i in range(3)])
        d_y.upload(np.zeros(3 * cols, np.float32))
        mv.gemv_segments_fused(Q4K, segs, cols, d_x.ptr, cols, mv.PRO_RMSNORM, d_g.ptr, 1e-6, d_y.ptr,
                               None, 1, 0)
        y = d_y.download(np.float32, 3 * cols).reshape(3, cols)
        for i in range(3):
            v = 0 if shared else i
            want, _ = oracle_matvec(Q4K, ws[i], rows[i], cols, np.ascontiguousarray(y[v]))
            assert np.array_equal(bits(d_os[i].download(np.float32, rows[i])), bits(want))
        if shared:
            assert np.all(y[1:] == 0.0)


def test_fused_prologue_argument_checks(oxh):
    cols, rows = 512, 16
    w = synth.weights(Q4K, rows, cols, seed=9)
    d_w = mv.DeviceBuffer.from_host(w)
    d_x = mv.DeviceBuffer.from_host(synth.normal(cols, seed=9))
    d_b = mv.DeviceBuffer.from_host(np.ones(cols, np.float32))
    d_o = mv.DeviceBuffer(rows * 4)
    segs = mv.make_segments([(d_w.ptr, d_o.ptr, rows, 0)])
    for bad in (lambda: mv.gemv_segments_fused(Q4K, segs, cols, d_x.ptr, cols, 7, d_b.ptr),
                lambda: mv.gemv_segments_fused(Q4K, segs, cols, d_x.ptr, cols, mv.PRO_RMSNORM, 0),
                lambda: mv.gemv_segments_fused(Q4K, segs, cols, d_x.ptr, cols, mv.PRO_RMSNORM, d_b.ptr,
                                               -1.0),
                # the stored result may not overlap an input
                lambda: mv.gemv_segments_fused(Q4K, segs, cols, d_x.ptr, cols, mv.PRO_RMSNORM, d_b.ptr,
                                               1e-5, d_x.ptr + 64),
                lambda: mv.gemv_segments_fused(Q4K, segs, cols, d_x.ptr, cols, mv.PRO_SWIGLU, d_b.ptr,
                                               0.0, d_b.ptr),
                # the residual form belongs to RMSNorm, and a stored sum needs something added
                lambda: mv.gemv_segments_fused(Q4K, segs, cols, d_x.ptr, cols, mv.PRO_SWIGLU, d_b.ptr,
                                               d_add=d_b.ptr),
                lambda: mv.gemv_segments_fused(Q4K, segs, cols, d_x.ptr, cols, mv.PRO_RMSNORM, d_b.ptr,
                                               1e-5, d_sum_out=d_o.ptr),
                lambda: mv.gemv_segments_fused(Q4K, segs, cols, d_x.ptr, cols, mv.PRO_RMSNORM, d_b.ptr,
                                               1e-5, d_add=d_b.ptr, d_sum_out=d_x.ptr)):
        with pytest.raises(_lib.OxhError) as e:
            bad()
        assert e.value.status == _lib.ERR_ARG


# ─── paired gate / up matrices: h = silu(W_gate x) * (W_up x) in one pass ───

def paired_case(qtype, rows, cols, n_vec, seed):
    wg = synth.weights(qtype, rows, cols, seed=seed, stream=1)
    wu = synth.weights(qtype, rows, cols, seed=seed, stream=2)
    xs = synth.normal(n_vec * cols, seed=seed, stream=3).reshape(n_vec, cols)
    return wg, wu, xs


def check_paired(qtype, wg, wu, rows, cols, x_used, h):
    """h against the oracle: gate and up exactly, their combination to rounding."""
    o = oxlibs.oracle()
    for v in range(x_used.shape[0]):
        gate, _ = oracle_matvec(qtype, wg, rows, cols, np.ascontiguousarray(x_used[v]))
        up, _ = oracle_matvec(qtype, wu, rows, cols, np.ascontiguousarray(x_used[v]))
        want = np.zeros(rows, np.float32)
        o.oxo_swiglu_f32(gate.ctypes.data, up.ctypes.data, want.ctypes.data, rows)
        assert np.all(np.abs(h[v] - want) <= FLOAT_RTOL * np.abs(want) + 1e-30), "vector %d" % v


@pytest.mark.parametrize("qtype,rows,cols,n_vec", [
    (Q4K, 14336, 4096, 1), (Q4K, 77, 512, 1), (Q4K, 1000, 1024, 3), (Q4K, 140000, 256, 1),
    (Q5K, 700, 2048, 1), (Q6K, 2000, 1024, 2), (Q80, 4864, 896, 1), (Q80, 100, 64, 8),
])
def test_paired_gate_up_swiglu(oxh, qtype, rows, cols, n_vec):
    wg, wu, xs = paired_case(qtype, rows, cols, n_vec, seed=21)
    d_g, d_u, d_x = (mv.DeviceBuffer.from_host(a) for a in (wg, wu, xs))
    d_h = mv.DeviceBuffer(n_vec * rows * 4)
    segs = mv.make_segments([(d_g.ptr, d_h.ptr, rows, 0, 0, d_u.ptr)])
    mv.gemv_segments_f32(qtype, segs, cols, d_x.ptr, cols, None, n_vec, rows)
    h = d_h.download(np.float32, n_vec * rows).reshape(n_vec, rows)
    check_paired(qtype, wg, wu, rows, cols, xs, h)
    # the same from the library's own separate launches: identical gate and up bits go in
    d_go, d_uo = mv.DeviceBuffer(n_vec * rows * 4), mv.DeviceBuffer(n_vec * rows * 4)
    for d_w, d_o in ((d_g, d_go), (d_u, d_uo)):
        mv.gemv_segments_f32(qtype, mv.make_segments([(d_w.ptr, d_o.ptr, rows, 0)]), cols, d_x.ptr, cols,
                             None, n_vec, rows)
    gate = d_go.download(np.float32, n_vec * rows)
    up = d_uo.download(np.float32, n_vec * rows)
    want = np.zeros(n_vec * rows, np.float32)
    oxlibs.oracle().oxo_swiglu_f32(gate.ctypes.data, up.ctypes.data, want.ctypes.data, want.size)
    assert np.all(np.abs(h.ravel() - want) <= FLOAT_RTOL * np.abs(want) + 1e-30)
    # pre-quantised activations take the same path
    nact = mv.act_bytes(qtype, cols)
    d_a = mv.DeviceBuffer(n_vec * nact)
    mv.quantize(qtype, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    d_h2 = mv.DeviceBuffer(n_vec * rows * 4)
    mv.gemv_segments(qtype, mv.make_segments([(d_g.ptr, d_h2.ptr, rows, 0, 0, d_u.ptr)]), cols, d_a.ptr,
                     n_vec, rows)
    assert np.array_equal(bits(d_h2.download(np.float32, n_vec * rows)), bits(h.ravel()))


def test_paired_with_rmsnorm_prologue_and_mixed_segments(oxh):
    """A feed-forward block's first launch: x + residual -> RMSNorm -> gate/up ->
    SwiGLU; and a launch that mixes a paired and a plain segment."""
    rows, cols = 2000, 4096
    wg, wu, xs = paired_case(Q4K, rows, cols, 1, seed=22)
    res = synth.normal(cols, seed=22, stream=9).reshape(1, cols)
    gamma = (synth.normal(cols, seed=23) * np.float32(0.1) + np.float32(1.0)).astype(np.float32)
    d_g, d_u, d_x, d_r, d_gm = (mv.DeviceBuffer.from_host(a) for a in (wg, wu, xs, res, gamma))
    d_h, d_y, d_s = mv.DeviceBuffer(rows * 4), mv.DeviceBuffer(cols * 4), mv.DeviceBuffer(cols * 4)
    segs = mv.make_segments([(d_g.ptr, d_h.ptr, rows, 0, 0, d_u.ptr)])
    mv.gemv_segments_fused(Q4K, segs, cols, d_x.ptr, cols, mv.PRO_RMSNORM, d_gm.ptr, 1e-5, d_y.ptr, None,
                           1, rows, d_add=d_r.ptr, d_sum_out=d_s.ptr)
    assert np.array_equal(bits(d_s.download(np.float32, cols)), bits((xs + res).ravel()))
    y = d_y.download(np.float32, cols).reshape(1, cols)
    check_paired(Q4K, wg, wu, rows, cols, y, d_h.download(np.float32, rows).reshape(1, rows))
    # mixed: segment 0 paired, segment 1 a plain matrix over the same input
    w3 = synth.weights(Q4K, 300, cols, seed=24)
    d_w3, d_o3 = mv.DeviceBuffer.from_host(w3), mv.DeviceBuffer(300 * 4)
    segs = mv.make_segments([(d_g.ptr, d_h.ptr, rows, 0, 0, d_u.ptr), (d_w3.ptr, d_o3.ptr, 300, 0)])
    mv.gemv_segments_f32(Q4K, segs, cols, d_x.ptr, cols, None, 1, 0)
    check_paired(Q4K, wg, wu, rows, cols, xs, d_h.download(np.float32, rows).reshape(1, rows))
    want, _ = oracle_matvec(Q4K, w3, 300, cols, np.ascontiguousarray(xs[0]))
    assert np.array_equal(bits(d_o3.download(np.float32, 300)), bits(want))


def test_decode_chain_stage_by_stage(oxh):
    """Two layers of the dependent decode chain (four launches per layer, float
    steps fused into the GEMVs).  Every stage is checked against the oracle
    applied to the stage's own inputs as the device produced them: sums and
    integer paths to the bit, RMSNorm and SwiGLU to rounding."""
    from oxidize_amd.workloads import DecodeChain, DecodeSet
    hidden, kv, ffn, layers = 1024, 256, 2816, 2
    ds = DecodeSet(hidden=hidden, kv=kv, ffn=ffn, layers=layers, seed=3, keep_host=range(layers))
    ch = DecodeChain(ds, eps=1e-5, seed=3, capture=True)
    ch.launch_step()
    mv.sync()
    o = oxlibs.oracle()

    def rms(x, g):
        out = np.zeros(x.size, np.float32)
        o.oxo_rms_norm_f32(x.ctypes.data, g.ctypes.data, out.ctypes.data, x.size, 1e-5)
        return out

    x, f = ch.x0_host, ch.f0_host
    for l in range(layers):
        c = {k: b.download(np.float32, b.nbytes // 4) for k, b in ch.cap[l].items()}
        assert np.array_equal(bits(c["x1"]), bits(x + f))
        want = rms(c["x1"], ch.g_attn_host[l])
        assert np.all(np.abs(c["n1"] - want) <= FLOAT_RTOL * np.abs(want))
        off = 0
        for seg, r in enumerate((hidden, kv, kv)):
            got, _ = oracle_matvec(Q4K, ds.host[(l, 0, seg)], r, hidden, c["n1"])
            assert np.array_equal(bits(c["qkv"][off:off + r]), bits(got))
            off += r
        got, _ = oracle_matvec(Q4K, ds.host[(l, 1, 0)], hidden, hidden, np.ascontiguousarray(c["qkv"][:hidden]))
        assert np.array_equal(bits(c["o"]), bits(got))
        assert np.array_equal(bits(c["x2"]), bits(c["x1"] + c["o"]))
        want = rms(c["x2"], ch.g_ffn_host[l])
        assert np.all(np.abs(c["n2"] - want) <= FLOAT_RTOL * np.abs(want))
        gate, _ = oracle_matvec(Q4K, ds.host[(l, 2, 0)], ffn, hidden, c["n2"])
        up, _ = oracle_matvec(Q4K, ds.host[(l, 2, 1)], ffn, hidden, c["n2"])
        want = np.zeros(ffn, np.float32)
        o.oxo_swiglu_f32(gate.ctypes.data, up.ctypes.data, want.ctypes.data, ffn)
        assert np.all(np.abs(c["h"] - want) <= FLOAT_RTOL * np.abs(want) + 1e-30)
        got, _ = oracle_matvec(Q6K, ds.host[(l, 3, 0)], hidden, ffn, c["h"])
        assert np.array_equal(bits(c["f"]), bits(got))
        x, f = c["x2"], c["f"]
    # a replay as one graph reproduces the eager run bit for bit
    eager = ch.last_x.download(np.float32, hidden)
    g = mv.Graph()
    with g:
        ch.launch_step(g.stream)
    for _ in range(3):
        g.launch()
        mv.sync()
        assert np.array_equal(bits(ch.last_x.download(np.float32, hidden)), bits(eager))
