"""Q4_K / Q5_K stored tile-major (oxh_tile16, OXH_Q4_K_T16 / OXH_Q5_K_T16): the rewrite is checked against
a numpy statement of the layout the header documents; the tile kernels must give from it the bits they give
from the file layout, which other tests hold to the oracle, in segment launches and in the expert layer."""
import numpy as np
import pytest

import oxlibs
from oxidize_amd import _lib, synth
from oxidize_amd import matvec as mv

pytestmark = pytest.mark.gpu
Q4K, Q5K, Q6K = 13, 15, 16
T16 = {Q4K: mv.Q4_K_T16, Q5K: mv.Q5_K_T16}
WB = {Q4K: 144, Q5K: 176}


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def tile_major(w, qtype, rows, cols):
    """block (row r, index b) at ((r // 16) * B + b) * 16 + r % 16; the last group padded with zeros"""
    nb, wb = cols // 256, WB[qtype]
    groups = (rows + 15) // 16
    padded = np.zeros((groups * 16, nb, wb), np.uint8)
    padded[:rows] = w.reshape(rows, nb, wb)
    return np.ascontiguousarray(padded.reshape(groups, 16, nb, wb).transpose(0, 2, 1, 3)).reshape(-1)


def tiled_copy(qtype, w, rows, cols):
    d_w = mv.DeviceBuffer.from_host(w)
    n = mv.tile16_bytes(qtype, rows, cols)
    assert n == (rows + 15) // 16 * 16 * synth.row_bytes(qtype, cols)
    d_t = mv.DeviceBuffer(n)
    mv.tile16(qtype, d_w.ptr, rows, cols, d_t.ptr)
    mv.sync()
    return d_w, d_t


@pytest.mark.parametrize("qtype", [Q4K, Q5K])
@pytest.mark.parametrize("rows,cols", [(1, 256), (16, 512), (100, 4096), (4096, 1024), (333, 14336)])
def test_rewrite_is_the_documented_permutation(oxh, qtype, rows, cols):
    w = synth.weights(qtype, rows, cols, seed=41, stream=rows)
    d_w, d_t = tiled_copy(qtype, w, rows, cols)
    got = d_t.download(np.uint8, d_t.nbytes)
    assert np.array_equal(got, tile_major(w, qtype, rows, cols))


def test_sizes_and_refusals(oxh):
    assert mv.tile16_bytes(Q6K, 64, 256) == 0
    assert mv.tile16_bytes(Q4K, 64, 300) == 0
    assert mv.tile16_bytes(Q4K, 17, 512) == 32 * 2 * 144
    d = mv.DeviceBuffer(1 << 16)
    with pytest.raises(mv.OxhError):
        mv.tile16(Q6K, d.ptr, 16, 256, d.ptr + 32768)
    with pytest.raises(mv.OxhError):
        mv.tile16(Q4K, d.ptr, 16, 256, d.ptr)           # in place
    # the plain GEMV entry point and the prefill entry point read the file layout only
    o = mv.DeviceBuffer(64 * 4)
    x = mv.DeviceBuffer.from_host(synth.normal(256, seed=1, stream=1))
    with pytest.raises(mv.OxhError):
        mv.gemv_segments_f32(mv.Q4_K_T16, mv.make_segments([(d.ptr, o.ptr, 64, 0)]), 256, x.ptr, 256, None, 1, 64)


@pytest.mark.parametrize("qtype", [Q4K, Q5K])
@pytest.mark.parametrize("rows,cols,n_vec", [(64, 256, 1), (100, 4096, 4), (1000, 2048, 3), (4096, 4096, 8),
                                             (777, 1024, 16), (14336, 4096, 5), (9, 512, 2)])
def test_segment_launch_bits_equal_the_file_layout(oxh, qtype, rows, cols, n_vec):
    w = synth.weights(qtype, rows, cols, seed=42, stream=rows + n_vec)
    d_w, d_t = tiled_copy(qtype, w, rows, cols)
    x = synth.normal(n_vec * cols, seed=42, stream=7000 + rows)
    d_x = mv.DeviceBuffer.from_host(x)
    acts = mv.DeviceBuffer(n_vec * mv.act_bytes(qtype, cols))
    mv.quantize(qtype, d_x.ptr, cols, n_vec, cols, acts.ptr)
    o1, o2, o3 = (mv.DeviceBuffer(n_vec * rows * 4) for _ in range(3))
    # the file layout through the prefill entry point (always the tile kernel), tile-major through the
    # segment entry points, with stored activations and with the quantiser in front
    mv.mmq(qtype, d_w.ptr, rows, cols, acts.ptr, n_vec, o1.ptr, rows)
    mv.gemv_segments(T16[qtype], mv.make_segments([(d_t.ptr, o2.ptr, rows, 0)]), cols, acts.ptr, n_vec, rows)
    a2 = mv.DeviceBuffer(acts.nbytes)
    mv.gemv_segments_f32(T16[qtype], mv.make_segments([(d_t.ptr, o3.ptr, rows, 0)]), cols, d_x.ptr, cols, a2.ptr,
                         n_vec, rows)
    mv.sync()
    want = o1.download(np.float32, n_vec * rows)
    assert np.array_equal(bits(o2.download(np.float32, n_vec * rows)), bits(want))
    assert np.array_equal(bits(o3.download(np.float32, n_vec * rows)), bits(want))
    # vector 0 against the oracle directly
    o = oxlibs.oracle()
    ref = np.zeros(rows, np.float32)
    tmp = np.zeros(cols, np.float32)
    x0 = np.ascontiguousarray(x[:cols])
    assert o.oxo_matvec_quantized(qtype, w.ctypes.data, rows, cols, synth.row_bytes(qtype, cols), x0.ctypes.data,
                                  ref.ctypes.data, tmp.ctypes.data) == 0
    assert np.array_equal(bits(want[:rows]), bits(ref))


def test_several_segments_with_their_own_counts(oxh):
    """Expert-style launch: slices of one tile-major stack, each over its own run of activations."""
    cols, rows, n_exp = 1024, 192, 5
    counts = [3, 0, 16, 1, 7]
    w = synth.weights(Q4K, n_exp * rows, cols, seed=43, stream=5)
    d_w, d_t = tiled_copy(Q4K, w, n_exp * rows, cols)
    n_act = sum(counts)
    x = synth.normal(n_act * cols, seed=43, stream=6)
    d_x = mv.DeviceBuffer.from_host(x)
    acts = mv.DeviceBuffer(n_act * mv.act_bytes(Q4K, cols))
    mv.quantize(Q4K, d_x.ptr, cols, n_act, cols, acts.ptr)
    o1, o2 = mv.DeviceBuffer(n_act * rows * 4), mv.DeviceBuffer(n_act * rows * 4)
    rb = synth.row_bytes(Q4K, cols)
    seg_f, seg_t, first = [], [], 0
    for e, c in enumerate(counts):
        if c:
            seg_f.append((d_w.ptr + e * rows * rb, o1.ptr + first * rows * 4, rows, first, c))
            seg_t.append((d_t.ptr + e * rows * rb, o2.ptr + first * rows * 4, rows, first, c))
        first += c
    for segs in seg_f:
        # file layout one segment at a time through the prefill entry point
        mv.mmq(Q4K, segs[0], rows, cols, acts.ptr + segs[3] * mv.act_bytes(Q4K, cols), segs[4], segs[1], rows)
    mv.gemv_segments(mv.Q4_K_T16, mv.make_segments(seg_t), cols, acts.ptr, 1, rows)
    mv.sync()
    assert np.array_equal(bits(o2.download(np.float32, n_act * rows)), bits(o1.download(np.float32, n_act * rows)))


@pytest.mark.parametrize("qt_gu,qt_dn,n_tok", [(Q4K, Q4K, 16), (Q5K, Q4K, 5), (Q4K, Q6K, 9), (Q4K, Q4K, 200)])
def test_expert_layer_bits_equal_the_file_layout(oxh, qt_gu, qt_dn, n_tok):
    n_expert, top_k, hidden, ffn = 8, 2, 512, 1280
    wg = synth.weights(qt_gu, n_expert * ffn, hidden, seed=44, stream=1)
    wu = synth.weights(qt_gu, n_expert * ffn, hidden, seed=44, stream=2)
    wd = synth.weights(qt_dn, n_expert * hidden, ffn, seed=44, stream=3)
    d_g, t_g = tiled_copy(qt_gu, wg, n_expert * ffn, hidden)
    d_u, t_u = tiled_copy(qt_gu, wu, n_expert * ffn, hidden)
    if qt_dn in T16:
        d_d, t_d = tiled_copy(qt_dn, wd, n_expert * hidden, ffn)
    else:
        d_d = t_d = mv.DeviceBuffer.from_host(wd)
    logits = synth.normal(n_tok * n_expert, seed=44, stream=4)
    x = synth.normal(n_tok * hidden, seed=44, stream=5)
    d_l, d_x = mv.DeviceBuffer.from_host(logits), mv.DeviceBuffer.from_host(x)
    y1, y2 = mv.DeviceBuffer(n_tok * hidden * 4), mv.DeviceBuffer(n_tok * hidden * 4)
    plain = mv.MoeLayer(qt_gu, qt_dn, d_g.ptr, d_u.ptr, d_d.ptr, n_expert, top_k, hidden, ffn, True, max_tok=n_tok)
    tiled = mv.MoeLayer(T16[qt_gu], T16.get(qt_dn, qt_dn), t_g.ptr, t_u.ptr, t_d.ptr, n_expert, top_k, hidden, ffn,
                        True, max_tok=n_tok)
    plain.forward(d_l.ptr, d_x.ptr, n_tok, y1.ptr)
    tiled.forward(d_l.ptr, d_x.ptr, n_tok, y2.ptr)
    mv.sync()
    assert np.array_equal(bits(y2.download(np.float32, n_tok * hidden)), bits(y1.download(np.float32, n_tok * hidden)))


def test_expert_layer_declines_rows_off_the_group_size(oxh):
    d = mv.DeviceBuffer(1 << 20)
    with pytest.raises(mv.OxhError):
        mv.MoeLayer(mv.Q4_K_T16, Q4K, d.ptr, d.ptr, d.ptr, 4, 2, 512, 1288, True, max_tok=4)


# ── Q8_0 ────────────────────────────────────────────────────────────────────
Q80 = 7


def q80_tile_major(w, rows, cols):
    """per (16-row group, run of four blocks) a 2176-byte unit: the 16-byte piece at 16 * (16q + r) of half h
    holds row r's values 8q..8q+7 of block 4c + 2h (bytes 0-7) and 4c + 2h + 1 (bytes 8-15); the scales of row
    r at 2048 + 8r; the last group padded with zeros"""
    nb = cols // 32
    groups, runs = (rows + 15) // 16, nb // 4
    padded = np.zeros((groups * 16, nb, 34), np.uint8)
    padded[:rows] = w.reshape(rows, nb, 34)
    g = padded.reshape(groups, 16, runs, 4, 34)                              # [group][row][run][k][34]
    out = np.zeros((groups, runs, 2176), np.uint8)
    for k in range(4):
        for q in range(4):
            for r in range(16):
                at = 1024 * (k >> 1) + 16 * (16 * q + r) + 8 * (k & 1)
                out[:, :, at:at + 8] = g[:, r, :, k, 2 + 8 * q:10 + 8 * q]
        for r in range(16):
            out[:, :, 2048 + 8 * r + 2 * k:2050 + 8 * r + 2 * k] = g[:, r, :, k, 0:2]
    return out.reshape(-1)


@pytest.mark.parametrize("rows,cols", [(1, 128), (16, 256), (100, 896), (4864, 896), (333, 4864)])
def test_q8_0_rewrite_is_the_documented_permutation(oxh, rows, cols):
    w = synth.weights(Q80, rows, cols, seed=45, stream=rows)
    d_w = mv.DeviceBuffer.from_host(w)
    n = mv.tile16_bytes(Q80, rows, cols)
    assert n == (rows + 15) // 16 * (cols // 128) * 2176
    d_t = mv.DeviceBuffer(n)
    mv.tile16(Q80, d_w.ptr, rows, cols, d_t.ptr)
    mv.sync()
    assert np.array_equal(d_t.download(np.uint8, n), q80_tile_major(w, rows, cols))


@pytest.mark.parametrize("rows,cols,n_vec", [(16, 128, 1), (100, 896, 4), (1000, 896, 8), (4864, 896, 2), (896, 4864, 8),
                                             (777, 1024, 16), (20000, 896, 5), (9, 256, 3), (4100, 2048, 12)])
def test_q8_0_segment_launch_bits_equal_the_file_layout(oxh, rows, cols, n_vec):
    w = synth.weights(Q80, rows, cols, seed=46, stream=rows + n_vec)
    d_w = mv.DeviceBuffer.from_host(w)
    d_t = mv.DeviceBuffer(mv.tile16_bytes(Q80, rows, cols))
    mv.tile16(Q80, d_w.ptr, rows, cols, d_t.ptr)
    x = synth.normal(n_vec * cols, seed=46, stream=8000 + rows)
    d_x = mv.DeviceBuffer.from_host(x)
    a1, a2 = mv.DeviceBuffer(n_vec * mv.act_bytes(Q80, cols)), mv.DeviceBuffer(n_vec * mv.act_bytes(Q80, cols))
    o1, o2, o3 = (mv.DeviceBuffer(n_vec * rows * 4) for _ in range(3))
    mv.gemv_segments_f32(Q80, mv.make_segments([(d_w.ptr, o1.ptr, rows, 0)]), cols, d_x.ptr, cols, a1.ptr, n_vec, rows)
    mv.gemv_segments_f32(mv.Q8_0_T16, mv.make_segments([(d_t.ptr, o2.ptr, rows, 0)]), cols, d_x.ptr, cols, a2.ptr,
                         n_vec, rows)
    mv.gemv_segments(mv.Q8_0_T16, mv.make_segments([(d_t.ptr, o3.ptr, rows, 0)]), cols, a1.ptr, n_vec, rows)
    mv.sync()
    want = o1.download(np.float32, n_vec * rows)
    assert np.array_equal(a1.download(np.uint8, a1.nbytes), a2.download(np.uint8, a2.nbytes))
    assert np.array_equal(bits(o2.download(np.float32, n_vec * rows)), bits(want))
    assert np.array_equal(bits(o3.download(np.float32, n_vec * rows)), bits(want))
    # f32 inputs with nowhere to put the quantised blocks: the workgroups quantise for themselves
    o4 = mv.DeviceBuffer(n_vec * rows * 4)
    mv.gemv_segments_f32(mv.Q8_0_T16, mv.make_segments([(d_t.ptr, o4.ptr, rows, 0)]), cols, d_x.ptr, cols, None,
                         n_vec, rows)
    mv.sync()
    assert np.array_equal(bits(o4.download(np.float32, n_vec * rows)), bits(want))


def test_q8_0_several_segments_with_their_own_counts(oxh):
    cols, rows = 896, 208
    counts = [3, 16, 1, 7]
    w = synth.weights(Q80, len(counts) * rows, cols, seed=47, stream=5)
    d_w = mv.DeviceBuffer.from_host(w)
    d_t = mv.DeviceBuffer(mv.tile16_bytes(Q80, len(counts) * rows, cols))
    mv.tile16(Q80, d_w.ptr, len(counts) * rows, cols, d_t.ptr)
    n_act = sum(counts)
    d_x = mv.DeviceBuffer.from_host(synth.normal(n_act * cols, seed=47, stream=6))
    acts = mv.DeviceBuffer(n_act * mv.act_bytes(Q80, cols))
    mv.quantize(Q80, d_x.ptr, cols, n_act, cols, acts.ptr)
    o1, o2 = mv.DeviceBuffer(n_act * rows * 4), mv.DeviceBuffer(n_act * rows * 4)
    rb = synth.row_bytes(Q80, cols)
    seg_f, seg_t, first = [], [], 0
    for e, c in enumerate(counts):
        seg_f.append((d_w.ptr + e * rows * rb, o1.ptr + first * rows * 4, rows, first, c))
        seg_t.append((d_t.ptr + e * rows * rb, o2.ptr + first * rows * 4, rows, first, c))
        first += c
    mv.gemv_segments(Q80, mv.make_segments(seg_f), cols, acts.ptr, 1, rows)
    mv.gemv_segments(mv.Q8_0_T16, mv.make_segments(seg_t), cols, acts.ptr, 1, rows)
    mv.sync()
    assert np.array_equal(bits(o2.download(np.float32, n_act * rows)), bits(o1.download(np.float32, n_act * rows)))


def test_q8_0_widths_off_the_run_size_are_declined(oxh):
    assert mv.tile16_bytes(Q80, 64, 96) == 0
    assert mv.tile16_bytes(Q80, 17, 256) == 2 * 2 * 2176
    d = mv.DeviceBuffer(1 << 16)
    with pytest.raises(mv.OxhError):
        mv.tile16(Q80, d.ptr, 16, 96, d.ptr + 32768)


def test_host_batch_keeps_a_tile_major_copy_of_a_tall_q8_0_matrix(oxh):
    """oc_matvec_quantized_batch over a Q8_0 matrix with enough rows for a 16-row group per wave: batches of
    2 to 16 run from a tile-major copy kept with the registry entry (counted in the cache's bytes), single
    vectors and refilled buffers keep giving the oracle's bits."""
    import ctypes
    rows, cols, n_vec = 70000, 128, 4
    rb = synth.row_bytes(Q80, cols)
    w = synth.weights(Q80, rows, cols, seed=48, stream=1)
    xs = synth.normal(n_vec * cols, seed=48, stream=2).reshape(n_vec, cols)
    temp = np.zeros(cols, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)

    def cached_bytes():
        v = [ctypes.c_size_t(0) for _ in range(4)]
        assert oxh.oxh_weight_stats(*[ctypes.byref(t) for t in v]) == 0
        return int(v[2].value)

    def check():
        outs = np.zeros((n_vec, rows), np.float32)
        assert mv.matvec_quantized_batch(Q80, w, rows, cols, rb, xs, cols, outs, rows, n_vec, temp, scratch) == 0
        o = oxlibs.oracle()
        for v in range(n_vec):
            want = np.zeros(rows, np.float32)
            x = np.ascontiguousarray(xs[v])
            assert o.oxo_matvec_quantized(Q80, w.ctypes.data, rows, cols, rb, x.ctypes.data, want.ctypes.data,
                                          temp.ctypes.data) == 0
            assert np.array_equal(bits(outs[v]), bits(want))

    assert oxh.oxh_weight_clear() == 0
    check()
    assert cached_bytes() == w.nbytes + mv.tile16_bytes(Q80, rows, cols)
    check()                                                 # the kept copy again
    assert cached_bytes() == w.nbytes + mv.tile16_bytes(Q80, rows, cols)
    w[:] = synth.weights(Q80, rows, cols, seed=49, stream=1)      # same buffer, other matrix: both copies go
    check()
    assert cached_bytes() == w.nbytes + mv.tile16_bytes(Q80, rows, cols)
    assert oxh.oxh_cpu_fallback_calls() == 0
    assert oxh.oxh_weight_clear() == 0


# ── plans over tile-major Q8_0: many matrices, several activations each, one launch ─────────────────────────
class _TiledOp:
    """One operation: segments over their own matrices and runs of activations of one f32 input, its outputs
    [activation][all segments' rows]; the file layout's launch beside the tile-major plan entry."""

    def __init__(self, cols, segs, seed, keep_acts=True):
        self.cols, self.segs = cols, segs                    # segs: [(rows, act_first, n_vec)]
        self.n_act = max(a + n for _, a, n in segs)
        self.total = sum(r for r, _, _ in segs)
        self.d_x = mv.DeviceBuffer.from_host(synth.normal(self.n_act * cols, seed=seed, stream=1))
        self.out_file, self.out_plan = mv.DeviceBuffer(16 * self.total * 4), mv.DeviceBuffer(16 * self.total * 4)
        for b in (self.out_file, self.out_plan):
            b.upload(np.full(16 * self.total, np.float32(-7.0)))
        self.acts_file = mv.DeviceBuffer(self.n_act * mv.act_bytes(Q80, cols))
        self.acts_plan = mv.DeviceBuffer(self.n_act * mv.act_bytes(Q80, cols)) if keep_acts else None
        self.keep = []
        file_items, plan_items, off = [], [], 0
        for k, (rows, first, n_vec) in enumerate(segs):
            w = synth.weights(Q80, rows, cols, seed=seed, stream=10 + k)
            d_w = mv.DeviceBuffer.from_host(w)
            d_t = mv.DeviceBuffer(mv.tile16_bytes(Q80, rows, cols))
            mv.tile16(Q80, d_w.ptr, rows, cols, d_t.ptr)
            self.keep += [d_w, d_t]
            file_items.append((d_w.ptr, self.out_file.ptr + off * 4, rows, first, n_vec))
            plan_items.append((d_t.ptr, self.out_plan.ptr + off * 4, rows, first, n_vec))
            off += rows
        self.file_items = file_items
        self.file_segs, self.plan_segs = mv.make_segments(file_items), mv.make_segments(plan_items)

    def launch_file_layout(self):
        """the quantiser, then every segment from the file layout, at most eight activations per launch (what
        the dot kernel takes)"""
        mv.quantize(Q80, self.d_x.ptr, self.cols, self.n_act, self.cols, self.acts_file.ptr)
        for d_w, d_out, rows, first, n_vec in self.file_items:
            for v0 in range(0, n_vec, 8):
                n = min(8, n_vec - v0)
                mv.gemv_segments(Q80, mv.make_segments([(d_w, d_out + v0 * self.total * 4, rows, first + v0, n)]),
                                 self.cols, self.acts_file.ptr, 1, self.total)

    def plan_op(self):
        return dict(qtype=mv.Q8_0_T16, segs=self.plan_segs, cols=self.cols, d_x=self.d_x.ptr,
                    d_act_out=None if self.acts_plan is None else self.acts_plan.ptr, out_stride=self.total)

    def check(self):
        n = 16 * self.total
        assert np.array_equal(bits(self.out_plan.download(np.float32, n)), bits(self.out_file.download(np.float32, n)))
        if self.acts_plan is not None:                       # the blocks of every activation a segment names
            got = self.acts_plan.download(np.uint8, self.acts_plan.nbytes).reshape(self.n_act, -1)
            want = self.acts_file.download(np.uint8, self.acts_file.nbytes).reshape(self.n_act, -1)
            named = sorted({v for _, first, n in self.segs for v in range(first, first + n)})
            assert np.array_equal(got[named], want[named])


def test_q8_0_tile_major_plan_gives_the_launches_bits(oxh):
    """Operations of different widths, ragged row counts, several segments with their own runs of activations,
    with and without the quantised blocks stored: one launch, the bits of the file layout's launches (which
    other tests hold to the oracle), nothing written beyond a segment's rows and activations."""
    ops = [_TiledOp(896, [(896, 0, 8), (128, 0, 8), (128, 0, 8)], seed=60),
           _TiledOp(4864, [(896, 0, 8)], seed=61),
           _TiledOp(896, [(4864, 0, 5), (4864, 0, 5)], seed=62, keep_acts=False),
           _TiledOp(128, [(1, 0, 1), (17, 1, 16), (333, 3, 2)], seed=63),
           _TiledOp(1024, [(50000, 2, 3)], seed=64),
           _TiledOp(256, [(15, 0, 16)], seed=65, keep_acts=False)]
    for o in ops:
        o.launch_file_layout()
    plan = mv.Plan([o.plan_op() for o in ops])
    info = plan.info()
    assert info["n_ops"] == len(ops) and info["n_waits"] == 0
    assert info["lds_bytes"] == 4864 // 32 * 576                  # the widest staged image
    for _ in range(2):                                       # a plan is launched again and again
        plan.launch()
    assert plan.status() == 0
    for o in ops:
        o.check()
    plan.destroy()


def test_q8_0_tile_major_plan_of_one_small_operation(oxh):
    o = _TiledOp(128, [(16, 0, 1)], seed=66)
    o.launch_file_layout()
    plan = mv.Plan([o.plan_op()])
    plan.launch()
    assert plan.status() == 0
    o.check()
    plan.destroy()


def test_q8_0_tile_major_plan_refusals(oxh):
    a, b = _TiledOp(896, [(64, 0, 4)], seed=67), _TiledOp(896, [(64, 0, 4)], seed=68)
    # an operation of another form among them
    other = dict(qtype=Q80, segs=a.file_segs, cols=896, d_x=a.d_x.ptr)
    with pytest.raises(mv.OxhError) as e:
        mv.Plan([a.plan_op(), other])
    assert e.value.status == mv.DECLINED
    # several activations and no stride
    op = a.plan_op()
    op["out_stride"] = 0
    with pytest.raises(mv.OxhError) as e:
        mv.Plan([op])
    assert e.value.status == _lib.ERR_ARG
    # more activations than a tile holds
    op = a.plan_op()
    op["segs"] = mv.make_segments([(a.keep[1].ptr, a.out_plan.ptr, 64, 0, 17)])
    with pytest.raises(mv.OxhError) as e:
        mv.Plan([op])
    assert e.value.status == _lib.ERR_ARG
    # a width that is not whole runs of four blocks
    op = a.plan_op()
    op["cols"] = 96
    with pytest.raises(mv.OxhError) as e:
        mv.Plan([op])
    assert e.value.status == mv.DECLINED
    # an operation that reads what another writes
    op = b.plan_op()
    op["d_x"] = a.out_plan.ptr
    with pytest.raises(mv.OxhError) as e:
        mv.Plan([a.plan_op(), op])
    assert e.value.status == mv.DECLINED
