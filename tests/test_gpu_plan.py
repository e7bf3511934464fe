"""A decode step as one persistent launch (oxh_plan_*) against the same matmuls launched one by one
(oxh_gemv_segments_fused / _f32, themselves held to the oracle elsewhere): every output, every stored
quantised activation and the residual stream must be bit-identical, launch after launch; and the bounded
wait between dependent operations must give up cleanly when it cannot be satisfied."""
import ctypes

import numpy as np
import pytest

import oxlibs
from oxidize_amd import _lib, synth
from oxidize_amd import matvec as mv
from oxidize_amd.workloads import DecodeChain, DecodeSet

pytestmark = pytest.mark.gpu
Q80, Q4K, Q5K, Q6K = 7, 13, 15, 16


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


@pytest.mark.parametrize("hidden,kv,ffn,layers", [(1024, 256, 2816, 3), (4096, 1024, 14336, 2), (256, 256, 512, 5)])
def test_independent_set_matches_single_launches_and_oracle(oxh, monkeypatch, hidden, kv, ffn, layers):
    d = DecodeSet(hidden=hidden, kv=kv, ffn=ffn, layers=layers, seed=3, keep_host=(0,))
    d.launch_step()
    mv.sync()
    want_out = [[d.output(l, op) for op in range(4)] for l in range(layers)]
    want_act = [[d.activation(l, op) for op in range(4)] for l in range(layers)]
    for l in range(layers):
        for op in range(4):
            mv.lib().oxh_memset(ctypes.c_void_p(d.out[l][op].ptr), 0xFF, d.out[l][op].nbytes, None)
            mv.lib().oxh_memset(ctypes.c_void_p(d.act[l][op].ptr), 0xFF, d.act[l][op].nbytes, None)
    plan = mv.Plan(d.plan_ops())
    info = plan.info()
    assert info["n_ops"] == 4 * layers and info["n_waits"] == 0      # nothing depends on anything here
    assert info["prestaged"]                                          # so the inputs are staged ahead
    # operations of one layout share table rows by default (q/k/v + o and the down projections of two layers
    # at a time); neighbours only (q/k/v + o of a layer) and every operation in a row of its own must give
    # the same bits
    monkeypatch.setenv("OXH_PLAN_MERGE", "1")
    neighbours = mv.Plan(d.plan_ops())
    monkeypatch.setenv("OXH_PLAN_MERGE", "0")
    apart = mv.Plan(d.plan_ops())
    monkeypatch.delenv("OXH_PLAN_MERGE")
    assert apart.info()["table_rows"] == 4 * layers and neighbours.info()["table_rows"] == 3 * layers
    assert info["table_rows"] < 3 * layers
    for rep in range(2):
        for p in (plan, neighbours, apart):
            for l in range(layers):
                for op in range(4):
                    mv.lib().oxh_memset(ctypes.c_void_p(d.out[l][op].ptr), 0xFF, d.out[l][op].nbytes, None)
                    mv.lib().oxh_memset(ctypes.c_void_p(d.act[l][op].ptr), 0xFF, d.act[l][op].nbytes, None)
            p.launch()
            assert p.status() == 0
            for l in range(layers):
                for op in range(4):
                    assert np.array_equal(bits(d.output(l, op)), bits(want_out[l][op])), (rep, l, op)
                    assert np.array_equal(d.activation(l, op), want_act[l][op]), (rep, l, op)
    apart.destroy()
    neighbours.destroy()
    # and one matrix against the oracle directly
    o = oxlibs.oracle()
    name, qt, rows, cols, _ = d.ops[3]
    w, x = d.host[(0, 3, 0)], d.x_host[(0, 3)]
    want = np.zeros(rows[0], np.float32)
    tmp = np.zeros(cols, np.float32)
    assert o.oxo_matvec_quantized(qt, w.ctypes.data, rows[0], cols, synth.row_bytes(qt, cols), x.ctypes.data,
                                  want.ctypes.data, tmp.ctypes.data) == 0
    assert np.array_equal(bits(d.output(0, 3)), bits(want))
    plan.destroy()


def chain_state(c):
    d = c.d
    return dict(qkv=c.qkv.download(np.float32, d.hidden + 2 * d.kv), o=c.o.download(np.float32, d.hidden),
                h=c.h.download(np.float32, d.ffn), f=c.f.download(np.float32, d.hidden),
                x=c.last_x.download(np.float32, d.hidden),
                res=[r.download(np.float32, d.hidden) for r in c.res])


@pytest.mark.parametrize("hidden,kv,ffn,layers", [(1024, 256, 2816, 4), (4096, 1024, 14336, 3), (5120, 1024, 8192, 2), (16384, 1024, 2048, 2)])
def test_dependent_chain_matches_single_launches(oxh, hidden, kv, ffn, layers):
    d = DecodeSet(hidden=hidden, kv=kv, ffn=ffn, layers=layers, seed=5)
    a, b = DecodeChain(d, seed=5), DecodeChain(d, seed=5)
    a.launch_step()
    mv.sync()
    want = chain_state(a)
    assert np.all(np.isfinite(want["x"])) and float(np.abs(want["f"]).max()) > 0
    plan = mv.Plan(b.plan_ops())
    info = plan.info()
    assert info["n_ops"] == 4 * layers
    assert info["n_waits"] == 4 * layers - 1          # every operation but the first reads its predecessor's output
    for rep in range(3):                              # the progress counters carry over from launch to launch
        plan.launch()
        assert plan.status() == 0
        got = chain_state(b)
        for k in ("qkv", "o", "h", "f", "x"):
            assert np.array_equal(bits(got[k]), bits(want[k])), (rep, k)
        for i in range(3):
            assert np.array_equal(bits(got["res"][i]), bits(want["res"][i])), (rep, i)
    # replayed from a graph, with eager work in between
    with mv.Graph() as g:
        plan.launch()
    for rep in range(3):
        mv.lib().oxh_memset(ctypes.c_void_p(b.f.ptr), 0, b.f.nbytes, None)
        g.launch()
        assert plan.status() == 0
        got = chain_state(b)
        assert np.array_equal(bits(got["f"]), bits(want["f"])) and np.array_equal(bits(got["x"]), bits(want["x"]))
    plan.destroy()


def test_mixed_types_with_q5k(oxh):
    """Q5_K operations take the kernel variant that carries the fifth-bit plane."""
    hidden, rows = 1024, 700
    xs = [mv.DeviceBuffer.from_host(synth.normal(hidden, seed=9, stream=i)) for i in range(3)]
    ws, outs, ops, host = [], [], [], []
    for i, qt in enumerate((Q5K, Q4K, Q6K)):
        w = synth.weights(qt, rows, hidden, seed=9, stream=10 + i)
        host.append(w)
        ws.append(mv.DeviceBuffer.from_host(w))
        outs.append(mv.DeviceBuffer(rows * 4))
        ops.append(dict(qtype=qt, segs=mv.make_segments([(ws[i].ptr, outs[i].ptr, rows, 0)]), cols=hidden,
                        d_x=xs[i].ptr))
    plan = mv.Plan(ops)
    plan.launch()
    assert plan.status() == 0
    o = oxlibs.oracle()
    for i, qt in enumerate((Q5K, Q4K, Q6K)):
        x = synth.normal(hidden, seed=9, stream=i)
        want = np.zeros(rows, np.float32)
        tmp = np.zeros(hidden, np.float32)
        assert o.oxo_matvec_quantized(qt, host[i].ctypes.data, rows, hidden, synth.row_bytes(qt, hidden),
                                      x.ctypes.data, want.ctypes.data, tmp.ctypes.data) == 0
        assert np.array_equal(bits(outs[i].download(np.float32, rows)), bits(want)), qt


@pytest.mark.parametrize("hidden,ffn", [(1024, 3072), (5120, 8192), (16384, 4096)])
def test_prestaged_plan_follows_its_inputs_from_launch_to_launch(oxh, monkeypatch, hidden, ffn):
    """A plan of independent operations keeps every staged input in memory of its own and re-reads it in
    every workgroup: new input values before a launch must reach every output of that launch (nothing
    may come from a cache line or an image of the launch before), with and without prologues, and the
    chained kernel must give the same bits for the same plan.  The longer vectors have more than
    sixteen blocks: a normalising prologue then sums squares over several blocks per lane, in the
    launches' order."""
    eps = 1e-5
    shapes = [(Q4K, 1800, hidden, None), (Q6K, 1024, ffn, None), (Q4K, 2 * 1536, hidden, "rms"),
              (Q5K, 640, hidden, "add_rms"), (Q6K, 512, hidden, "swiglu"), (Q4K, 777, hidden, None)]
    bufs, ops = [], []
    for i, (qt, rows, cols, pro) in enumerate(shapes):
        w = mv.DeviceBuffer.from_host(synth.weights(qt, rows, cols, seed=21, stream=i))
        b = dict(w=w, x=mv.DeviceBuffer(cols * 4), out=mv.DeviceBuffer(rows * 4), act=mv.DeviceBuffer(mv.act_bytes(qt, cols)),
                 g=mv.DeviceBuffer.from_host((synth.normal(cols, seed=21, stream=100 + i) * np.float32(0.1) + np.float32(1)).astype(np.float32)),
                 add=mv.DeviceBuffer(cols * 4), pout=mv.DeviceBuffer(cols * 4), sout=mv.DeviceBuffer(cols * 4))
        if pro == "rms" and i == 2:        # a gate/up pair
            half = rows // 2
            segs = mv.make_segments([(w.ptr, b["out"].ptr, half, 0, 0, w.ptr + half * synth.row_bytes(qt, cols))])
        else:
            segs = mv.make_segments([(w.ptr, b["out"].ptr, rows, 0)])
        op = dict(qtype=qt, segs=segs, cols=cols, d_x=b["x"].ptr, d_act_out=b["act"].ptr)
        if pro == "rms":
            op.update(kind=mv.PRO_RMSNORM, d_b=b["g"].ptr, eps=eps, d_pro_out=b["pout"].ptr)
        elif pro == "add_rms":
            op.update(kind=mv.PRO_RMSNORM, d_b=b["g"].ptr, eps=eps, d_add=b["add"].ptr, d_sum_out=b["sout"].ptr,
                      d_pro_out=b["pout"].ptr)
        elif pro == "swiglu":
            op.update(kind=mv.PRO_SWIGLU, d_b=b["add"].ptr, d_pro_out=b["pout"].ptr)
        bufs.append(b)
        ops.append(op)
    plan = mv.Plan(ops)
    assert plan.info()["prestaged"]
    monkeypatch.setenv("OXH_PLAN_PRESTAGE", "0")
    chained = mv.Plan(ops)
    monkeypatch.delenv("OXH_PLAN_PRESTAGE")
    assert not chained.info()["prestaged"] and chained.info()["n_waits"] == 0

    def state():
        out = []
        for (qt, rows, cols, pro), b in zip(shapes, bufs):
            n_out = rows // 2 if (pro == "rms") else rows
            out.append((b["out"].download(np.float32, n_out), b["act"].download(np.uint8, mv.act_bytes(qt, cols)),
                        b["pout"].download(np.float32, cols), b["sout"].download(np.float32, cols)))
        return out

    def clear():
        for b in bufs:
            for k in ("out", "act", "pout", "sout"):
                mv.lib().oxh_memset(ctypes.c_void_p(b[k].ptr), 0xFF, b[k].nbytes, None)

    for rep in range(3):
        for i, ((qt, rows, cols, pro), b) in enumerate(zip(shapes, bufs)):
            b["x"].upload(synth.normal(cols, seed=50 + rep, stream=i))
            b["add"].upload(synth.normal(cols, seed=50 + rep, stream=40 + i))
        clear()
        for op in ops:          # the reference result: the same calls one by one
            if op.get("kind"):
                mv.gemv_segments_fused(op["qtype"], op["segs"], op["cols"], op["d_x"], op["cols"], op["kind"], op["d_b"],
                                       op.get("eps", 0.0), op.get("d_pro_out"), op["d_act_out"], 1, 0, None,
                                       d_add=op.get("d_add"), d_sum_out=op.get("d_sum_out"))
            else:
                mv.gemv_segments_f32(op["qtype"], op["segs"], op["cols"], op["d_x"], op["cols"], op["d_act_out"])
        mv.sync()
        want = state()
        for p in (plan, chained):
            clear()
            p.launch()
            assert p.status() == 0
            got = state()
            for i, (w_, g_) in enumerate(zip(want, got)):
                assert np.array_equal(bits(w_[0]), bits(g_[0])), (rep, i, "out")
                assert np.array_equal(w_[1], g_[1]), (rep, i, "act")
                assert np.array_equal(bits(w_[2]), bits(g_[2])), (rep, i, "prologue out")
                assert np.array_equal(bits(w_[3]), bits(g_[3])), (rep, i, "sum out")
    plan.destroy()
    chained.destroy()


def test_clock_stamps_run_the_stamped_kernels_with_the_same_bits(oxh):
    """The measurement hook swaps in the kernel variants that write clock stamps (the ordinary ones carry no
    stamp code): same outputs, and every workgroup leaves stamps for every operation."""
    hidden, kv, ffn, layers = 1024, 256, 2816, 2
    d = DecodeSet(hidden=hidden, kv=kv, ffn=ffn, layers=layers, seed=6)
    a, b = DecodeChain(d, seed=6), DecodeChain(d, seed=6)
    a.launch_step()
    mv.sync()
    want = chain_state(a)
    plan = mv.Plan(b.plan_ops())
    n_ops, grid = 4 * layers, plan.info()["workgroups"]
    stamps = mv.DeviceBuffer(n_ops * grid * 8 * 8)
    _lib.check(_lib.lib().oxh_memset(ctypes.c_void_p(stamps.ptr), 0, stamps.nbytes, None))
    plan.launch()                                       # the ordinary kernel
    assert plan.status() == 0
    assert not stamps.download(np.uint64, n_ops * grid * 8).any()
    _lib.check(_lib.lab().plan_stamps(plan.handle, ctypes.c_void_p(stamps.ptr)))
    for rep in range(2):
        plan.launch()                                   # the stamped one
        assert plan.status() == 0
        got = chain_state(b)
        for k in ("qkv", "o", "h", "f", "x"):
            assert np.array_equal(bits(got[k]), bits(want[k])), (rep, k)
    st = stamps.download(np.uint64, n_ops * grid * 8).reshape(n_ops, grid, 8)
    assert (st[:, :, 0] != 0).all()                     # slot 0: the operation's start, by every workgroup
    assert (st[1:, :, 0].astype(np.int64) - st[:-1, :, 0].astype(np.int64) > 0).all()   # in order
    _lib.check(_lib.lab().plan_stamps(plan.handle, None))
    plan.destroy()


def test_a_wait_that_cannot_be_satisfied_gives_up(oxh):
    """The waits expect one workgroup more than exist and may poll 300 times: every workgroup must leave,
    the launch must end, the status must say so, and the plan must work again afterwards."""
    d = DecodeSet(hidden=1024, kv=256, ffn=2816, layers=2, seed=7)
    a, b = DecodeChain(d, seed=7), DecodeChain(d, seed=7)
    a.launch_step()
    mv.sync()
    want = chain_state(a)
    plan = mv.Plan(b.plan_ops())
    plan.set_spin_limit(300, phantom_workgroup=True)
    plan.launch()
    assert plan.status() == _lib.ERR_TIMEOUT
    assert b"ran out of polls" in oxh.oxh_last_error()
    plan.set_spin_limit(4000000, phantom_workgroup=False)
    for rep in range(2):
        plan.launch()
        assert plan.status() == 0
        got = chain_state(b)
        assert np.array_equal(bits(got["f"]), bits(want["f"])) and np.array_equal(bits(got["x"]), bits(want["x"]))


def test_what_a_plan_declines(oxh):
    x = mv.DeviceBuffer(4 * 32768)
    w = mv.DeviceBuffer(1 << 20)
    out = mv.DeviceBuffer(4 * 64)
    seg = mv.make_segments([(w.ptr, out.ptr, 8, 0)])
    for qt, cols in ((25, 1024), (8, 1024), (Q4K, 32768), (Q4K, 1000)):       # IQ3_S, Q2_K: no plan; too wide; not whole blocks
        with pytest.raises(mv.OxhError) as e:
            mv.Plan([dict(qtype=qt, segs=seg, cols=cols, d_x=x.ptr)])
        assert e.value.status == mv.DECLINED
    # an operation storing over its own input
    with pytest.raises(mv.OxhError) as e:
        mv.Plan([dict(qtype=Q4K, segs=mv.make_segments([(w.ptr, x.ptr, 8, 0)]), cols=1024, d_x=x.ptr)])
    assert e.value.status == _lib.ERR_ARG


@pytest.mark.parametrize("seed", range(20))
def test_random_independent_plans_match_the_launches(oxh, seed):
    """Seeded random plans of independent operations: one to four segments of ragged sizes (fewer rows than
    waves, rows no multiple of anything), pairs, every kind a plan takes (the regrouped Q6_K included),
    vector lengths that make neighbours mergeable and not, prologues with side outputs; each operation is
    also launched on its own and every output, stored activation and side output compared bit for bit,
    on two launches with new inputs in between."""
    rng = np.random.default_rng(1000 + seed)
    G8 = mv.Q6_K_G8
    kinds = [Q4K, Q4K, Q5K, Q6K, G8]
    n_ops = int(rng.integers(3, 12))
    ops, bufs = [], []
    cols_choices = [256, 1024, 2048, 4096]
    cols = int(rng.choice(cols_choices))
    for i in range(n_ops):
        if rng.random() < 0.4:
            cols = int(rng.choice(cols_choices))          # else: same length as the neighbour (mergeable)
        qt = int(rng.choice(kinds))
        if qt == G8 and cols % 2048:
            qt = Q6K
        file_qt = Q6K if qt == G8 else qt
        rb = synth.row_bytes(file_qt, cols)
        n_seg = int(rng.integers(1, 5))
        paired = rng.random() < 0.25
        if paired:
            n_seg = min(n_seg, 2)
        seg_rows = [int(rng.choice([1, 3, 17, 100, 257, 1000, 2500, int(rng.integers(1, 3000))])) for _ in range(n_seg)]
        total = sum(seg_rows) * (2 if paired else 1)
        w_host = synth.weights(file_qt, total, cols, seed=seed, stream=100 + i)
        w = mv.DeviceBuffer.from_host(w_host)
        if qt == G8:
            g = mv.DeviceBuffer(w_host.nbytes)
            mv.q6_k_group(w.ptr, total, cols, g.ptr)
            mv.sync()
            w = g
        b = dict(w=w, x=mv.DeviceBuffer(cols * 4), add=mv.DeviceBuffer(cols * 4), out=mv.DeviceBuffer(sum(seg_rows) * 4),
                 act=mv.DeviceBuffer(mv.act_bytes(file_qt, cols)), pout=mv.DeviceBuffer(cols * 4), sout=mv.DeviceBuffer(cols * 4),
                 g=mv.DeviceBuffer.from_host((synth.normal(cols, seed=seed, stream=300 + i) * np.float32(0.1) + np.float32(1)).astype(np.float32)),
                 cols=cols, n_out=sum(seg_rows), act_bytes=mv.act_bytes(file_qt, cols))
        items, row, out_off = [], 0, 0
        for r in seg_rows:
            first = w.ptr + row * rb
            if paired:
                items.append((first, b["out"].ptr + out_off * 4, r, 0, 0, first + r * rb))
                row += 2 * r
            else:
                items.append((first, b["out"].ptr + out_off * 4, r, 0))
                row += r
            out_off += r
        op = dict(qtype=qt, segs=mv.make_segments(items), cols=cols, d_x=b["x"].ptr)
        if rng.random() < 0.5:
            op["d_act_out"] = b["act"].ptr
        pro = rng.random()
        if pro < 0.2:
            op.update(kind=mv.PRO_RMSNORM, d_b=b["g"].ptr, eps=1e-5, d_pro_out=b["pout"].ptr)
        elif pro < 0.35:
            op.update(kind=mv.PRO_RMSNORM, d_b=b["g"].ptr, eps=1e-5, d_add=b["add"].ptr, d_sum_out=b["sout"].ptr)
        elif pro < 0.45:
            op.update(kind=mv.PRO_SWIGLU, d_b=b["add"].ptr, d_pro_out=b["pout"].ptr)
        ops.append(op)
        bufs.append(b)
    plan = mv.Plan(ops)
    assert plan.info()["prestaged"]

    def state():
        return [(b["out"].download(np.float32, b["n_out"]), b["act"].download(np.uint8, b["act_bytes"]),
                 b["pout"].download(np.float32, b["cols"]), b["sout"].download(np.float32, b["cols"])) for b in bufs]

    def clear():
        for b in bufs:
            for k in ("out", "act", "pout", "sout"):
                mv.lib().oxh_memset(ctypes.c_void_p(b[k].ptr), 0xFF, b[k].nbytes, None)

    for rep in range(2):
        for i, b in enumerate(bufs):
            b["x"].upload(synth.normal(b["cols"], seed=seed * 10 + rep, stream=i))
            b["add"].upload(synth.normal(b["cols"], seed=seed * 10 + rep, stream=50 + i))
        clear()
        for op in ops:
            if op.get("kind"):
                mv.gemv_segments_fused(op["qtype"], op["segs"], op["cols"], op["d_x"], op["cols"], op["kind"], op["d_b"],
                                       op.get("eps", 0.0), op.get("d_pro_out"), op.get("d_act_out"), 1, 0, None,
                                       d_add=op.get("d_add"), d_sum_out=op.get("d_sum_out"))
            else:
                mv.gemv_segments_f32(op["qtype"], op["segs"], op["cols"], op["d_x"], op["cols"], op.get("d_act_out"))
        mv.sync()
        want = state()
        clear()
        plan.launch()
        assert plan.status() == 0
        for i, (w_, g_) in enumerate(zip(want, state())):
            for k, name in enumerate(("out", "act", "prologue out", "sum out")):
                a, c = np.ascontiguousarray(w_[k]).view(np.uint8), np.ascontiguousarray(g_[k]).view(np.uint8)
                assert np.array_equal(a, c), (seed, rep, i, name, ops[i]["qtype"], ops[i]["cols"])
    plan.destroy()


@pytest.mark.parametrize("qtype", [7, 3, 4, 5, 6, 18])
@pytest.mark.parametrize("hidden,kv,ffn,layers", [(896, 128, 4864, 3), (256, 64, 96, 2)])
def test_plan_over_a_32_value_format_matches_single_launches(oxh, qtype, hidden, kv, ffn, layers):
    """Operations of one 32-value format that do not depend on each other run as one launch whose
    workgroups share out the rows of all of them: outputs and stored activations bit for bit those of
    the launches one by one, launch after launch, and against the oracle for one matrix."""
    d = DecodeSet(hidden=hidden, kv=kv, ffn=ffn, layers=layers, seed=5, keep_host=(0,), qtypes=(qtype, qtype))
    d.launch_step()
    mv.sync()
    want_out = [[d.output(l, op) for op in range(4)] for l in range(layers)]
    want_act = [[d.activation(l, op) for op in range(4)] for l in range(layers)]
    plan = mv.Plan(d.plan_ops())
    info = plan.info()
    # the rows of all operations are cut into runs and dealt to the workgroups: at least a run per operation
    assert info["n_ops"] == 4 * layers and info["n_waits"] == 0 and info["table_rows"] >= 4 * layers
    for rep in range(3):
        for l in range(layers):
            for op in range(4):
                mv.lib().oxh_memset(ctypes.c_void_p(d.out[l][op].ptr), 0xFF, d.out[l][op].nbytes, None)
                mv.lib().oxh_memset(ctypes.c_void_p(d.act[l][op].ptr), 0xFF, d.act[l][op].nbytes, None)
        plan.launch()
        assert plan.status() == 0
        for l in range(layers):
            for op in range(4):
                assert np.array_equal(bits(d.output(l, op)), bits(want_out[l][op])), (rep, l, op)
                assert np.array_equal(d.activation(l, op), want_act[l][op]), (rep, l, op)
    plan.destroy()
    o = oxlibs.oracle()
    name, qt, rows, cols, _ = d.ops[3]
    w, x = d.host[(0, 3, 0)], d.x_host[(0, 3)]
    want = np.zeros(rows[0], np.float32)
    tmp = np.zeros(cols, np.float32)
    assert o.oxo_matvec_quantized(qt, w.ctypes.data, rows[0], cols, synth.row_bytes(qt, cols), x.ctypes.data,
                                  want.ctypes.data, tmp.ctypes.data) == 0
    assert np.array_equal(bits(want_out[0][3]), bits(want))


def test_plan_over_a_32_value_format_declines_a_dependency(oxh):
    """No workgroup waits for another in such a plan, so an operation that reads what an earlier one
    writes cannot be part of it; nor can one of another weight format."""
    rows, cols = 256, 256
    w = mv.DeviceBuffer.from_host(synth.weights(7, rows, cols, seed=1))
    x = mv.DeviceBuffer.from_host(synth.normal(cols, seed=1))
    y = mv.DeviceBuffer(rows * 4)
    z = mv.DeviceBuffer(rows * 4)
    first = dict(qtype=7, segs=mv.make_segments([(w.ptr, y.ptr, rows, 0)]), cols=cols, d_x=x.ptr, d_act_out=None)
    second = dict(qtype=7, segs=mv.make_segments([(w.ptr, z.ptr, rows, 0)]), cols=cols, d_x=y.ptr, d_act_out=None)
    with pytest.raises(mv.OxhError) as e:
        mv.Plan([first, second])
    assert e.value.status == mv.DECLINED
    w4 = mv.DeviceBuffer.from_host(synth.weights(13, rows, cols, seed=1))
    other = dict(qtype=13, segs=mv.make_segments([(w4.ptr, z.ptr, rows, 0)]), cols=cols, d_x=x.ptr, d_act_out=None)
    with pytest.raises(mv.OxhError) as e:
        mv.Plan([first, other])
    assert e.value.status == mv.DECLINED
    independent = dict(qtype=7, segs=mv.make_segments([(w.ptr, z.ptr, rows, 0)]), cols=cols, d_x=x.ptr, d_act_out=None)
    plan = mv.Plan([first, independent])
    plan.launch()
    assert plan.status() == 0
    a, b = y.download(np.float32, rows), z.download(np.float32, rows)
    assert np.array_equal(bits(a), bits(b)) and np.any(a != 0)
    plan.destroy()


@pytest.mark.parametrize("qtype", [7, 5])
def test_plan_over_a_32_value_format_with_several_runs_of_one_input_per_workgroup(oxh, qtype):
    """300 000 short rows: every workgroup gets three runs of the one operation (a run is at most 16 x 32
    rows) and stages the input once; a second operation over another input follows in the same launch."""
    rows, cols = 300000, 32
    w = mv.DeviceBuffer.from_host(synth.weights(qtype, rows, cols, seed=9))
    xs = [mv.DeviceBuffer.from_host(synth.normal(cols, seed=10 + k)) for k in range(2)]
    want = []
    for k in range(2):
        o = mv.DeviceBuffer(rows * 4)
        mv.gemv_segments_f32(qtype, mv.make_segments([(w.ptr, o.ptr, rows, 0)]), cols, xs[k].ptr, cols, None, 1, rows)
        want.append(o.download(np.float32, rows))
        o.free()
    outs = [mv.DeviceBuffer(rows * 4) for _ in range(2)]
    plan = mv.Plan([dict(qtype=qtype, segs=mv.make_segments([(w.ptr, outs[k].ptr, rows, 0)]), cols=cols,
                         d_x=xs[k].ptr, d_act_out=None) for k in range(2)])
    assert plan.info()["table_rows"] > 2 * 256
    for rep in range(2):
        for o in outs:
            mv.lib().oxh_memset(ctypes.c_void_p(o.ptr), 0xFF, o.nbytes, None)
        plan.launch()
        assert plan.status() == 0
        for k in range(2):
            assert np.array_equal(bits(outs[k].download(np.float32, rows)), bits(want[k])), (rep, k)
    assert np.any(want[0] != want[1])
    plan.destroy()


@pytest.mark.parametrize("seed", range(12))
def test_random_plans_over_a_32_value_format_match_the_launches(oxh, seed):
    """Seeded random plans over one of the six 32-value formats: one to six segments of ragged sizes (a
    single row, fewer rows than waves, more rows than a run holds), vector lengths from one block to 150,
    some operations sharing an input, some storing their quantised activation; each operation is also
    launched on its own and every output and stored activation compared bit for bit, on two launches with
    new inputs in between."""
    rng = np.random.default_rng(7000 + seed)
    qt = int([7, 3, 4, 5, 6, 18][seed % 6])
    n_ops = int(rng.integers(2, 14))
    ops, bufs = [], []
    shared_x = None
    for i in range(n_ops):
        cols = 32 * int(rng.choice([1, 3, 28, 64, 128, 150]))
        rb = synth.row_bytes(qt, cols)
        n_seg = int(rng.integers(1, 7))
        seg_rows = [int(rng.choice([1, 5, 17, 100, 700, 3000, int(rng.integers(1, 9000))])) for _ in range(n_seg)]
        total = sum(seg_rows)
        w = mv.DeviceBuffer.from_host(synth.weights(qt, total, cols, seed=seed, stream=100 + i))
        if shared_x is not None and shared_x[1] == cols and rng.random() < 0.5:
            x = shared_x[0]
        else:
            x = mv.DeviceBuffer(cols * 4)
            shared_x = (x, cols)
        b = dict(w=w, x=x, out=mv.DeviceBuffer(total * 4), act=mv.DeviceBuffer(mv.act_bytes(qt, cols)), cols=cols,
                 n_out=total, store=rng.random() < 0.5)
        items, row = [], 0
        for r in seg_rows:
            items.append((w.ptr + row * rb, b["out"].ptr + row * 4, r, 0))
            row += r
        b["segs"] = mv.make_segments(items)
        ops.append(dict(qtype=qt, segs=b["segs"], cols=cols, d_x=x.ptr, d_act_out=b["act"].ptr if b["store"] else None))
        bufs.append(b)
    plan = mv.Plan(ops)
    assert plan.info()["n_ops"] == n_ops and plan.info()["n_waits"] == 0
    for rep in range(2):
        seen = set()
        for i, b in enumerate(bufs):
            if b["x"].ptr not in seen:
                b["x"].upload(synth.normal(b["cols"], seed=seed, stream=500 + 20 * rep + i))
                seen.add(b["x"].ptr)
        want = []
        for b in bufs:
            mv.lib().oxh_memset(ctypes.c_void_p(b["act"].ptr), 0xEE, b["act"].nbytes, None)
            mv.gemv_segments_f32(qt, b["segs"], b["cols"], b["x"].ptr, b["cols"], b["act"].ptr, 1, 0)
            want.append((b["out"].download(np.float32, b["n_out"]), b["act"].download(np.uint8, b["act"].nbytes)))
        for b in bufs:
            mv.lib().oxh_memset(ctypes.c_void_p(b["out"].ptr), 0xFF, b["out"].nbytes, None)
            mv.lib().oxh_memset(ctypes.c_void_p(b["act"].ptr), 0xEE, b["act"].nbytes, None)
        plan.launch()
        assert plan.status() == 0
        for i, b in enumerate(bufs):
            assert np.array_equal(bits(b["out"].download(np.float32, b["n_out"])), bits(want[i][0])), (rep, i)
            got_act = b["act"].download(np.uint8, b["act"].nbytes)
            if b["store"]:
                assert np.array_equal(got_act, want[i][1]), (rep, i)
            else:
                assert np.all(got_act == 0xEE), (rep, i)
    plan.destroy()
