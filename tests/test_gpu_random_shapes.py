"""Seeded random launches of the device-resident layer against the oracle: any
weight type, one to four matrices per launch, each with its own run of
activations and its own count, ragged rows, padded output strides, with and
without a buffer for the quantised activations (with one, launches of several
activations run on the matrix cores).  Every output must carry the oracle's
bits; whatever lies between the rows of a padded output must stay untouched."""
import os

import numpy as np
import pytest

import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth

pytestmark = pytest.mark.gpu

TYPES = (3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20)
BASE = {17: 3, 19: 5, 20: 7, 9: 10, 11: 10, 12: 13, 14: 15}      # ids that share another id's layout
SHIFT = int(os.environ.get("OXH_TEST_SEED_SHIFT", "0"))           # other shapes from the same generators


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


@pytest.mark.parametrize("seed", range(144))
def test_random_launch(oxh, seed):
    rng = np.random.default_rng(1000 + seed + 100000 * SHIFT)
    qt = int(TYPES[seed % len(TYPES)])
    layout = BASE.get(qt, qt)
    group = synth.BLOCK_ELEMS[layout]
    blocks = int(rng.integers(1, 41 if group == 256 else 160))
    cols = blocks * group
    n_segs = int(rng.integers(1, 5))
    rows = [int(rng.integers(1, 300)) for _ in range(n_segs)]
    with_buffer = bool((seed // len(TYPES)) & 1)
    # with a buffer for the quantised activations these types run on the matrix cores, up to 16 per weight
    wide = with_buffer and (layout in (13, 15, 16) or group == 32)
    nvs = [int(rng.integers(1, 9)) for _ in range(n_segs)]
    if wide and group == 32 and blocks > 128:
        wide = False                             # sixteen staged activations of that width do not fit LDS
    if wide:
        nvs[0] = int(rng.integers(9, 17))
    firsts = [int(rng.integers(0, 4)) for _ in range(n_segs)]
    n_act = max(f + n for f, n in zip(firsts, nvs))
    pad = int(rng.integers(0, 3)) * 4
    ws = [synth.weights(layout, r, cols, seed=seed, stream=i) for i, r in enumerate(rows)]
    xs = synth.normal(n_act * cols, seed=seed, stream=77).reshape(n_act, cols)
    d_ws = [mv.DeviceBuffer.from_host(w) for w in ws]
    d_x = mv.DeviceBuffer.from_host(xs)
    d_act = mv.DeviceBuffer(n_act * mv.act_bytes(qt, cols)) if with_buffer else None
    items, at, areas = [], 0, []
    stride = max(rows) + pad                     # one out_stride applies to the whole launch
    total = sum(n * stride for n in nvs)
    d_out = mv.DeviceBuffer(total * 4)
    d_out.upload(np.full(total, -3.5, np.float32))
    for d_w, r, n, f in zip(d_ws, rows, nvs, firsts):
        items.append((d_w.ptr, d_out.ptr + at * 4, r, f, n))
        areas.append(at)
        at += n * stride
    mv.gemv_segments_f32(qt, mv.make_segments(items), cols, d_x.ptr, cols,
                         None if d_act is None else d_act.ptr, max(nvs), stride)
    mv.sync()
    got = d_out.download(np.float32, total)
    o = oxlibs.oracle()
    rb = synth.row_bytes(layout, cols)
    for w, r, n, f, at in zip(ws, rows, nvs, firsts, areas):
        area = got[at:at + n * stride].reshape(n, stride)
        assert np.all(area[:, r:] == -3.5), "written beyond the rows"
        for v in range(n):
            want = np.zeros(r, np.float32)
            temp = np.zeros(cols, np.float32)
            assert o.oxo_matvec_quantized(qt, w.ctypes.data, r, cols, rb, np.ascontiguousarray(xs[f + v]).ctypes.data,
                                          want.ctypes.data, temp.ctypes.data) == 0
            assert np.array_equal(bits(area[v, :r]), bits(want)), (qt, cols, r, n, f, v, with_buffer)


def oracle_rows(qt, layout, w, rows, cols, x):
    o = oxlibs.oracle()
    want = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert o.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, synth.row_bytes(layout, cols), x.ctypes.data,
                                  want.ctypes.data, temp.ctypes.data) == 0
    return want, temp


@pytest.mark.parametrize("seed", range(51))
def test_random_host_calls(oxh, seed):
    """The reference's four entry points on host arrays with random shapes: single,
    fused (shared input, possibly mixed types and empty matrices), multi-input,
    and batch (1..40 vectors, padded strides)."""
    rng = np.random.default_rng(5000 + seed + 100000 * SHIFT)
    qt = int(TYPES[seed % len(TYPES)])
    layout = BASE.get(qt, qt)
    group = synth.BLOCK_ELEMS[layout]
    cols = int(rng.integers(1, 25 if group == 256 else 100)) * group
    rb = synth.row_bytes(layout, cols)
    temp = np.zeros(cols, np.float32)
    which = seed % 3
    if which == 0:                                             # fused and multi-input
        n = int(rng.integers(1, 6))
        rows = [int(rng.integers(0, 200)) for _ in range(n)]
        qts = [qt] * n
        if seed % 2 and n > 1:                                 # one matrix of another type with the same block width
            other = 16 if group == 256 and layout != 16 else (7 if group == 32 and layout != 7 else qt)
            qts[-1] = other
        lays = [BASE.get(q, q) for q in qts]
        ws = [synth.weights(l, r, cols, seed=seed, stream=i) if r else np.zeros(1, np.uint8)
              for i, (l, r) in enumerate(zip(lays, rows))]
        rbs = [synth.row_bytes(l, cols) for l in lays]
        x = synth.normal(cols, seed=seed, stream=50)
        outs = [np.full(max(r, 1), -3.5, np.float32) for r in rows]
        assert mv.matvec_quantized_fused(qts, ws, rows, cols, rbs, x, outs, temp) == 0
        for q, l, w, r, out in zip(qts, lays, ws, rows, outs):
            if r:
                assert np.array_equal(bits(out[:r]), bits(oracle_rows(q, l, w, r, cols, x)[0]))
        xs = [synth.normal(cols, seed=seed, stream=60 + i) for i in range(n)]
        outs = [np.full(max(r, 1), -3.5, np.float32) for r in rows]
        assert mv.matvec_quantized_multi_input(qts, ws, rows, cols, rbs, xs, outs, temp) == 0
        for q, l, w, r, xv, out in zip(qts, lays, ws, rows, xs, outs):
            if r:
                assert np.array_equal(bits(out[:r]), bits(oracle_rows(q, l, w, r, cols, xv)[0]))
    else:                                                      # single and batch
        rows = int(rng.integers(1, 400))
        w = synth.weights(layout, rows, cols, seed=seed, stream=3)
        x = synth.normal(cols, seed=seed, stream=51)
        out = np.full(rows, -3.5, np.float32)
        assert mv.matvec_quantized(qt, w, rows, cols, rb, x, out, temp) == 0
        want, want_temp = oracle_rows(qt, layout, w, rows, cols, x)
        nact = mv.act_bytes(qt, cols)
        assert np.array_equal(temp.view(np.uint8)[:nact], want_temp.view(np.uint8)[:nact])
        assert np.array_equal(bits(out), bits(want))
        n_vec = int(rng.integers(1, 41))
        in_stride, out_stride = cols + int(rng.integers(0, 3)) * 8, rows + int(rng.integers(0, 3))
        xb = synth.normal(n_vec * in_stride, seed=seed, stream=52).reshape(n_vec, in_stride)
        ob = np.full((n_vec, out_stride), -3.5, np.float32)
        scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
        assert mv.matvec_quantized_batch(qt, w, rows, cols, rb, xb, in_stride, ob, out_stride, n_vec, temp,
                                         scratch) == 0
        assert np.all(ob[:, rows:] == -3.5)
        for v in rng.choice(n_vec, size=min(n_vec, 6), replace=False):
            want, _ = oracle_rows(qt, layout, w, rows, cols, np.ascontiguousarray(xb[v, :cols]))
            assert np.array_equal(bits(ob[v, :rows]), bits(want)), (qt, rows, cols, n_vec, int(v))


@pytest.mark.parametrize("seed", range(24))
def test_random_prefill_and_lookup(oxh, seed):
    """oxh_mmq (9..300 activations; Q4_K, Q5_K, Q6_K) with padded output stride, and
    oxh_get_rows over random ids for every type."""
    rng = np.random.default_rng(9000 + seed + 100000 * SHIFT)
    o = oxlibs.oracle()
    qt = (13, 15, 16, 12, 14)[seed % 5]
    layout = BASE.get(qt, qt)
    cols = int(rng.integers(1, 20)) * 256
    rows = int(rng.integers(1, 500))
    n_vec = int(rng.integers(9, 301))
    stride = rows + int(rng.integers(0, 3)) * 4
    w = synth.weights(layout, rows, cols, seed=seed, stream=1)
    xs = synth.normal(n_vec * cols, seed=seed, stream=2).reshape(n_vec, cols)
    d_w, d_x = mv.DeviceBuffer.from_host(w), mv.DeviceBuffer.from_host(xs)
    d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(qt, cols))
    d_o = mv.DeviceBuffer(n_vec * stride * 4)
    d_o.upload(np.full(n_vec * stride, -3.5, np.float32))
    mv.quantize(qt, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    mv.mmq(qt, d_w.ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, stride)
    mv.sync()
    got = d_o.download(np.float32, n_vec * stride).reshape(n_vec, stride)
    assert np.all(got[:, rows:] == -3.5)
    for v in list(rng.choice(n_vec, size=5, replace=False)) + [0, n_vec - 1]:
        want, _ = oracle_rows(qt, layout, w, rows, cols, np.ascontiguousarray(xs[v]))
        assert np.array_equal(bits(got[v, :rows]), bits(want)), (qt, rows, cols, n_vec, int(v))
    # embedding lookup, any type
    qt2 = int(TYPES[seed % len(TYPES)])
    lay2 = BASE.get(qt2, qt2)
    group = synth.BLOCK_ELEMS[lay2]
    cols2 = int(rng.integers(1, 12)) * (256 if group == 256 else 32 * int(rng.integers(1, 9)))
    rows2 = int(rng.integers(1, 200))
    rb2 = synth.row_bytes(lay2, cols2)
    w2 = synth.weights(lay2, rows2, cols2, seed=seed, stream=3)
    ids = rng.integers(0, rows2, size=int(rng.integers(1, 40))).astype(np.uint32)
    d_w2, d_ids = mv.DeviceBuffer.from_host(w2), mv.DeviceBuffer.from_host(ids)
    d_r = mv.DeviceBuffer(ids.size * cols2 * 4)
    mv.get_rows(qt2, d_w2.ptr, rows2, cols2, d_ids.ptr, ids.size, d_r.ptr, cols2)
    got = d_r.download(np.float32, ids.size * cols2).reshape(ids.size, cols2)
    for k, i in enumerate(ids):
        deq = np.zeros(cols2, np.float32)
        assert o.oxo_dequant_row(qt2, w2[int(i) * rb2:].ctypes.data, cols2, deq.ctypes.data) == 0
        assert np.array_equal(bits(got[k]), bits(deq)), (qt2, cols2, int(i))


@pytest.mark.parametrize("seed", range(51))
def test_random_fused_prologue_launch(oxh, seed):
    """RMSNorm, residual add + RMSNorm or SwiGLU in front of any weight type, one to three
    segments, one to four input vectors, optionally a paired gate/up segment.  The float
    step is read back from the device; from there on everything is exact: the quantised
    bytes, plain segments' outputs, and the two halves of a pair before silu(gate)*up."""
    rng = np.random.default_rng(7000 + seed + 100000 * SHIFT)
    o = oxlibs.oracle()
    qt = int(TYPES[seed % len(TYPES)])
    layout = BASE.get(qt, qt)
    group = synth.BLOCK_ELEMS[layout]
    cols = int(rng.integers(1, 17 if group == 256 else 60)) * group
    n_vec = int(rng.integers(1, 5))
    kind = ("rms", "add_rms", "swiglu")[seed % 3]
    n_segs = int(rng.integers(1, 4))
    rows = [int(rng.integers(1, 250)) for _ in range(n_segs)]
    paired = [bool(rng.integers(0, 2)) and seed % 4 == 0 for _ in range(n_segs)]
    ws = [synth.weights(layout, r, cols, seed=seed, stream=2 * i) for i, r in enumerate(rows)]
    w2 = [synth.weights(layout, r, cols, seed=seed, stream=2 * i + 1) if p else None
          for i, (r, p) in enumerate(zip(rows, paired))]
    xs = (synth.normal(n_vec * cols, seed=seed, stream=90) * np.float32(1.7)).reshape(n_vec, cols)
    b = synth.normal((n_vec if kind == "swiglu" else 1) * cols, seed=seed, stream=91)
    add = synth.normal(n_vec * cols, seed=seed, stream=92).reshape(n_vec, cols)
    d_ws = [mv.DeviceBuffer.from_host(w) for w in ws]
    d_w2 = [mv.DeviceBuffer.from_host(w) if w is not None else None for w in w2]
    d_x, d_b, d_add = mv.DeviceBuffer.from_host(xs), mv.DeviceBuffer.from_host(b), mv.DeviceBuffer.from_host(add)
    nact = mv.act_bytes(qt, cols)
    d_y, d_sum = mv.DeviceBuffer(n_vec * cols * 4), mv.DeviceBuffer(n_vec * cols * 4)
    d_a = mv.DeviceBuffer(n_vec * nact)
    stride = max(rows)
    d_o = mv.DeviceBuffer(n_segs * n_vec * stride * 4)
    items = [(d_w.ptr, d_o.ptr + i * n_vec * stride * 4, r, 0, 0, None if p is None else p.ptr)
             for i, (d_w, r, p) in enumerate(zip(d_ws, rows, d_w2))]
    eps = 1e-5
    mv.gemv_segments_fused(qt, mv.make_segments(items), cols, d_x.ptr, cols,
                           mv.PRO_SWIGLU if kind == "swiglu" else mv.PRO_RMSNORM, d_b.ptr, eps, d_y.ptr, d_a.ptr,
                           n_vec, stride, None, d_add.ptr if kind == "add_rms" else None,
                           d_sum.ptr if kind == "add_rms" else None)
    mv.sync()
    y = d_y.download(np.float32, n_vec * cols).reshape(n_vec, cols)
    acts = d_a.download(np.uint8, n_vec * nact).reshape(n_vec, nact)
    out = d_o.download(np.float32, n_segs * n_vec * stride).reshape(n_segs, n_vec, stride)
    for v in range(n_vec):                                      # the float step, to rounding
        want = np.zeros(cols, np.float32)
        if kind == "swiglu":
            o.oxo_swiglu_f32(xs[v].ctypes.data, b[v * cols:].ctypes.data, want.ctypes.data, cols)
        else:
            src = xs[v] + add[v] if kind == "add_rms" else xs[v]
            src = np.ascontiguousarray(src, np.float32)
            if kind == "add_rms":
                got_sum = d_sum.download(np.float32, n_vec * cols).reshape(n_vec, cols)[v]
                assert np.array_equal(bits(got_sum), bits(src))
            o.oxo_rms_norm_f32(src.ctypes.data, b.ctypes.data, want.ctypes.data, cols, eps)
        assert np.all(np.abs(y[v] - want) <= 4e-6 * np.abs(want) + 1e-30), (kind, v)
    for i, (w, wp, r) in enumerate(zip(ws, w2, rows)):          # the integer path, exactly
        for v in range(n_vec):
            yv = np.ascontiguousarray(y[v])
            want, temp = oracle_rows(qt, layout, w, r, cols, yv)
            assert np.array_equal(acts[v], temp.view(np.uint8)[:nact])
            if wp is None:
                assert np.array_equal(bits(out[i, v, :r]), bits(want)), (qt, kind, i, v)
            else:
                up, _ = oracle_rows(qt, layout, wp, r, cols, yv)
                h = np.zeros(r, np.float32)
                o.oxo_swiglu_f32(want.ctypes.data, up.ctypes.data, h.ctypes.data, r)
                assert np.all(np.abs(out[i, v, :r] - h) <= 4e-6 * np.abs(h) + 1e-30), (qt, kind, i, v)


def test_host_calls_from_several_threads(oxh):
    """Four threads call the host entry points at once (ctypes drops the interpreter lock during a
    call): the library serialises them on its shared staging buffers, and every result is still the
    oracle's to the bit.  Shapes differ per thread so that the staging buffers are regrown mid-run."""
    import threading
    jobs = []
    for t, (qt, rows, cols) in enumerate([(13, 300, 4096), (16, 150, 2048), (7, 257, 896), (10, 90, 5120)]):
        layout = BASE.get(qt, qt)
        w = synth.weights(layout, rows, cols, seed=900 + t)
        xs = [synth.normal(cols, seed=901, stream=10 * t + i) for i in range(6)]
        wants = [oracle_rows(qt, layout, w, rows, cols, x)[0] for x in xs]
        jobs.append((qt, rows, cols, synth.row_bytes(layout, cols), w, xs, wants))
    failures = []

    def worker(job):
        qt, rows, cols, rb, w, xs, wants = job
        temp = np.zeros(cols, np.float32)
        scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
        try:
            for rep in range(5):
                for x, want in zip(xs, wants):
                    out = np.full(rows, -3.5, np.float32)
                    assert mv.matvec_quantized(qt, w, rows, cols, rb, x, out, temp) == 0
                    assert np.array_equal(bits(out), bits(want))
                xb = np.stack(xs)
                ob = np.full((len(xs), rows), -3.5, np.float32)
                assert mv.matvec_quantized_batch(qt, w, rows, cols, rb, xb, cols, ob, rows, len(xs), temp,
                                                 scratch) == 0
                assert np.array_equal(bits(ob), bits(np.stack(wants)))
        except Exception as e:                                   # noqa: BLE001 - reported below
            failures.append((qt, repr(e)))

    threads = [threading.Thread(target=worker, args=(j,)) for j in jobs]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not failures, failures
