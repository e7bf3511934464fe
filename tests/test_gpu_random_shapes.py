"""Seeded random launches of the device-resident layer against the oracle: any
weight type, one to four matrices per launch, each with its own run of
activations and its own count, ragged rows, padded output strides, with and
without a buffer for the quantised activations (with one, launches of several
activations run on the matrix cores).  Every output must carry the oracle's
bits; whatever lies between the rows of a padded output must stay untouched."""
import numpy as np
import pytest

import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth

pytestmark = pytest.mark.gpu

TYPES = (3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 19, 20)
BASE = {17: 3, 19: 5, 20: 7, 9: 10, 11: 10, 12: 13, 14: 15}      # ids that share another id's layout


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


@pytest.mark.parametrize("seed", range(136))
def test_random_launch(oxh, seed):
    rng = np.random.default_rng(1000 + seed)
    qt = int(TYPES[seed % len(TYPES)])
    layout = BASE.get(qt, qt)
    group = synth.BLOCK_ELEMS[layout]
    blocks = int(rng.integers(1, 41 if group == 256 else 160))
    cols = blocks * group
    n_segs = int(rng.integers(1, 5))
    rows = [int(rng.integers(1, 300)) for _ in range(n_segs)]
    nvs = [int(rng.integers(1, 9)) for _ in range(n_segs)]
    firsts = [int(rng.integers(0, 4)) for _ in range(n_segs)]
    n_act = max(f + n for f, n in zip(firsts, nvs))
    pad = int(rng.integers(0, 3)) * 4
    with_buffer = bool(seed & 1)
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
