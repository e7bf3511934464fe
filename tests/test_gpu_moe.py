"""Mixture-of-experts feed-forward with the routing on the device
(oxh_moe_route, oxh_moe_ffn) against the oracle.

Two bars, as everywhere a float step sits in front of the integer path:
  * expert ids, counts, offsets, the sorted order and the quantised bytes of the
    gathered tokens are exact; gate and up are bit-identical to the oracle's
    matvec of that token through that expert; the down outputs are bit-identical
    to the oracle's dot over the device's own quantised silu(gate)*up; the
    combination is bit-identical to the ascending-expert sum of the device's
    own weights and down outputs;
  * gate weights, silu(gate)*up and the layer's output agree with the oracle's
    whole layer to float rounding (the device's expf is not libm's).
"""
import ctypes

import numpy as np
import pytest

import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth

pytestmark = pytest.mark.gpu
Q4K, Q5K, Q6K = 13, 15, 16


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def group(ids, n_expert):
    """counting sort by expert, token order kept (llama.c:6060-6069)"""
    n_tok, k = ids.shape
    counts = np.bincount(ids.ravel(), minlength=n_expert).astype(np.uint32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32)
    fill = offsets[:-1].astype(np.int64).copy()
    perm = np.zeros(n_tok * k, np.uint32)
    slot = np.zeros(n_tok * k, np.uint32)
    for t in range(n_tok):
        for j in range(k):
            e = ids[t, j]
            perm[fill[e]] = t
            slot[t * k + j] = fill[e]
            fill[e] += 1
    return counts, offsets, perm, slot


@pytest.mark.parametrize("n_tok,n_exp,k,renorm", [(1, 8, 2, 1), (16, 8, 2, 1), (100, 32, 8, 0), (1500, 3, 1, 1),
                                                  (37, 16, 4, 1), (5, 2, 2, 0), (4096, 8, 2, 1), (300, 64, 8, 1),
                                                  (9, 60, 4, 0)])
def test_route_and_grouping(oxh, n_tok, n_exp, k, renorm):
    o = oxlibs.oracle()
    logits = synth.normal(n_tok * n_exp, seed=n_tok, stream=4242).reshape(n_tok, n_exp)
    if n_exp > 2:
        logits[:, 1] = -40.0                                  # an expert that gets no token
    d_l = mv.DeviceBuffer.from_host(logits)
    n = n_tok * k
    d = {name: mv.DeviceBuffer(4 * size) for name, size in (("ids", n), ("wts", n), ("counts", n_exp),
                                                          ("offsets", n_exp + 1), ("perm", n), ("slot", n))}
    mv.moe_route(d_l.ptr, n_tok, n_exp, k, renorm, d["ids"].ptr, d["wts"].ptr, d["counts"].ptr, d["offsets"].ptr,
                 d["perm"].ptr, d["slot"].ptr)
    mv.sync()
    ids = d["ids"].download(np.int32, n).reshape(n_tok, k)
    wts = d["wts"].download(np.float32, n).reshape(n_tok, k)
    want_ids = np.zeros((n_tok, k), np.int32)
    want_w = np.zeros((n_tok, k), np.float32)
    o.oxo_moe_route(logits.ctypes.data, n_tok, n_exp, k, renorm, want_ids.ctypes.data, want_w.ctypes.data)
    assert np.array_equal(ids, want_ids)
    assert np.allclose(wts, want_w, rtol=2e-6, atol=1e-30)
    counts, offsets, perm, slot = group(ids, n_exp)
    assert np.array_equal(d["counts"].download(np.uint32, n_exp), counts)
    assert np.array_equal(d["offsets"].download(np.uint32, n_exp + 1), offsets)
    assert np.array_equal(d["perm"].download(np.uint32, n), perm)
    assert np.array_equal(d["slot"].download(np.uint32, n), slot)
    if n_exp > 2 and k < n_exp - 1:
        assert counts[1] == 0


def test_route_ties_follow_the_swapping_selection(oxh):
    """Equal probabilities: the reference's selection sort swaps index-list
    entries as it goes, so the winner among equals is the earliest in the
    current list.  [0, 0, 0, 5] with k = 3: expert 3 first, which moves expert 0
    to the end of the list, so the tie then goes to 1 and 2 (worked by hand from
    llama.c:5998-6012), not to 0 and 1."""
    o = oxlibs.oracle()
    rows = [[0, 0, 0, 5], [5, 0, 0, 0], [0, 5, 0, 0], [1, 1, 1, 1], [0, 2, 2, 0], [3, 0, 3, 0]]
    logits = np.array(rows, np.float32)
    rng = np.random.default_rng(3)
    many = np.round(rng.normal(size=(300, 4)) * 1.2).astype(np.float32)      # plenty of equal logits
    logits = np.concatenate([logits, many])
    n_tok, n_exp, k = logits.shape[0], 4, 3
    want = np.zeros((n_tok, k), np.int32)
    want_w = np.zeros((n_tok, k), np.float32)
    o.oxo_moe_route(logits.ctypes.data, n_tok, n_exp, k, 1, want.ctypes.data, want_w.ctypes.data)
    assert list(want[0]) == [3, 1, 2] and list(want[1]) == [0, 1, 2] and list(want[2]) == [1, 0, 2]
    assert list(want[3]) == [0, 1, 2] and list(want[4]) == [1, 2, 0] and list(want[5]) == [0, 2, 1]
    d_l = mv.DeviceBuffer.from_host(logits)
    n = n_tok * k
    d = [mv.DeviceBuffer(4 * max(n, n_exp + 1)) for _ in range(6)]
    mv.moe_route(d_l.ptr, n_tok, n_exp, k, 1, *[b.ptr for b in d])
    mv.sync()
    assert np.array_equal(d[0].download(np.int32, n).reshape(n_tok, k), want)
    assert np.allclose(d[1].download(np.float32, n).reshape(n_tok, k), want_w, rtol=2e-6)


def dot_fn(qt):
    o = oxlibs.oracle()
    if qt == Q6K:
        return lambda row, blocks, act: o.oxo_dot_q6_k_q8_k(row, blocks, act, None)
    f = o.oxo_dot_q5_k_q8_k if qt == Q5K else o.oxo_dot_q4_k_q8_k
    return lambda row, blocks, act: f(row, blocks, act, None, None)


def check_layer(qt_gu, qt_dn, n_exp, k, hidden, ffn, n_tok, seed, renorm=1, skew=True, sample=None, replay=False):
    o = oxlibs.oracle()
    rb_gu, rb_dn = synth.row_bytes(qt_gu, hidden), synth.row_bytes(qt_dn, ffn)
    wg = synth.weights(qt_gu, n_exp * ffn, hidden, seed=seed, stream=1, sigma=0.02)
    wu = synth.weights(qt_gu, n_exp * ffn, hidden, seed=seed, stream=2, sigma=0.02)
    wd = synth.weights(qt_dn, n_exp * hidden, ffn, seed=seed, stream=3, sigma=0.02)
    logits = synth.normal(n_tok * n_exp, seed=seed, stream=4).reshape(n_tok, n_exp)
    if skew:
        logits[:, n_exp - 1] = -40.0                          # nobody selects the last expert
        logits[:, 0] += 2.0                                   # and the first one is popular
    x = synth.normal(n_tok * hidden, seed=seed, stream=5).reshape(n_tok, hidden)
    d_wg, d_wu, d_wd = (mv.DeviceBuffer.from_host(a) for a in (wg, wu, wd))
    d_l, d_x = mv.DeviceBuffer.from_host(logits), mv.DeviceBuffer.from_host(x)
    d_out = mv.DeviceBuffer(n_tok * hidden * 4)
    layer = mv.MoeLayer(qt_gu, qt_dn, d_wg.ptr, d_wu.ptr, d_wd.ptr, n_exp, k, hidden, ffn, renorm, max_tok=n_tok)
    if replay:
        layer.forward(d_l.ptr, d_x.ptr, n_tok, d_out.ptr)     # warm: every kernel loaded before capture
        mv.sync()
        with mv.Graph() as g:
            layer.forward(d_l.ptr, d_x.ptr, n_tok, d_out.ptr)
        first = None
        for _ in range(3):
            mv.lib().oxh_memset(ctypes.c_void_p(d_out.ptr), 0xFF, d_out.nbytes, None)
            mv.sync()
            g.launch()
            mv.sync()
            got = d_out.download(np.float32, n_tok * hidden)
            first = got if first is None else first
            assert np.array_equal(bits(got), bits(first))
        g.destroy()
    layer.forward(d_l.ptr, d_x.ptr, n_tok, d_out.ptr)
    mv.sync()
    out = d_out.download(np.float32, n_tok * hidden).reshape(n_tok, hidden)
    if replay:
        assert np.array_equal(bits(out.ravel()), bits(first))
    P = layer.parts(n_tok)
    n = n_tok * k
    ws = layer.workspace
    ids = ws.download(np.int32, n, P["ids"]).reshape(n_tok, k)
    wts = ws.download(np.float32, n, P["wts"]).reshape(n_tok, k)
    slot = ws.download(np.uint32, n, P["slot_pos"])
    perm = ws.download(np.uint32, n, P["perm"])
    counts = ws.download(np.uint32, n_exp, P["counts"])
    offsets = ws.download(np.uint32, n_exp + 1, P["offsets"])
    ab_x, ab_h = mv.act_bytes(qt_gu, hidden), mv.act_bytes(qt_dn, ffn)
    act_x = ws.download(np.uint8, n * ab_x, P["act_x"]).reshape(n, ab_x)
    act_h = ws.download(np.uint8, n * ab_h, P["act_h"]).reshape(n, ab_h)
    gate = ws.download(np.float32, n * ffn, P["gate"]).reshape(n, ffn)
    up = ws.download(np.float32, n * ffn, P["up"]).reshape(n, ffn)
    y = ws.download(np.float32, n * hidden, P["y"]).reshape(n, hidden)

    # routing and grouping: exact
    want_ids = np.zeros((n_tok, k), np.int32)
    want_w = np.zeros((n_tok, k), np.float32)
    o.oxo_moe_route(logits.ctypes.data, n_tok, n_exp, k, renorm, want_ids.ctypes.data, want_w.ctypes.data)
    assert np.array_equal(ids, want_ids)
    assert np.allclose(wts, want_w, rtol=2e-6)
    c2, o2, p2, s2 = group(ids, n_exp)
    assert np.array_equal(counts, c2) and np.array_equal(offsets, o2)
    assert np.array_equal(perm, p2) and np.array_equal(slot, s2)
    if skew and k < n_exp - 1:
        assert counts[n_exp - 1] == 0 and counts[0] == counts.max()

    expert_of = np.repeat(np.arange(n_exp), counts)
    pairs = range(n) if sample is None else sample(n, offsets)
    dgu, ddn = dot_fn(qt_gu), dot_fn(qt_dn)
    rows_gu = range(ffn) if sample is None else range(0, ffn, 97)
    rows_dn = range(hidden) if sample is None else range(0, hidden, 53)
    for pidx in pairs:
        e, t = int(expert_of[pidx]), int(perm[pidx])
        # gathered token, quantised: exact
        want_act = np.zeros(ab_x, np.uint8)
        o.oxo_quantize_q8_k(x[t].ctypes.data, hidden, want_act.ctypes.data)
        assert np.array_equal(act_x[pidx], want_act), (pidx, e, t)
        # gate, up: the oracle's matvec bits for this token through this expert
        for name, w, got in (("gate", wg, gate), ("up", wu, up)):
            for r in rows_gu:
                row = w[(e * ffn + r) * rb_gu:]
                v = np.float32(dgu(row.ctypes.data, hidden // 256, want_act.ctypes.data))
                assert bits(got[pidx, r:r + 1])[0] == bits(np.array([v]))[0], (name, pidx, e, r)
        # silu(gate)*up: a float step; its quantised form within one code of the oracle's
        h = np.zeros(ffn, np.float32)
        o.oxo_swiglu_f32(gate[pidx].ctypes.data, up[pidx].ctypes.data, h.ctypes.data, ffn)
        want_h = np.zeros(ab_h, np.uint8)
        o.oxo_quantize_q8_k(h.ctypes.data, ffn, want_h.ctypes.data)
        for b in range(ffn // 256):
            blk_g, blk_w = act_h[pidx, b * 292:(b + 1) * 292], want_h[b * 292:(b + 1) * 292]
            dg, dw = blk_g[:4].view(np.float32)[0], blk_w[:4].view(np.float32)[0]
            assert abs(dg - dw) <= 4e-6 * abs(dw)
            assert np.abs(blk_g[4:260].view(np.int8).astype(int) - blk_w[4:260].view(np.int8).astype(int)).max() <= 1
        # down: exact over the device's own activation bytes
        dev_h = np.ascontiguousarray(act_h[pidx])
        for r in rows_dn:
            row = wd[(e * hidden + r) * rb_dn:]
            v = np.float32(ddn(row.ctypes.data, ffn // 256, dev_h.ctypes.data))
            assert bits(y[pidx, r:r + 1])[0] == bits(np.array([v]))[0], ("down", pidx, e, r)
    # combination: ascending expert order, one product and one addition per step
    want_out = np.zeros((n_tok, hidden), np.float32)
    for t in range(n_tok):
        for j in np.argsort(ids[t], kind="stable"):
            want_out[t] = want_out[t] + wts[t, j] * y[slot[t * k + j]]
    assert np.array_equal(bits(out), bits(want_out))
    return dict(wg=wg, wu=wu, wd=wd, logits=logits, x=x, out=out)


@pytest.mark.parametrize("qt_gu,qt_dn", [(Q4K, Q4K), (Q4K, Q6K), (Q5K, Q6K), (Q6K, Q5K)])
@pytest.mark.parametrize("n_tok", [1, 5, 40])
def test_layer_stage_by_stage(oxh, qt_gu, qt_dn, n_tok):
    """4 experts, top-2; with 40 tokens the popular expert gets more than two
    16-token tiles and the last expert none."""
    r = check_layer(qt_gu, qt_dn, 4, 2, 512, 768, n_tok, seed=11 + n_tok)
    o = oxlibs.oracle()
    whole = np.zeros_like(r["out"])
    assert o.oxo_moe_ffn(qt_gu, qt_dn, r["wg"].ctypes.data, r["wu"].ctypes.data, r["wd"].ctypes.data, 4, 2, 512,
                         768, 1, r["logits"].ctypes.data, r["x"].ctypes.data, n_tok, whole.ctypes.data) == 0
    # whole layer: the device's expf against libm's moves a quantised code by one here and there
    scale = np.abs(whole).max()
    assert np.abs(r["out"] - whole).max() <= 2e-3 * scale


def test_layer_top1_and_all_experts(oxh):
    check_layer(Q4K, Q4K, 3, 1, 256, 256, 9, seed=3, renorm=0, skew=False)
    check_layer(Q4K, Q6K, 16, 8, 256, 512, 6, seed=4, renorm=1, skew=False)


@pytest.mark.parametrize("qt_gu,qt_dn", [(Q4K, Q6K), (Q5K, Q4K), (Q6K, Q5K)])
def test_layer_with_prefill_sized_token_counts(oxh, qt_gu, qt_dn):
    """150 pairs per expert on average: the expert launches take the 128-row x 64-token tile and walk
    three token tiles per expert, the popular expert more."""
    check_layer(qt_gu, qt_dn, 4, 2, 512, 768, 300, seed=21, sample=lambda n, offsets: sorted(
        set(int(v) for v in offsets[:-1] if v < n) | set(int(v) - 1 for v in offsets[1:] if v > 0) |
        set(range(0, n, 37))))


@pytest.mark.parametrize("qt_gu,qt_dn", [(Q4K, Q4K), (Q4K, Q6K), (Q6K, Q5K)])
def test_layer_whose_down_projection_gives_two_workgroups_per_cu(oxh, qt_gu, qt_dn):
    """8 experts x 4096 output rows: 512 workgroups of the 64-row tile (two per CU on a 256-CU device), which
    then stage two super-blocks per barrier; likewise 9 experts x 3584 rows.  (With OXH_MOE_WIDE_SMALL=1 a
    Q4_K down launch of this size runs on 128-row tiles of eight waves instead: the test below.)"""
    check_layer(qt_gu, qt_dn, 8, 2, 4096, 256, 16, seed=31, skew=False)
    check_layer(qt_gu, qt_dn, 9, 3, 3584, 512, 9, seed=32, skew=True)


def test_the_128_row_tile_when_switched_on(oxh):
    """OXH_MOE_WIDE_SMALL=1 is read once per process: the layers above, the Mixtral-shaped layer and
    configuration 4's expert launches over host-made lists, in a process of their own with the switch on,
    against the same oracle checks."""
    import os
    import subprocess
    import sys
    if os.environ.get("OXH_MOE_WIDE_SMALL") == "1":
        pytest.skip("this is the process with the switch on")
    env = dict(os.environ, OXH_MOE_WIDE_SMALL="1")
    proc = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider", "--timeout", "120",
                           "--timeout-method", "thread",
                           "tests/test_gpu_moe.py::test_layer_whose_down_projection_gives_two_workgroups_per_cu",
                           "tests/test_gpu_moe.py::test_mixtral_shape_sampled_and_graph_replay",
                           "tests/test_gpu_configs.py::test_config4_moe_expert_gemvs"],
                          cwd=oxlibs.ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert proc.returncode == 0 and " passed" in proc.stdout, proc.stdout[-2000:]


def test_layer_with_more_experts_than_one_launch_carries(oxh):
    """40 and 64 experts: the gate/up launch carries 16 experts, the down launch 32, so both repeat."""
    check_layer(Q4K, Q4K, 40, 4, 256, 256, 50, seed=8, skew=True)
    check_layer(Q5K, Q6K, 64, 6, 256, 512, 23, seed=9, skew=False)


def test_mixtral_shape_sampled_and_graph_replay(oxh):
    """8 experts, top-2, 16 tokens, 4096 x 14336 Q4_K: sampled pairs and rows
    stage by stage, the combination in full, and three graph replays."""
    def sample(n, offsets):
        edge = set(int(v) for v in offsets[:-1] if v < n) | set(int(v) - 1 for v in offsets[1:] if v > 0)
        return sorted(edge)[:6]
    check_layer(Q4K, Q4K, 8, 2, 4096, 14336, 16, seed=0, skew=False, sample=sample, replay=True)


def test_argument_checks(oxh):
    d = mv.DeviceBuffer(1 << 16)
    with pytest.raises(mv.OxhError):
        mv.MoeLayer(Q4K, Q4K, d.ptr, d.ptr, d.ptr, 65, 2, 256, 256)          # too many experts
    with pytest.raises(mv.OxhError):
        mv.MoeLayer(Q4K, Q4K, d.ptr, d.ptr, d.ptr, 4, 5, 256, 256)           # top_k > n_expert
    with pytest.raises(mv.OxhError):
        mv.MoeLayer(7, Q4K, d.ptr, d.ptr, d.ptr, 4, 2, 256, 256)             # Q8_0 experts: declined
    with pytest.raises(mv.OxhError):
        mv.MoeLayer(Q4K, Q4K, d.ptr, d.ptr, d.ptr, 4, 2, 256, 300)           # ffn not in whole blocks
    layer = mv.MoeLayer(Q4K, Q4K, d.ptr, d.ptr, d.ptr, 4, 2, 256, 256, max_tok=4)
    with pytest.raises(mv.OxhError):
        mv.check(mv.lib().oxh_moe_ffn(ctypes.byref(layer.desc), ctypes.c_void_p(d.ptr), ctypes.c_void_p(d.ptr), 256,
                                      4, ctypes.c_void_p(d.ptr), 256, ctypes.c_void_p(layer.workspace.ptr), 128,
                                      None))                                  # workspace too small
    with pytest.raises(mv.OxhError):
        mv.moe_route(d.ptr, 4, 65, 2, 1, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr, d.ptr)


@pytest.mark.parametrize("seed", range(16))
def test_random_layers(oxh, seed):
    """Random expert counts (1..64), top-k, widths, token counts and type pairs, stage by stage."""
    rng = np.random.default_rng(300 + seed)
    n_exp = int(rng.integers(1, 65))
    k = int(rng.integers(1, min(8, n_exp) + 1))
    hidden, ffn = int(rng.integers(1, 4)) * 256, int(rng.integers(1, 4)) * 256
    n_tok = int(rng.integers(1, 70))
    qt_gu = (Q4K, Q5K, Q6K)[int(rng.integers(0, 3))]
    qt_dn = (Q4K, Q5K, Q6K)[int(rng.integers(0, 3))]
    check_layer(qt_gu, qt_dn, n_exp, k, hidden, ffn, n_tok, seed=40 + seed, renorm=seed & 1,
                skew=n_exp >= 3 and k < n_exp - 1)
