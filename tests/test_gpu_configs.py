"""GPU parity at the benchmark configurations' real shapes, through the C ABI.

  config 0   Q4_K 4096x4096, seed 0: outputs and activation bytes against the
             checksums taken from the compiled reference (tests/golden)
  config 1   one full Llama-3-8B layer of the decode set (qkv, o, gate/up, down)
             bit-exact against the oracle, plus a determinism check over layers
  config 2   Q8_0 lm_head 151936x896 with batch 1 and 8
  config 3   MMQ prefill 512 x 4096 against 14336/4096 rows: sampled tokens
             bit-exact against the oracle, linearity-free property: every
             token's output equals the single-vector GEMV of that token
  config 4   Mixtral-shaped expert GEMVs (8 experts, top-2, 16 tokens)
"""
import os
import zlib

import ctypes

import numpy as np
import pytest

import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth, workloads

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
Q80, Q4K, Q5K, Q6K = 7, 13, 15, 16


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def oracle_matvec(qtype, w, rows, cols, x):
    o = oxlibs.oracle()
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert o.oxo_matvec_quantized(qtype, w.ctypes.data, rows, cols, synth.row_bytes(qtype, cols),
                                  x.ctypes.data, out.ctypes.data, temp.ctypes.data) == 0
    return out, temp


@pytest.mark.parametrize("name,qt,rows,cols", [("cfg0_q4k_4096x4096", Q4K, 4096, 4096),
                                               ("down_q6k_4096x14336", Q6K, 4096, 14336),
                                               ("ffn_q80_4864x896", Q80, 4864, 896)])
def test_config0_against_reference_checksums(oxh, name, qt, rows, cols):
    g = np.load(os.path.join(GOLD, "full_size.npz"))
    w = synth.weights(qt, rows, cols, seed=0, stream=0)
    x = synth.normal(cols, seed=0, stream=1000)
    out = np.zeros(rows, np.float32)
    temp = np.zeros(cols, np.float32)
    assert mv.matvec_quantized(qt, w, rows, cols, synth.row_bytes(qt, cols), x, out, temp) == 0
    nact = mv.act_bytes(qt, cols)
    assert zlib.crc32(temp.view(np.uint8)[:nact].tobytes()) == int(g[name + "_crc_act"][0])
    if qt == Q80:
        ref = g[name + "_out"]
        assert np.all(np.abs(out - ref) <= 1e-4 + 1e-5 * np.abs(ref))
    else:
        assert zlib.crc32(out.tobytes()) == int(g[name + "_crc_out"][0])
        assert np.array_equal(bits(out), bits(g[name + "_out"]))


def test_config1_decode_layer_bit_exact_and_repeatable(oxh):
    ds = workloads.DecodeSet(layers=2, seed=0, keep_host=(0, 1))
    ds.launch_step()
    mv.sync()
    first = [[ds.output(layer, op) for op in range(4)] for layer in range(2)]
    for layer in range(2):
        for op, (name, qt, rows, cols, _) in enumerate(ds.ops):
            x = ds.x_host[(layer, op)]
            off = 0
            o = oxlibs.oracle()
            act = np.zeros(mv.act_bytes(qt, cols), np.uint8)
            o.oxo_quantize_q8_k(x.ctypes.data, cols, act.ctypes.data)
            assert np.array_equal(ds.activation(layer, op), act), (layer, name)
            for seg, r in enumerate(rows):
                want, _ = oracle_matvec(qt, ds.host[(layer, op, seg)], r, cols, x)
                assert np.array_equal(bits(first[layer][op][off:off + r]), bits(want)), (layer, name, seg)
                off += r
    # replay through a HIP graph: identical bits every time
    g = mv.Graph()
    with g:
        ds.launch_step()
    for _ in range(3):
        g.launch()
        mv.sync()
        for layer in range(2):
            for op in range(4):
                assert np.array_equal(bits(ds.output(layer, op)), bits(first[layer][op]))
    g.destroy()


@pytest.mark.parametrize("n_vec", [1, 8])
def test_config2_q8_0_lm_head(oxh, n_vec):
    rows, cols = 151936, 896
    w = synth.weights(Q80, rows, cols, seed=0, stream=5)
    xs = synth.normal(n_vec * cols, seed=0, stream=6).reshape(n_vec, cols)
    outs = np.zeros((n_vec, rows), np.float32)
    temp = np.zeros(cols, np.float32)
    scratch = np.zeros(mv.batch_scratch_bytes(cols), np.uint8)
    assert mv.matvec_quantized_batch(Q80, w, rows, cols, synth.row_bytes(Q80, cols), xs, cols, outs,
                                     rows, n_vec, temp, scratch) == 0
    for v in range(n_vec):
        want, _ = oracle_matvec(Q80, w, rows, cols, np.ascontiguousarray(xs[v]))
        assert np.array_equal(bits(outs[v]), bits(want))
    ref = oxlibs.ref()
    if ref is not None:
        r_out = np.zeros(rows, np.float32)
        ref.oc_matvec_quantized(Q80, w.ctypes.data, rows, cols, synth.row_bytes(Q80, cols),
                                xs[0].ctypes.data, r_out.ctypes.data, temp.ctypes.data)
        assert np.all(np.abs(outs[0] - r_out) <= 1e-4 + 1e-5 * np.abs(r_out))


@pytest.mark.parametrize("rows", [14336, 4096])
def test_config3_mmq_prefill_512_tokens(oxh, rows):
    cols, n_vec = 4096, 512
    w = synth.weights(Q4K, rows, cols, seed=0, stream=0)
    xs = synth.normal(n_vec * cols, seed=0, stream=2000).reshape(n_vec, cols)
    d_w = mv.DeviceBuffer.from_host(w)
    d_x = mv.DeviceBuffer.from_host(xs)
    nact = mv.act_bytes(Q4K, cols)
    d_a = mv.DeviceBuffer(n_vec * nact)
    d_o = mv.DeviceBuffer(n_vec * rows * 4)
    mv.quantize(Q4K, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    mv.mmq(Q4K, d_w.ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows)
    out = d_o.download(np.float32, n_vec * rows).reshape(n_vec, rows)
    acts = d_a.download(np.uint8, n_vec * nact).reshape(n_vec, nact)
    o = oxlibs.oracle()
    for v in (0, 1, 31, 32, 63, 64, 255, 300, 511):
        want, wtemp = oracle_matvec(Q4K, w, rows, cols, np.ascontiguousarray(xs[v]))
        assert np.array_equal(acts[v], wtemp.view(np.uint8)[:nact]), v
        assert np.array_equal(bits(out[v]), bits(want)), v
    # the MFMA path against the dot-instruction GEMV kernel on the same device data
    # (two activations per launch: three or more would run on the matrix cores too)
    d_o2 = mv.DeviceBuffer(2 * rows * 4)
    for v0 in (8, 10, 120, 126, 504, 510):
        segs = mv.make_segments([(d_w.ptr, d_o2.ptr, rows, v0)])
        mv.gemv_segments(Q4K, segs, cols, d_a.ptr, 2, rows)
        got = d_o2.download(np.float32, 2 * rows).reshape(2, rows)
        assert np.array_equal(bits(got), bits(out[v0:v0 + 2]))


@pytest.mark.parametrize("qtype,rows,cols,n_vec", [
    (Q4K, 7165, 512, 507),      # 256x128 tiles would be 28 x 4 workgroups: 128x64 tiles, 56 x 8
    (Q4K, 14329, 256, 500),     # 256x128 tiles: 56 x 4 = 224 workgroups
    (Q4K, 4100, 512, 40),       # too few workgroups for either: 64x32 tiles, 65 x 2
    (Q6K, 7165, 512, 507),      # Q6_K: 128x128 tiles, 56 x 4
    (Q6K, 3600, 256, 500),      # Q6_K: 64x128 tiles on four waves, 57 x 4
    (Q6K, 14250, 256, 100),     # Q6_K: 128x64 tiles, 112 x 2 (223 tiles of 64x128 would leave CUs idle)
    (Q6K, 4100, 512, 40),       # Q6_K: 64x32 tiles
    (Q5K, 7165, 512, 507),      # Q5_K: 128x128 tiles, 56 x 4
    (Q5K, 3600, 256, 500),      # Q5_K: 128x64 tiles, 29 x 8
    (Q5K, 4100, 512, 40),       # Q5_K: 64x32 tiles
])
def test_mmq_tile_variants_ragged(oxh, qtype, rows, cols, n_vec):
    """The MFMA kernel comes in several tile shapes (256x128, 128x64, 64x32,
    64x16 rows x tokens, and 64x128 for Q6_K), picked from the launch size;
    these cases select all but 64x16 on a 256-CU device and leave the last row tile and the last
    token tile partly filled.  Every output is checked against the
    dot-instruction GEMV kernel on the same device data (two activations per
    launch: three or more would run on the matrix cores too), and a sample of
    tokens against the oracle."""
    info = mv.device_info()
    if info["n_cu"] != 256:
        pytest.skip("tile choice is tied to 256 compute units")
    w = synth.weights(qtype, rows, cols, seed=5, stream=rows)
    xs = synth.normal(n_vec * cols, seed=5, stream=n_vec).reshape(n_vec, cols)
    d_w = mv.DeviceBuffer.from_host(w)
    d_x = mv.DeviceBuffer.from_host(xs)
    nact = mv.act_bytes(qtype, cols)
    d_a = mv.DeviceBuffer(n_vec * nact)
    stride = rows + 3
    d_o = mv.DeviceBuffer(n_vec * stride * 4)
    d_o.upload(np.full(n_vec * stride, -7.25, np.float32))
    mv.quantize(qtype, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    mv.mmq(qtype, d_w.ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, stride)
    out = d_o.download(np.float32, n_vec * stride).reshape(n_vec, stride)
    assert np.all(out[:, rows:] == -7.25)
    for v in (0, 31, 32, n_vec // 2, n_vec - 1):
        want, _ = oracle_matvec(qtype, w, rows, cols, np.ascontiguousarray(xs[v]))
        assert np.array_equal(bits(out[v, :rows]), bits(want)), v
    d_o2 = mv.DeviceBuffer(n_vec * rows * 4)
    for v0 in range(0, n_vec, 2):
        nv = min(2, n_vec - v0)
        segs = mv.make_segments([(d_w.ptr, d_o2.ptr + v0 * rows * 4, rows, v0)])
        mv.gemv_segments(qtype, segs, cols, d_a.ptr, nv, rows)
    got = d_o2.download(np.float32, n_vec * rows).reshape(n_vec, rows)
    assert np.array_equal(bits(got), bits(out[:, :rows]))


@pytest.mark.parametrize("qtype", [Q4K, Q5K, Q6K])
def test_small_batch_launch_on_128_row_tiles(oxh, qtype):
    """Five activations over 30000 rows: 469 tiles of 64 rows would be fewer than two per CU on a 256-CU
    device, 235 tiles of 128 rows still nearly one per CU, so a Q4_K launch takes the eight-wave tile with
    three super-blocks per stage (Q5_K and Q6_K stay on 64-row tiles with two); the last tile is ragged.
    Bits against the oracle."""
    rows, cols, n_vec = 30000, 768, 5
    w = synth.weights(qtype, rows, cols, seed=12, stream=3)
    xs = synth.normal(n_vec * cols, seed=12, stream=4).reshape(n_vec, cols)
    d_w, d_x = mv.DeviceBuffer.from_host(w), mv.DeviceBuffer.from_host(xs)
    d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(qtype, cols))
    d_o = mv.DeviceBuffer(n_vec * rows * 4)
    mv.gemv_segments_f32(qtype, mv.make_segments([(d_w.ptr, d_o.ptr, rows, 0)]), cols, d_x.ptr, cols, d_a.ptr,
                         n_vec, rows)
    got = d_o.download(np.float32, n_vec * rows).reshape(n_vec, rows)
    for v in range(n_vec):
        want, _ = oracle_matvec(qtype, w, rows, cols, np.ascontiguousarray(xs[v]))
        assert np.array_equal(bits(got[v]), bits(want)), v


def test_config4_moe_expert_gemvs(oxh):
    ms = workloads.MoESet(seed=0, keep_host=True)
    o = oxlibs.oracle()
    ids = np.zeros((16, 2), np.int32)
    wts = np.zeros((16, 2), np.float32)
    o.oxo_moe_route(ms.logits.ctypes.data, 16, 8, 2, 1, ids.ctypes.data, wts.ctypes.data)
    assert np.array_equal(ids, ms.ids)
    assert np.allclose(wts, ms.gate_w, rtol=1e-6)
    assert ms.offsets[-1] == 32 and sorted(ms.pair_tok[:ms.offsets[1]]) == list(ms.pair_tok[:ms.offsets[1]])
    ms.launch_step()
    mv.sync()
    gate, up, down = ms.outputs()
    rb_gu, rb_dn = synth.row_bytes(Q4K, 4096), synth.row_bytes(Q4K, 14336)
    rng = np.random.default_rng(0)
    for e in range(8):
        lo, hi = int(ms.offsets[e]), int(ms.offsets[e + 1])
        for pidx in range(lo, hi):
            if rng.random() > 0.4 and pidx not in (lo, hi - 1):
                continue
            wg = ms.host["gate"][e * 14336 * rb_gu:(e + 1) * 14336 * rb_gu]
            wu = ms.host["up"][e * 14336 * rb_gu:(e + 1) * 14336 * rb_gu]
            wd = ms.host["down"][e * 4096 * rb_dn:(e + 1) * 4096 * rb_dn]
            x = np.ascontiguousarray(ms.xg[pidx])
            assert np.array_equal(x, ms.x_tok[ms.pair_tok[pidx]])
            assert e in ms.ids[ms.pair_tok[pidx]]
            assert np.array_equal(bits(gate[pidx]), bits(oracle_matvec(Q4K, wg, 14336, 4096, x)[0]))
            assert np.array_equal(bits(up[pidx]), bits(oracle_matvec(Q4K, wu, 14336, 4096, x)[0]))
            h = np.ascontiguousarray(ms.h[pidx])
            assert np.array_equal(bits(down[pidx]), bits(oracle_matvec(Q4K, wd, 4096, 14336, h)[0]))


@pytest.mark.parametrize("qtype,rows,cols,n_vec", [
    (Q4K, 14336, 4096, 512), (Q4K, 4096, 4096, 512), (Q4K, 3000, 2048, 130),
    (Q5K, 7165, 512, 507), (Q5K, 3600, 256, 500), (Q6K, 2048, 1024, 300), (Q4K, 4100, 512, 20),
])
def test_mmq_relaxed_mode_is_opt_in_and_within_tolerance(oxh, qtype, rows, cols, n_vec):
    """OXH_MMQ_RELAXED evaluates the float step of the Q4_K / Q5_K prefill tiles with fused multiply-adds.
    Bar, written here: |relaxed - exact| <= 1e-5 * |exact| + 2e-6 * rms(exact) for every output (each
    block term moves by an ulp or two of itself, and a term is of the size of the outputs' spread, not of
    the one output it lands in); flags = 0 through the
    same entry point stays bit-identical to oxh_mmq; types and launch sizes without a relaxed kernel
    (Q6_K, launches on the small tiles) give the exact bits under the flag as well."""
    w = synth.weights(qtype, rows, cols, seed=6, stream=rows)
    xs = synth.normal(n_vec * cols, seed=6, stream=n_vec).reshape(n_vec, cols)
    d_w = mv.DeviceBuffer.from_host(w)
    d_x = mv.DeviceBuffer.from_host(xs)
    d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(qtype, cols))
    mv.quantize(qtype, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    outs = []
    for mode in ("plain", "zero", "relaxed"):
        d_o = mv.DeviceBuffer(n_vec * rows * 4)
        if mode == "plain":
            mv.mmq(qtype, d_w.ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows)
        elif mode == "zero":
            assert mv.lib().oxh_mmq_ex(qtype, ctypes.c_void_p(d_w.ptr), rows, cols, ctypes.c_void_p(d_a.ptr), n_vec,
                                       ctypes.c_void_p(d_o.ptr), rows, 0, None) == 0
        else:
            mv.mmq(qtype, d_w.ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows, flags=mv.MMQ_RELAXED)
        mv.sync()
        outs.append(d_o.download(np.float32, n_vec * rows))
        d_o.free()
    exact, zero, relaxed = outs
    assert np.array_equal(bits(exact), bits(zero))
    rms = float(np.sqrt(np.mean(exact.astype(np.float64) ** 2)))
    assert np.all(np.abs(relaxed - exact) <= 1e-5 * np.abs(exact) + 2e-6 * rms)
    # the relaxed step exists for the two prefill tiles (256 or 128 rows x 128 tokens, 128 x 64), which a
    # launch gets when it fills the device with them
    has_relaxed_kernel = (qtype, rows) in ((Q4K, 14336), (Q4K, 4096), (Q5K, 7165), (Q5K, 3600)) and \
        mv.device_info()["n_cu"] == 256
    if has_relaxed_kernel:
        assert not np.array_equal(bits(exact), bits(relaxed))       # it is a different evaluation
    else:
        assert np.array_equal(bits(exact), bits(relaxed))
    assert mv.lib().oxh_mmq_ex(qtype, ctypes.c_void_p(d_w.ptr), rows, cols, ctypes.c_void_p(d_a.ptr), n_vec,
                               ctypes.c_void_p(d_w.ptr), rows, 2, None) != 0           # unknown flag


@pytest.mark.parametrize("qt", [13, 15, 16])
@pytest.mark.parametrize("rows,cols,n_vec", [(4096, 14336, 16), (1000, 4096, 5), (70, 2048, 40), (64, 8192, 64),
                                             (3000, 2304, 17), (1, 14336, 1), (33, 5120, 3), (257, 7168, 31),
                                             (100, 5376, 9), (2049, 6400, 18), (4000, 14336, 45), (4096, 4096, 24)])
def test_mmq_with_a_tile_s_columns_shared_between_workgroups(oxh, qt, rows, cols, n_vec):
    """oxh_mmq_split: every super-block's terms go to a workspace and are added in block order by a second
    launch: bit for bit what oxh_mmq gives, padding between rows and out_stride untouched, and without a
    workspace (or for a launch that would not be split) it is oxh_mmq."""
    out_stride = rows + 3
    w = mv.DeviceBuffer.from_host(synth.weights(qt, rows, cols, seed=rows, stream=qt))
    x = mv.DeviceBuffer.from_host(synth.normal(n_vec * cols, seed=n_vec, stream=qt))
    a = mv.DeviceBuffer(n_vec * mv.act_bytes(qt, cols))
    mv.quantize(qt, x.ptr, cols, n_vec, cols, a.ptr)
    want = mv.DeviceBuffer(n_vec * out_stride * 4)
    got = mv.DeviceBuffer(n_vec * out_stride * 4)
    for b in (want, got):
        mv.lib().oxh_memset(ctypes.c_void_p(b.ptr), 0x7F, b.nbytes, None)
    mv.mmq(qt, w.ptr, rows, cols, a.ptr, n_vec, want.ptr, out_stride)
    need = mv.mmq_split_workspace(qt, rows, cols, n_vec, out_stride)
    full = cols // 256 * n_vec * out_stride * 4
    assert need == (0 if (rows, cols) in ((70, 2048), (3000, 2304)) else full)     # those two: too little to save
    ws = mv.DeviceBuffer(full)
    need = full                     # a launch that would not be split ignores the workspace
    mv.mmq_split(qt, w.ptr, rows, cols, a.ptr, n_vec, got.ptr, out_stride, ws.ptr, need)
    a_, b_ = want.download(np.uint32, n_vec * out_stride), got.download(np.uint32, n_vec * out_stride)
    assert np.array_equal(a_, b_)
    assert np.all(a_.reshape(n_vec, out_stride)[:, rows:] == 0x7F7F7F7F)
    # no workspace: the plain launch
    mv.lib().oxh_memset(ctypes.c_void_p(got.ptr), 0x7F, got.nbytes, None)
    mv.mmq_split(qt, w.ptr, rows, cols, a.ptr, n_vec, got.ptr, out_stride, None, 0)
    assert np.array_equal(a_, got.download(np.uint32, n_vec * out_stride))
    # launches that are not split: many tiles, few super-blocks, a long batch
    assert mv.mmq_split_workspace(qt, 28672, 4096, 16, 28672) == 0
    assert mv.mmq_split_workspace(qt, 4096, 1024, 16, 4096) == 0
    assert mv.mmq_split_workspace(qt, 4096, 14336, 512, 4096) == 0
    assert mv.mmq_split_workspace(7, 4096, 4096, 16, 4096) == 0


@pytest.mark.parametrize("qt", [13, 15, 16, 10, 8])
@pytest.mark.parametrize("rows,cols,n_vec", [(300, 5120, 9), (1000, 4096, 7), (130, 14336, 33)])
def test_batch_entry_point_over_few_rows_and_many_columns(oxh, qt, rows, cols, n_vec):
    """oc_matvec_quantized_batch over shapes whose tiles share their columns between workgroups (seven
    vectors or more of a K-quant; Q2_K and Q3_K from nine on, through their rewritten forms): padded
    strides, every output with the oracle's bits, nothing written between rows and out_stride."""
    assert mv.mmq_split_workspace(16 if qt in (10, 8) else qt, rows, cols, n_vec, rows) > 0
    rb = synth.row_bytes(qt, cols)
    w = synth.weights(qt, rows, cols, seed=71, stream=n_vec)
    in_stride, out_stride = cols + 8, rows + 3
    xb = synth.normal(n_vec * in_stride, seed=72, stream=n_vec).reshape(n_vec, in_stride)
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
