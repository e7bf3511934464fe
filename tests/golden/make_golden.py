"""Writes tests/golden/*.npz: input/output vectors taken from the COMPILED
REFERENCE (oracle/_ref/liboxref.so, built by `make -C oracle` from the
reference checkout).  Run in the build container only; the fixtures are
committed, this script documents how they were made.

    python tests/golden/make_golden.py

    python tests/golden/make_golden.py q5_k     # only q5_k.npz
    python tests/golden/make_golden.py float    # only float_steps.npz
    python tests/golden/make_golden.py dequant  # only dequant_rows.npz
    python tests/golden/make_golden.py legacy   # only legacy_formats.npz
    python tests/golden/make_golden.py q23_k    # only q23_k.npz
    python tests/golden/make_golden.py iq       # only iq_types.npz
    python tests/golden/make_golden.py iq4      # only iq4_types.npz

Every array is data: inputs and the reference's outputs for them.
"""
import ctypes
import os
import sys
import zlib

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oxlibs  # noqa: E402
from oxidize_amd import synth  # noqa: E402

Q80, Q4K, Q5K, Q6K = 7, 13, 15, 16


def xorshift_bytes(n, seed):
    """The byte stream of the reference's raw-block tests
    (tests/test_oxk_avx2_parity.c:125-131): xorshift32, low byte of each draw."""
    out = np.empty(n, np.uint8)
    s = seed & 0xFFFFFFFF
    for i in range(n):
        s ^= (s << 13) & 0xFFFFFFFF
        s ^= s >> 17
        s ^= (s << 5) & 0xFFFFFFFF
        out[i] = s & 0xFF
    return out


def finite_scale_bits(rng, n):
    """f16 bit patterns of finite positive scales in [0.0005, 0.0405]."""
    vals = (0.0005 + rng.integers(0, 1000, n) * 4e-5).astype(np.float32)
    return vals.astype(np.float16).view(np.uint16)


def q8k_acts(rng, trials, nb):
    act = np.zeros((trials, nb, 292), np.uint8)
    d = (0.001 + rng.integers(0, 1000, (trials, nb)) * 2e-5).astype(np.float32)
    act[:, :, 0:4] = d.view(np.uint8).reshape(trials, nb, 4)
    q = rng.integers(-127, 128, (trials, nb, 256)).astype(np.int8)
    act[:, :, 4:260] = q.view(np.uint8)
    bs = q.reshape(trials, nb, 16, 16).sum(axis=3).astype(np.int16)
    act[:, :, 260:292] = bs.view(np.uint8).reshape(trials, nb, 32)
    return act


def q5_k(ref):
    """q5_k.npz: the same three kinds of vectors as the other files, for Q5_K
    (a file and a generator of its own, so the older fixtures stay byte for
    byte what they were)."""
    rng = np.random.default_rng(20240915)
    out = {}
    nb, trials = 12, 24
    w = xorshift_bytes(trials * nb * 176, 0x9E3779B9 ^ Q5K).reshape(trials, nb, 176)
    for off in (0, 2):
        bits = finite_scale_bits(rng, trials * nb).reshape(trials, nb)
        w[:, :, off] = bits & 0xFF
        w[:, :, off + 1] = bits >> 8
    act = q8k_acts(rng, trials, nb)
    scalar = np.empty((trials, 2), np.uint32)
    disp = np.empty((trials, 2), np.uint32)
    for t in range(trials):
        wt = np.ascontiguousarray(w[t])
        at = np.ascontiguousarray(act[t])
        for k, blocks in enumerate((1, nb)):
            scalar[t, k] = np.float32(ref.oc_oxk_dot_q5_k_q8_k_scalar(
                wt.ctypes.data, blocks, at.ctypes.data)).view(np.uint32)
            disp[t, k] = np.float32(ref.oc_oxk_dot_q5_k_q8_k(
                wt.ctypes.data, blocks, at.ctypes.data)).view(np.uint32)
    out["raw_w"], out["raw_act"] = w, act
    out["raw_scalar_bits"], out["raw_dispatched_bits"] = scalar, disp

    # API level, both type ids
    for qt, rows, cols in ((15, 40, 1280), (14, 9, 256)):
        rb = synth.row_bytes(qt, cols)
        wm = synth.weights(qt, rows, cols, seed=7, stream=qt)
        x = synth.normal(cols, seed=7, stream=100 + qt)
        o = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qt, wm.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data,
                                temp.ctypes.data)
        key = "api%d_" % qt
        out[key + "w"], out[key + "x"] = wm, x
        out[key + "shape"] = np.array([rows, cols, rb], np.int64)
        out[key + "out_bits"] = o.view(np.uint32).copy()
        out[key + "act"] = temp.view(np.uint8)[:cols // 256 * 292].copy()
        n_vec, in_stride, out_stride = 5, cols + 8, rows + 3
        xs = synth.normal(n_vec * in_stride, seed=8, stream=qt).reshape(n_vec, in_stride)
        outs = np.full((n_vec, out_stride), -1.0, np.float32)
        scratch = np.zeros(ref.oc_matvec_batch_scratch_bytes(cols), np.uint8)
        ref.oc_matvec_quantized_batch(qt, wm.ctypes.data, rows, cols, rb, xs.ctypes.data, in_stride,
                                      outs.ctypes.data, out_stride, n_vec, temp.ctypes.data,
                                      scratch.ctypes.data, scratch.nbytes)
        out[key + "batch_x"] = xs
        out[key + "batch_out_bits"] = outs.view(np.uint32).copy()

    # full-size shapes: checksums and the f32 outputs
    for name, rows, cols in (("big_4096x4096", 4096, 4096), ("big_4096x14336", 4096, 14336)):
        rb = synth.row_bytes(Q5K, cols)
        wm = synth.weights(Q5K, rows, cols, seed=0, stream=0)
        x = synth.normal(cols, seed=0, stream=1000)
        o = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(Q5K, wm.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data,
                                temp.ctypes.data)
        out[name + "_crc_w"] = np.array([zlib.crc32(wm.tobytes())], np.uint32)
        out[name + "_crc_x"] = np.array([zlib.crc32(x.tobytes())], np.uint32)
        out[name + "_crc_out"] = np.array([zlib.crc32(o.tobytes())], np.uint32)
        out[name + "_out"] = o.copy()
    np.savez_compressed(os.path.join(HERE, "q5_k.npz"), **out)


def float_steps(ref):
    """float_steps.npz: RMSNorm and SwiGLU as the compiled reference computes
    them (oc_rms_norm_f32, oc_swiglu_inplace_f32)."""
    out = {}
    for n in (256, 896, 4096):
        x = synth.normal(n, seed=11, stream=n) * np.float32(3.0)
        w = (synth.normal(n, seed=12, stream=n) * np.float32(0.1) + np.float32(1.0)).astype(np.float32)
        for eps in (1e-5, 1e-6):
            o = np.zeros(n, np.float32)
            ref.oc_rms_norm_f32(x.ctypes.data, w.ctypes.data, o.ctypes.data, n, eps)
            out["rms_%d_%g_out" % (n, eps)] = o
        out["rms_%d_x" % n], out["rms_%d_w" % n] = x, w
    g = np.concatenate([synth.normal(4000, seed=13) * np.float32(4.0),
                        np.array([0.0, -0.0, 1e-8, -1e-8, 20.0, -20.0, 87.9, -87.9, 100.0, -100.0,
                                  1e4, -1e4], np.float32),
                        np.linspace(-12, 12, 84, dtype=np.float32)]).astype(np.float32)
    u = synth.normal(g.size, seed=14)
    o = g.copy()
    ref.oc_swiglu_inplace_f32(o.ctypes.data, u.ctypes.data, g.size)
    out["swiglu_gate"], out["swiglu_up"], out["swiglu_out"] = g, u, o
    np.savez_compressed(os.path.join(HERE, "float_steps.npz"), **out)


def q23_k(ref):
    """q23_k.npz: Q2_K (type id 8) and Q3_K (ids 9, 10, 11): raw-block dots by
    the scalar and the dispatched kernels, the matvec entry points (single and
    batch), dequantised rows and full-size checksums."""
    rng = np.random.default_rng(20241125)
    out = {}
    nb, trials = 12, 24
    for name, qt, bsize, scale_at in (("q2_k", 8, 84, (80, 82)), ("q3_k", 10, 110, (108,))):
        w = xorshift_bytes(trials * nb * bsize, 0x9E3779B9 ^ qt).reshape(trials, nb, bsize)
        for off in scale_at:
            bits = finite_scale_bits(rng, trials * nb).reshape(trials, nb)
            w[:, :, off] = bits & 0xFF
            w[:, :, off + 1] = bits >> 8
        act = q8k_acts(rng, trials, nb)
        scalar = np.empty((trials, 2), np.uint32)
        disp = np.empty((trials, 2), np.uint32)
        fs, fd = getattr(ref, "oc_oxk_dot_%s_q8_k_scalar" % name), getattr(ref, "oc_oxk_dot_%s_q8_k" % name)
        for t in range(trials):
            wt, at = np.ascontiguousarray(w[t]), np.ascontiguousarray(act[t])
            for k, blocks in enumerate((1, nb)):
                scalar[t, k] = np.float32(fs(wt.ctypes.data, blocks, at.ctypes.data)).view(np.uint32)
                disp[t, k] = np.float32(fd(wt.ctypes.data, blocks, at.ctypes.data)).view(np.uint32)
        out[name + "_raw_w"], out[name + "_raw_act"] = w, act
        out[name + "_raw_scalar_bits"], out[name + "_raw_dispatched_bits"] = scalar, disp
    for qt, rows, cols in ((8, 40, 1280), (9, 9, 256), (10, 40, 1280), (11, 17, 512)):
        rb = synth.row_bytes(qt, cols)
        wm = synth.weights(qt, rows, cols, seed=7, stream=qt)
        x = synth.normal(cols, seed=7, stream=100 + qt)
        o = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qt, wm.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data,
                                temp.ctypes.data)
        key = "api%d_" % qt
        out[key + "w"], out[key + "x"] = wm, x
        out[key + "shape"] = np.array([rows, cols, rb], np.int64)
        out[key + "out_bits"] = o.view(np.uint32).copy()
        out[key + "act"] = temp.view(np.uint8)[:cols // 256 * 292].copy()
        n_vec, in_stride, out_stride = 5, cols + 8, rows + 3
        xs = synth.normal(n_vec * in_stride, seed=8, stream=qt).reshape(n_vec, in_stride)
        outs = np.full((n_vec, out_stride), -1.0, np.float32)
        scratch = np.zeros(ref.oc_matvec_batch_scratch_bytes(cols), np.uint8)
        ref.oc_matvec_quantized_batch(qt, wm.ctypes.data, rows, cols, rb, xs.ctypes.data, in_stride,
                                      outs.ctypes.data, out_stride, n_vec, temp.ctypes.data,
                                      scratch.ctypes.data, scratch.nbytes)
        out[key + "batch_x"] = xs
        out[key + "batch_out_bits"] = outs.view(np.uint32).copy()
        deq = np.zeros((2, cols), np.float32)
        for r in range(2):
            assert ref.oc_quant_dequant_row(qt, wm[r * rb:].ctypes.data, rb, deq[r].ctypes.data, cols) == 0
        out[key + "dequant_bits"] = deq.view(np.uint32).copy()
    for qt, name in ((8, "big_q2_k_4096x4096"), (10, "big_q3_k_4096x4096")):
        rows = cols = 4096
        rb = synth.row_bytes(qt, cols)
        wm = synth.weights(qt, rows, cols, seed=0, stream=0)
        x = synth.normal(cols, seed=0, stream=1000)
        o = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qt, wm.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data,
                                temp.ctypes.data)
        out[name + "_crc_w"] = np.array([zlib.crc32(wm.tobytes())], np.uint32)
        out[name + "_crc_out"] = np.array([zlib.crc32(o.tobytes())], np.uint32)
        out[name + "_out"] = o.copy()
    np.savez_compressed(os.path.join(HERE, "q23_k.npz"), **out)


def dequant_rows(ref):
    """dequant_rows.npz: rows of every type the embedding lookup handles,
    expanded by the compiled reference (oc_quant_dequant_row)."""
    out = {}
    for name, qt, cols in (("q4_k", 13, 768), ("q5_k", 15, 768), ("q6_k", 16, 768), ("q8_0", 7, 160),
                           ("q4_0", 3, 160), ("q4_1", 4, 160), ("q5_0", 5, 160), ("q5_1", 6, 160)):
        rows = 3
        rb = synth.row_bytes(qt, cols)
        w = synth.weights(qt, rows, cols, seed=17, stream=qt)
        f = np.zeros((rows, cols), np.float32)
        for r in range(rows):
            rc = ref.oc_quant_dequant_row(qt, w[r * rb:].ctypes.data, rb, f[r].ctypes.data, cols)
            assert rc == 0
        out[name + "_w"], out[name + "_bits"] = w, f.view(np.uint32).copy()
        out[name + "_shape"] = np.array([rows, cols, rb], np.int64)
    np.savez_compressed(os.path.join(HERE, "dequant_rows.npz"), **out)


LEGACY = (("q4_0", 3, 18), ("q4_1", 4, 20), ("q5_0", 5, 22), ("q5_1", 6, 24), ("al5_xs", 18, 14))


ALIASES = (("al5", 17, 3), ("al6", 19, 5), ("al8", 20, 7))


def legacy_formats(ref):
    """legacy_formats.npz: Q4_0 / Q4_1 / Q5_0 / Q5_1 against Q8_0 activations,
    raw-block dots (scalar and dispatched kernels) and the matvec entry points."""
    rng = np.random.default_rng(20241101)
    out = {}
    nb, trials = 12, 16
    for name, qt, bsize in LEGACY:
        w = xorshift_bytes(trials * nb * bsize, 0x9E3779B9 ^ qt).reshape(trials, nb, bsize)
        for off in ((0, 2) if name.endswith("_1") else (0,)):
            bits = finite_scale_bits(rng, trials * nb).reshape(trials, nb)
            w[:, :, off] = bits & 0xFF
            w[:, :, off + 1] = bits >> 8
        act = np.zeros((trials, nb, 34), np.uint8)
        bits = finite_scale_bits(rng, trials * nb).reshape(trials, nb)
        act[:, :, 0] = bits & 0xFF
        act[:, :, 1] = bits >> 8
        act[:, :, 2:] = rng.integers(-127, 128, (trials, nb, 32)).astype(np.int8).view(np.uint8)
        scalar = np.empty((trials, 2), np.uint32)
        disp = np.empty((trials, 2), np.uint32)
        fs = getattr(ref, "oc_oxk_dot_%s_q8_0_scalar" % name)
        fd = getattr(ref, "oc_oxk_dot_%s_q8_0" % name)
        for t in range(trials):
            wt, at = np.ascontiguousarray(w[t]), np.ascontiguousarray(act[t])
            for k, blocks in enumerate((1, nb)):
                scalar[t, k] = np.float32(fs(wt.ctypes.data, blocks, at.ctypes.data)).view(np.uint32)
                disp[t, k] = np.float32(fd(wt.ctypes.data, blocks, at.ctypes.data)).view(np.uint32)
        out[name + "_w"], out[name + "_act"] = w, act
        out[name + "_scalar_bits"], out[name + "_dispatched_bits"] = scalar, disp
        rows, cols = 40, 896
        rb = synth.row_bytes(qt, cols)
        wm = synth.weights(qt, rows, cols, seed=7, stream=qt)
        x = synth.normal(cols, seed=7, stream=100 + qt)
        o = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qt, wm.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data,
                                temp.ctypes.data)
        out[name + "_api_w"], out[name + "_api_x"] = wm, x
        out[name + "_api_shape"] = np.array([rows, cols, rb], np.int64)
        out[name + "_api_out"] = o.copy()
        out[name + "_api_act"] = temp.view(np.uint8)[:cols // 32 * 34].copy()
        if name == "al5_xs":
            deq = np.zeros((2, cols), np.float32)
            for r in range(2):
                assert ref.oc_quant_dequant_row(qt, wm[r * rb:].ctypes.data, rb, deq[r].ctypes.data, cols) == 0
            out[name + "_dequant_bits"] = deq.view(np.uint32).copy()
    # AL5 / AL6 / AL8: the Q4_0 / Q5_0 / Q8_0 layouts under their own type ids
    for name, qt, base in ALIASES:
        rows, cols = 24, 896
        rb = synth.row_bytes(base, cols)
        wm = synth.weights(base, rows, cols, seed=8, stream=qt)
        x = synth.normal(cols, seed=8, stream=200 + qt)
        o, temp, deq = np.zeros(rows, np.float32), np.zeros(cols, np.float32), np.zeros((2, cols), np.float32)
        ref.oc_matvec_quantized(qt, wm.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data, temp.ctypes.data)
        for r in range(2):
            assert ref.oc_quant_dequant_row(qt, wm[r * rb:].ctypes.data, rb, deq[r].ctypes.data, cols) == 0
        out[name + "_api_w"], out[name + "_api_x"] = wm, x
        out[name + "_api_shape"] = np.array([rows, cols, rb], np.int64)
        out[name + "_api_out"] = o.copy()
        out[name + "_api_act"] = temp.view(np.uint8)[:cols // 32 * 34].copy()
        out[name + "_dequant_bits"] = deq.view(np.uint32).copy()
    np.savez_compressed(os.path.join(HERE, "legacy_formats.npz"), **out)


def iq_types(ref):
    """iq_types.npz: IQ3_S (type id 25) and IQ1_XXXS (id 36), the two codebook formats on the reference's
    integer path: raw-block dots (IQ3_S by its scalar and its dispatched kernel; IQ1_XXXS has one form),
    the matvec entry points (single and batch) and a full-size checksum."""
    rng = np.random.default_rng(20241126)
    out = {}
    nb, trials = 12, 24
    F, V, Z = ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t
    forms = {"iq3_s": ("oc_oxk_dot_iq3_s_q8_k_scalar", "oc_oxk_dot_iq3_s_q8_k"),
             "iq1_xxxs": ("oc_quant_dot_iq1_xxxs_q8_k", "oc_quant_dot_iq1_xxxs_q8_k")}
    for name, qt, bsize in (("iq3_s", 25, 110), ("iq1_xxxs", 36, 38)):
        w = xorshift_bytes(trials * nb * bsize, 0x9E3779B9 ^ qt).reshape(trials, nb, bsize)
        bits = finite_scale_bits(rng, trials * nb).reshape(trials, nb)
        w[:, :, 0] = bits & 0xFF
        w[:, :, 1] = bits >> 8
        act = q8k_acts(rng, trials, nb)
        res = np.empty((trials, 2, 2), np.uint32)
        fns = []
        for sym in forms[name]:
            f = getattr(ref, sym)
            f.argtypes, f.restype = [V, Z, V], F
            fns.append(f)
        for t in range(trials):
            wt, at = np.ascontiguousarray(w[t]), np.ascontiguousarray(act[t])
            for k, blocks in enumerate((1, nb)):
                for j, f in enumerate(fns):
                    res[t, k, j] = np.float32(f(wt.ctypes.data, blocks, at.ctypes.data)).view(np.uint32)
        out[name + "_raw_w"], out[name + "_raw_act"] = w, act
        out[name + "_raw_scalar_bits"], out[name + "_raw_dispatched_bits"] = res[:, :, 0].copy(), res[:, :, 1].copy()
    for qt, rows, cols in ((25, 40, 1280), (36, 33, 768)):
        rb = synth.row_bytes(qt, cols)
        wm = synth.weights(qt, rows, cols, seed=7, stream=qt)
        x = synth.normal(cols, seed=7, stream=100 + qt)
        o = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qt, wm.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data,
                                temp.ctypes.data)
        key = "api%d_" % qt
        out[key + "w"], out[key + "x"] = wm, x
        out[key + "shape"] = np.array([rows, cols, rb], np.int64)
        out[key + "out_bits"] = o.view(np.uint32).copy()
        out[key + "act"] = temp.view(np.uint8)[:cols // 256 * 292].copy()
        n_vec, in_stride, out_stride = 5, cols + 8, rows + 3
        xs = synth.normal(n_vec * in_stride, seed=8, stream=qt).reshape(n_vec, in_stride)
        outs = np.full((n_vec, out_stride), -1.0, np.float32)
        scratch = np.zeros(ref.oc_matvec_batch_scratch_bytes(cols), np.uint8)
        ref.oc_matvec_quantized_batch(qt, wm.ctypes.data, rows, cols, rb, xs.ctypes.data, in_stride,
                                      outs.ctypes.data, out_stride, n_vec, temp.ctypes.data,
                                      scratch.ctypes.data, scratch.nbytes)
        out[key + "batch_x"] = xs
        out[key + "batch_out_bits"] = outs.view(np.uint32).copy()
    for qt, name in ((25, "big_iq3_s_2048x4096"), (36, "big_iq1_xxxs_2048x4096")):
        rows, cols = 2048, 4096
        rb = synth.row_bytes(qt, cols)
        wm = synth.weights(qt, rows, cols, seed=0, stream=0)
        x = synth.normal(cols, seed=0, stream=1000)
        o = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qt, wm.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data,
                                temp.ctypes.data)
        out[name + "_crc_w"] = np.array([zlib.crc32(wm.tobytes())], np.uint32)
        out[name + "_crc_out"] = np.array([zlib.crc32(o.tobytes())], np.uint32)
    np.savez_compressed(os.path.join(HERE, "iq_types.npz"), **out)


def iq4_types(ref):
    """iq4_types.npz: IQ4_NL (type id 26) and IQ4_XS (id 27), the 4-bit codebook formats of the reference's
    dequantise path: rows expanded by oc_quant_dequant_row (raw xorshift bytes behind a finite f16 scale,
    so every nibble, scale nibble and scale high-bit pattern occurs) and oc_matvec_quantized's outputs
    (the dequantise loop, matvec.c:799-831; float bits of THIS host's SIMD dot, held to a tolerance)."""
    rng = np.random.default_rng(20241127)
    out = {}
    for name, qt, bsize, belems in (("iq4_nl", 26, 18, 32), ("iq4_xs", 27, 136, 256)):
        rows, nb = 6, 5
        cols, rb = nb * belems, nb * bsize
        w = xorshift_bytes(rows * rb, 0xC0FFEE ^ qt).reshape(rows * nb, bsize)
        bits = finite_scale_bits(rng, rows * nb)
        w[:, 0], w[:, 1] = bits & 0xFF, bits >> 8
        w = np.ascontiguousarray(w.reshape(-1))
        f = np.zeros((rows, cols), np.float32)
        for r in range(rows):
            assert ref.oc_quant_dequant_row(qt, w[r * rb:].ctypes.data, rb, f[r].ctypes.data, cols) == 0
        out[name + "_w"], out[name + "_bits"] = w, f.view(np.uint32).copy()
        out[name + "_shape"] = np.array([rows, cols, rb], np.int64)
        rows, cols = 48, 1280
        rb = synth.row_bytes(qt, cols)
        wm = synth.weights(qt, rows, cols, seed=9, stream=qt)
        x = synth.normal(cols, seed=9, stream=100 + qt)
        o = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qt, wm.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data, temp.ctypes.data)
        out[name + "_api_w"], out[name + "_api_x"], out[name + "_api_out"] = wm, x, o.copy()
        out[name + "_api_shape"] = np.array([rows, cols, rb], np.int64)
    np.savez_compressed(os.path.join(HERE, "iq4_types.npz"), **out)


def main():
    ref = oxlibs.ref()
    if ref is None:
        raise SystemExit("oracle/_ref/liboxref.so missing: run `make -C oracle` first")
    ref.oc_parallel_set_threads(1)
    only = sys.argv[1] if len(sys.argv) > 1 else None
    if only in (None, "q5_k"):
        q5_k(ref)
    if only in (None, "float"):
        float_steps(ref)
    if only in (None, "dequant"):
        dequant_rows(ref)
    if only in (None, "legacy"):
        legacy_formats(ref)
    if only in (None, "q23_k"):
        q23_k(ref)
    if only in (None, "iq"):
        iq_types(ref)
    if only in (None, "iq4"):
        iq4_types(ref)
    if only is not None:
        return
    rng = np.random.default_rng(20240607)

    # ── scalar helpers ────────────────────────────────────────────────────
    h = np.arange(65536, dtype=np.uint16)
    f16_to_f32 = np.empty(65536, np.uint32)
    two = (ctypes.c_uint8 * 2)()
    for i in range(65536):
        two[0], two[1] = i & 255, i >> 8
        f16_to_f32[i] = np.float32(ref.oc_oxk_f16_le_to_f32(two)).view(np.uint32)
    # f32 -> f16: random magnitudes, exact ties, subnormal range, overflow edge
    parts = [rng.standard_normal(3000).astype(np.float32) * s
             for s in (1e-9, 1e-7, 6e-6, 1e-4, 1e-2, 1.0, 300.0, 7e4)]
    ties = ((np.arange(0x33000000, 0x47800000, 0x2000, dtype=np.uint32) | 0x1000)).view(np.float32)
    near = ((np.arange(0x33000000, 0x47800000, 0x2000, dtype=np.uint32) | 0x0FFF)).view(np.float32)
    edge = np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e10, -1e10, np.inf, -np.inf,
                     5.9604645e-8, 2.9802322e-8, 2.98e-8, 6.0975552e-5, 6.1035156e-5],
                    dtype=np.float32)
    f32_in = np.concatenate(parts + [ties[::37], near[::41], edge]).astype(np.float32)
    f32_to_f16 = np.array([ref.oc_f32_to_f16_bits(float(v)) for v in f32_in], dtype=np.uint16)

    scales = rng.integers(0, 256, (512, 12), dtype=np.uint8)
    sc_out = np.empty((512, 8, 2), np.uint8)
    a = ctypes.c_uint8()
    b = ctypes.c_uint8()
    for i in range(512):
        for j in range(8):
            ref.oc_oxk_get_scale_min_k4(j, scales[i].ctypes.data, ctypes.byref(a), ctypes.byref(b))
            sc_out[i, j] = (a.value, b.value)
    np.savez_compressed(os.path.join(HERE, "scalar_helpers.npz"),
                        f16_to_f32_bits=f16_to_f32, f32_in=f32_in, f32_to_f16_bits=f32_to_f16,
                        k4_scales=scales, k4_sc_min=sc_out)

    # ── raw-block dots (random bytes, finite scales, acts in [-127,127]) ──
    nb, trials = 12, 24
    out = {}
    for name, qt, bsize, d_offs in (("q4_k", Q4K, 144, (0, 2)), ("q6_k", Q6K, 210, (208,)),
                                    ("q8_0", Q80, 34, (0,))):
        w = xorshift_bytes(trials * nb * bsize, 0x9E3779B9 ^ qt).reshape(trials, nb, bsize)
        for off in d_offs:
            bits = finite_scale_bits(rng, trials * nb).reshape(trials, nb)
            w[:, :, off] = bits & 0xFF
            w[:, :, off + 1] = bits >> 8
        if qt == Q80:
            act = np.zeros((trials, nb, 34), np.uint8)
            bits = finite_scale_bits(rng, trials * nb).reshape(trials, nb)
            act[:, :, 0] = bits & 0xFF
            act[:, :, 1] = bits >> 8
            act[:, :, 2:] = rng.integers(-127, 128, (trials, nb, 32)).astype(np.int8).view(np.uint8)
        else:
            act = np.zeros((trials, nb, 292), np.uint8)
            d = (0.001 + rng.integers(0, 1000, (trials, nb)) * 2e-5).astype(np.float32)
            act[:, :, 0:4] = d.view(np.uint8).reshape(trials, nb, 4)
            q = rng.integers(-127, 128, (trials, nb, 256)).astype(np.int8)
            act[:, :, 4:260] = q.view(np.uint8)
            bs = q.reshape(trials, nb, 16, 16).sum(axis=3).astype(np.int16)
            act[:, :, 260:292] = bs.view(np.uint8).reshape(trials, nb, 32)
        scalar = np.empty((trials, 2), np.uint32)
        disp = np.empty((trials, 2), np.uint32)
        fs = getattr(ref, "oc_oxk_dot_%s_%s_scalar" % (name, "q8_0" if qt == Q80 else "q8_k"))
        fd = getattr(ref, "oc_oxk_dot_%s_%s" % (name, "q8_0" if qt == Q80 else "q8_k"))
        for t in range(trials):
            wt = np.ascontiguousarray(w[t])
            at = np.ascontiguousarray(act[t])
            for k, blocks in enumerate((1, nb)):
                scalar[t, k] = np.float32(fs(wt.ctypes.data, blocks, at.ctypes.data)).view(np.uint32)
                disp[t, k] = np.float32(fd(wt.ctypes.data, blocks, at.ctypes.data)).view(np.uint32)
        out[name + "_w"] = w
        out[name + "_act"] = act
        out[name + "_scalar_bits"] = scalar
        out[name + "_dispatched_bits"] = disp
    np.savez_compressed(os.path.join(HERE, "raw_block_dots.npz"), **out)

    # ── API level: small matrices stored whole ───────────────────────────
    api = {}
    for name, qt, rows, cols in (("q4_k", Q4K, 48, 1024), ("q6_k", Q6K, 24, 768), ("q8_0", Q80, 40, 896)):
        rb = synth.row_bytes(qt, cols)
        w = synth.weights(qt, rows, cols, seed=7, stream=qt)
        x = synth.normal(cols, seed=7, stream=100 + qt)
        o = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data,
                                temp.ctypes.data)
        nact = cols // synth.BLOCK_ELEMS[qt] * (34 if qt == Q80 else 292)
        api[name + "_w"] = w
        api[name + "_x"] = x
        api[name + "_shape"] = np.array([rows, cols, rb], np.int64)
        api[name + "_out_bits"] = o.view(np.uint32).copy()
        api[name + "_act"] = temp.view(np.uint8)[:nact].copy()
        # batch with padded strides, 5 vectors
        n_vec, in_stride, out_stride = 5, cols + 8, rows + 3
        xs = synth.normal(n_vec * in_stride, seed=8, stream=qt).reshape(n_vec, in_stride)
        outs = np.full((n_vec, out_stride), -1.0, np.float32)
        scratch = np.zeros(ref.oc_matvec_batch_scratch_bytes(cols), np.uint8)
        ref.oc_matvec_quantized_batch(qt, w.ctypes.data, rows, cols, rb, xs.ctypes.data, in_stride,
                                      outs.ctypes.data, out_stride, n_vec, temp.ctypes.data,
                                      scratch.ctypes.data, scratch.nbytes)
        api[name + "_batch_x"] = xs
        api[name + "_batch_out_bits"] = outs.view(np.uint32).copy()
    np.savez_compressed(os.path.join(HERE, "matvec_api.npz"), **api)

    # ── full-size benchmark configuration 0 and friends: checksums ───────
    big = {}
    for name, qt, rows, cols in (("cfg0_q4k_4096x4096", Q4K, 4096, 4096),
                                 ("down_q6k_4096x14336", Q6K, 4096, 14336),
                                 ("ffn_q80_4864x896", Q80, 4864, 896)):
        rb = synth.row_bytes(qt, cols)
        w = synth.weights(qt, rows, cols, seed=0, stream=0)
        x = synth.normal(cols, seed=0, stream=1000)
        o = np.zeros(rows, np.float32)
        temp = np.zeros(cols, np.float32)
        ref.oc_matvec_quantized(qt, w.ctypes.data, rows, cols, rb, x.ctypes.data, o.ctypes.data,
                                temp.ctypes.data)
        nact = cols // synth.BLOCK_ELEMS[qt] * (34 if qt == Q80 else 292)
        big[name + "_crc_w"] = np.array([zlib.crc32(w.tobytes())], np.uint32)
        big[name + "_crc_x"] = np.array([zlib.crc32(x.tobytes())], np.uint32)
        big[name + "_crc_act"] = np.array([zlib.crc32(temp.view(np.uint8)[:nact].tobytes())], np.uint32)
        big[name + "_crc_out"] = np.array([zlib.crc32(o.tobytes())], np.uint32)
        big[name + "_out"] = o.copy()
    np.savez_compressed(os.path.join(HERE, "full_size.npz"), **big)
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
