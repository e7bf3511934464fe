#!/usr/bin/env python3
"""Benchmark of the quantized-matvec hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode token of the Llama-3-8B-shaped GEMV set: 32 layers x
{fused q/k/v, o, fused gate/up (Q4_K), down (Q6_K)}, every GEMV preceded by
the Q8_K quantisation of its own f32 input (done inside the kernel).  The 128
matmuls of a step run as ONE launch of the persistent plan kernel (oxh_plan);
`--mode graph` runs them as 128 launches replayed as one HIP graph instead,
and that figure is reported next to the headline one either way.  All inputs
are resident in HBM before the timed region starts.

Prints ONE JSON line.  `value` is whole-step algorithmic GB/s (packed weights
at their on-disk size + f32 activations in + f32 outputs out, divided by the
wall time of the K timed steps).  `roofline` is the kernel the step runs in
(k_plan_ext: one launch = one step, every input quantised once ahead of the
chain), timed with HIP events on the launch stream.
`cpu_baseline` is the reference's own CPU code (oracle/_ref, or the oracle
port when that was never built) on this host's cores, streaming eight distinct
layers in turn (1.1 GB: beyond the host's last-level cache).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes one gate/up launch moves, from two rocprofv3 --pmc runs (FETCH_SIZE
# 32410.7 KiB x 2.000, WRITE_SIZE 116.57 KiB x 1.000; the factors are what the
# same counters read for a 256 MiB device-to-device copy).  Not measured live.
GATE_UP_TRAFFIC_BYTES = 66496518
# HBM bytes one k_plan_ext launch (a whole 32-layer step) moves, measured the same way: FETCH_SIZE
# 2170528.0 KiB x 1.9998, WRITE_SIZE 7322.03 KiB x 1.000 (algorithmic: 4419223552, ratio 1.0075).
PLAN_STEP_TRAFFIC_BYTES = 4441622891
INT8_PEAK_TOPS = 5033.0     # dense int8 MFMA: 256 CU x 2.4 GHz x 8192 op/clk/CU


LEG_SPINUP_MS = 50.0        # --leg-spinup-ms


def timed(fn, reps, mv):
    """Average microseconds of fn() over `reps` back-to-back calls (HIP events), after LEG_SPINUP_MS
    milliseconds of the same calls untimed: between two legs the host generates and uploads data while the
    device idles, and the first tens of launches after that run slower (an expert step 171 us where it settles
    at 161).  Runs under a tracing profiler pass --leg-spinup-ms 0: the untimed calls multiply the dispatches
    it has to record."""
    fn()
    mv.sync()
    t_spin = time.perf_counter()
    while (time.perf_counter() - t_spin) * 1e3 < LEG_SPINUP_MS:
        for _ in range(4):
            fn()
        mv.sync()
    e0, e1 = mv.Event(), mv.Event()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    mv.sync()
    return e1.ms_since(e0) * 1e3 / reps


def chain_figure(mv, ds, steps):
    """The same 32 layers as a dependent chain, with the float steps a decode
    layer runs between its matmuls (residual add + RMSNorm in front of q/k/v and
    of gate/up, SwiGLU behind gate/up) fused into the four matmuls of a layer:
    as one launch of the plan kernel, and as 128 launches in a graph."""
    from oxidize_amd.workloads import DecodeChain
    chain = DecodeChain(ds)
    graph = mv.Graph()
    with graph:
        chain.launch_step()
    us_graph = timed(graph.launch, max(5, steps), mv)
    chain2 = DecodeChain(ds)
    plan = mv.Plan(chain2.plan_ops())
    us = timed(plan.launch, max(5, steps), mv)
    assert plan.status() == 0
    waits = plan.info()["n_waits"]
    plan.destroy()
    nbytes = chain.bytes_per_step
    return {"us_per_step": round(us, 1), "gbps": round(nbytes / us / 1e3, 1),
            "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
            "launches_per_step": 1, "waits_per_step": waits, "bytes_per_step": nbytes,
            "as_graph_of_128_launches_us": round(us_graph, 1),
            "note": "attention itself is outside this library: the q projection stands in for its "
                    "output so that every launch depends on the previous one"}


def _lib_check_memset(buf):
    import ctypes
    from oxidize_amd import _lib
    _lib.check(_lib.lib().oxh_memset(ctypes.c_void_p(buf.ptr), 0x5A, buf.nbytes, None))


def secondary_figures(mv, synth):
    """The other benchmark configurations, measured the same way (inputs
    resident, HIP events on the launch stream).  Reported next to the headline
    figure, never folded into it."""
    from oxidize_amd.workloads import MoESet
    out = {}
    Q80, Q4K = 7, 13
    # MMQ prefill (configuration 3): 512 tokens, Q4_K 14336x4096 and 4096x4096
    cols, n_vec = 4096, 512
    x = synth.normal(n_vec * cols, seed=0, stream=2000)
    d_x = mv.DeviceBuffer.from_host(x)
    d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(Q4K, cols))
    mmq = {}
    for rows in (14336, 4096):
        w = synth.weights(Q4K, rows, cols, seed=0, stream=0)
        copies = [mv.DeviceBuffer.from_host(w) for _ in range(3)]
        d_o = mv.DeviceBuffer(n_vec * rows * 4)
        state = {"i": 0}

        def run():
            state["i"] += 1
            mv.quantize(Q4K, d_x.ptr, cols, n_vec, cols, d_a.ptr)
            mv.mmq(Q4K, copies[state["i"] % 3].ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows)

        def run_mma_only():
            state["i"] += 1
            mv.mmq(Q4K, copies[state["i"] % 3].ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows)

        def run_mma_relaxed():
            state["i"] += 1
            mv.mmq(Q4K, copies[state["i"] % 3].ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows, flags=mv.MMQ_RELAXED)

        us = timed(run, 12, mv)
        us_mma = timed(run_mma_only, 12, mv)
        us_rel = timed(run_mma_relaxed, 12, mv)
        ops = 2.0 * rows * cols * n_vec
        mmq["%dx%dx%d" % (rows, cols, n_vec)] = {
            "us": round(us, 2), "tops": round(ops / us / 1e6, 1),
            "frac_of_int8_peak": round(ops / us / 1e6 / INT8_PEAK_TOPS, 4),
            "includes": "Q8_K quantisation of the 512 activations + k_mmq_q4_k",
            "mfma_kernel_only_us": round(us_mma, 2),
            "mfma_kernel_only_frac_of_int8_peak": round(ops / us_mma / 1e6 / INT8_PEAK_TOPS, 4),
            "relaxed_float_step_opt_in": {"mfma_kernel_only_us": round(us_rel, 2),
                                          "frac_of_int8_peak": round(ops / us_rel / 1e6 / INT8_PEAK_TOPS, 4),
                                          "note": "OXH_MMQ_RELAXED: within 1e-5*|exact| + 2e-6*rms(outputs) of the exact outputs"}}
        for c in copies:
            c.free()
    out["mmq_prefill_q4k"] = mmq
    # what bounds that kernel: int8 MFMA rate of the device with 0 / 1 / 2 / 4 independent vector instructions
    # after every MFMA, at two and four waves per SIMD (they do not overlap on this device)
    import ctypes
    from oxidize_amd import _lib
    probe = {}
    for nv in (0, 1, 2, 4):
        for wps in (2, 4):
            pops = ctypes.c_double()
            if _lib.lab().mfma_probe(nv, wps, ctypes.byref(pops)) == 0:
                probe["valu_%d_per_mfma_%d_waves_per_simd" % (nv, wps)] = round(pops.value, 3)
    out["int8_mfma_pops_with_vector_work_beside"] = probe
    d_x.free()
    d_a.free()
    # the down projection of the same model is Q6_K: 4096 x 14336, 512 tokens
    Q6K = 16
    rows, cols = 4096, 14336
    x = synth.normal(n_vec * cols, seed=0, stream=2001)
    d_x = mv.DeviceBuffer.from_host(x)
    d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(Q6K, cols))
    w = synth.weights(Q6K, rows, cols, seed=0, stream=3)
    copies = [mv.DeviceBuffer.from_host(w) for _ in range(3)]
    d_o = mv.DeviceBuffer(n_vec * rows * 4)
    mv.quantize(Q6K, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    state = {"i": 0}

    def run_q6():
        state["i"] += 1
        mv.mmq(Q6K, copies[state["i"] % 3].ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows)

    us = timed(run_q6, 12, mv)
    ops = 2.0 * rows * cols * n_vec
    out["mmq_prefill_q6k"] = {"%dx%dx%d" % (rows, cols, n_vec): {
        "mfma_kernel_only_us": round(us, 2), "tops": round(ops / us / 1e6, 1),
        "mfma_kernel_only_frac_of_int8_peak": round(ops / us / 1e6 / INT8_PEAK_TOPS, 4)}}
    for c in copies:
        c.free()
    d_x.free()
    d_a.free()
    d_o.free()
    # Q5_K (the other K-quant behind the same API): decode GEMV and 512-token
    # prefill at the gate/up shape, 28672 x 4096
    Q5K = 15
    rows, cols = 28672, 4096
    w = synth.weights(Q5K, rows, cols, seed=0, stream=4)
    copies = [mv.DeviceBuffer.from_host(w) for _ in range(8)]    # 646 MB: beyond the last-level cache
    x = synth.normal(n_vec * cols, seed=0, stream=2002)
    d_x = mv.DeviceBuffer.from_host(x)
    d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(Q5K, cols))
    d_o = mv.DeviceBuffer(n_vec * rows * 4)
    segs = [mv.make_segments([(c.ptr, d_o.ptr, rows, 0)]) for c in copies]
    state = {"i": 0}

    def run_q5_gemv():
        state["i"] += 1
        mv.gemv_segments_f32(Q5K, segs[state["i"] % 8], cols, d_x.ptr, cols, None, 1, rows)

    def run_q5_mmq():
        state["i"] += 1
        mv.mmq(Q5K, copies[state["i"] % 8].ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows)

    us = timed(run_q5_gemv, 32, mv)
    nbytes = w.nbytes + 4 * cols + 4 * rows
    mv.quantize(Q5K, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    us_mma = timed(run_q5_mmq, 12, mv)
    ops = 2.0 * rows * cols * n_vec
    out["q5k_28672x4096"] = {
        "gemv_batch1": {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                        "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)},
        "mmq_512_tokens": {"mfma_kernel_only_us": round(us_mma, 2), "tops": round(ops / us_mma / 1e6, 1),
                           "mfma_kernel_only_frac_of_int8_peak": round(ops / us_mma / 1e6 / INT8_PEAK_TOPS, 4)}}
    for c in copies:
        c.free()
    d_x.free()
    d_a.free()
    d_o.free()
    # the remaining weight types behind the same entry points: batch-1 GEMV at the gate/up shape,
    # eight distinct copies in turn (beyond the last-level cache)
    others = {}
    x = synth.normal(cols, seed=0, stream=2003)
    d_x = mv.DeviceBuffer.from_host(x)
    d_o = mv.DeviceBuffer(rows * 4)
    for name, qt in (("q2_k", 8), ("q3_k", 10), ("q4_0", 3), ("q4_1", 4), ("q5_0", 5), ("q5_1", 6),
                     ("iq3_s", 25), ("iq1_xxxs", 36), ("iq4_nl_f32_inputs", 26), ("iq4_xs_f32_inputs", 27)):
        w = synth.weights(qt, rows, cols, seed=0, stream=7)
        copies = [mv.DeviceBuffer.from_host(w) for _ in range(8)]
        segs = [mv.make_segments([(c.ptr, d_o.ptr, rows, 0)]) for c in copies]
        state = {"i": 0}

        def run_other():
            state["i"] += 1
            mv.gemv_segments_f32(qt, segs[state["i"] % 8], cols, d_x.ptr, cols, None, 1, rows)

        us = timed(run_other, 32, mv)
        nbytes = w.nbytes + 4 * cols + 4 * rows
        others[name] = {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                        "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
        for c in copies:
            c.free()
    d_x.free()
    d_o.free()
    out["other_types_gemv_28672x4096"] = others
    # Q2_K and Q3_K prefill (512 tokens, 14336 x 4096): the matrix is rewritten into 210-byte blocks
    # and then runs on the Q6_K tile kernel; both steps timed, Q8_K activations already made
    rows, cols = 14336, 4096
    x = synth.normal(n_vec * cols, seed=0, stream=2004)
    d_x = mv.DeviceBuffer.from_host(x)
    d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(Q6K, cols))
    mv.quantize(Q6K, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    d_o = mv.DeviceBuffer(n_vec * rows * 4)
    d_wide = mv.DeviceBuffer(rows * (cols // 256) * 210)
    pre = {}
    for name, qt in (("q2_k", 8), ("q3_k", 10)):
        d_w = mv.DeviceBuffer.from_host(synth.weights(qt, rows, cols, seed=0, stream=8))
        if qt == 8:
            def rewrite():
                mv.q2_k_widen(d_w.ptr, rows, cols, d_wide.ptr)
            as_type = mv.Q2_K_WIDE
        else:
            def rewrite():
                mv.q3_k_as_q6_k(d_w.ptr, rows, cols, d_wide.ptr)
            as_type = Q6K

        def tiles():
            mv.mmq(as_type, d_wide.ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows)

        us_rw = timed(rewrite, 12, mv)
        us_mma = timed(tiles, 12, mv)
        ops = 2.0 * rows * cols * n_vec
        pre[name] = {"rewrite_us": round(us_rw, 2), "mfma_kernel_only_us": round(us_mma, 2),
                     "tops": round(ops / (us_rw + us_mma) / 1e6, 1),
                     "frac_of_int8_peak": round(ops / (us_rw + us_mma) / 1e6 / INT8_PEAK_TOPS, 4)}
        d_w.free()
    out["q2k_q3k_prefill_14336x4096x512"] = pre
    for b_ in (d_x, d_a, d_o, d_wide):
        b_.free()
    # the 32-value formats, 512 activations: 128 x 64 tiles, one 16x16x32 MFMA per block and token chunk
    rows, cols, nv = 4096, 4096, 512
    d_x = mv.DeviceBuffer.from_host(synth.normal(nv * cols, seed=0, stream=2009))
    d_a = mv.DeviceBuffer(nv * mv.act_bytes(Q80, cols))
    d_o = mv.DeviceBuffer(nv * rows * 4)
    mv.quantize(Q80, d_x.ptr, cols, nv, cols, d_a.ptr)
    pre32 = {}
    for name, qt in (("q8_0", Q80), ("q4_0", 3), ("q5_1", 6)):
        d_w = mv.DeviceBuffer.from_host(synth.weights(qt, rows, cols, seed=0, stream=2010 + qt))
        us = timed(lambda: mv.mmq(qt, d_w.ptr, rows, cols, d_a.ptr, nv, d_o.ptr, rows), 20, mv)
        ops = 2.0 * rows * cols * nv
        pre32[name] = {"mfma_kernel_only_us": round(us, 2), "tops": round(ops / us / 1e6, 1),
                       "frac_of_int8_peak": round(ops / us / 1e6 / INT8_PEAK_TOPS, 4)}
        d_w.free()
    pre32["note"] = ("exact per-block float step: four vector operations per output and 32-value block beside one "
                     "16x16x32 MFMA per 256 outputs")
    out["q8_0_family_prefill_4096x4096x512"] = pre32
    for b_ in (d_x, d_a, d_o):
        b_.free()
    # configuration 0 (the reference's own CPU-runnable case): one 4096 x 4096 Q4_K matvec, over 32 distinct
    # copies in turn (302 MB: from HBM) and over one copy again and again (resident in the last-level cache)
    rows, cols = 4096, 4096
    w = synth.weights(Q4K, rows, cols, seed=0, stream=0)
    copies = [mv.DeviceBuffer.from_host(w) for _ in range(32)]
    d_x = mv.DeviceBuffer.from_host(synth.normal(cols, seed=0, stream=2005))
    d_o = mv.DeviceBuffer(rows * 4)
    segs = [mv.make_segments([(c.ptr, d_o.ptr, rows, 0)]) for c in copies]
    state = {"i": 0}

    def run_cold():
        state["i"] += 1
        mv.gemv_segments_f32(Q4K, segs[state["i"] % 32], cols, d_x.ptr, cols, None, 1, rows)

    def run_hot():
        mv.gemv_segments_f32(Q4K, segs[0], cols, d_x.ptr, cols, None, 1, rows)

    nbytes = w.nbytes + 4 * cols + 4 * rows
    us_cold, us_hot = timed(run_cold, 64, mv), timed(run_hot, 64, mv)
    out["q4k_gemv_4096x4096_config0"] = {
        "cold": {"us": round(us_cold, 2), "gbps": round(nbytes / us_cold / 1e3, 1)},
        "cache_resident": {"us": round(us_hot, 2), "gbps": round(nbytes / us_hot / 1e3, 1)},
        "note": "back-to-back launches on one stream, launch gaps included"}
    for c in copies:
        c.free()
    d_x.free()
    d_o.free()
    # the host-pointer entry point itself (never `value`: inputs and outputs cross the bus on every call):
    # oc_matvec_quantized's wall time per call from this process, weights resident after the first call
    host_api = {}
    for name, qt, r_, c_ in (("q4_k_4096x4096", Q4K, 4096, 4096), ("q4_k_14336x4096", Q4K, 14336, 4096),
                             ("q6_k_4096x14336", Q6K, 4096, 14336)):
        w = synth.weights(qt, r_, c_, seed=0, stream=11)
        x = synth.normal(c_, seed=0, stream=2010)
        import numpy as np
        o_, t_ = np.zeros(r_, np.float32), np.zeros(c_, np.float32)
        rb = synth.row_bytes(qt, c_)
        # the call as a C program makes it: the eight arguments made once (finding a numpy array's address
        # costs this interpreter 3 us per call, which is not the library's time)
        import ctypes
        from oxidize_amd import _lib
        call = _lib.lib().oxh_matvec_quantized
        cargs = (ctypes.c_uint32(qt), ctypes.c_void_p(w.ctypes.data), ctypes.c_size_t(r_), ctypes.c_size_t(c_),
                 ctypes.c_size_t(rb), ctypes.c_void_p(x.ctypes.data), ctypes.c_void_p(o_.ctypes.data),
                 ctypes.c_void_p(t_.ctypes.data))
        mv.matvec_quantized(qt, w, r_, c_, rb, x, o_, t_)
        best = None
        for rep in range(4):
            t0 = time.perf_counter()
            for _ in range(100):
                rc = call(*cargs)
            dt = (time.perf_counter() - t0) / 100 * 1e6
            assert rc == 0
            best = dt if best is None or dt < best else best
        host_api[name] = round(best, 1)
    from oxidize_amd import _lib
    _lib.check(_lib.lib().oxh_weight_clear())
    out["host_pointer_api_us_per_call"] = host_api
    # small batches over the decode matrices with few rows: the dot kernels (up to eight activations), one
    # workgroup per 64 x 16 tile (oxh_mmq), and the tiles' columns shared between workgroups (oxh_mmq_split)
    small = {}
    for name, qt, r_, c_ in (("q6_k_4096x14336", Q6K, 4096, 14336), ("q4_k_4096x4096", Q4K, 4096, 4096)):
        w = synth.weights(qt, r_, c_, seed=0, stream=12)
        copies = [mv.DeviceBuffer.from_host(w) for _ in range(6)]
        per = {}
        for nv in (4, 8, 16):
            d_x = mv.DeviceBuffer.from_host(synth.normal(nv * c_, seed=0, stream=2011))
            d_a = mv.DeviceBuffer(nv * mv.act_bytes(qt, c_))
            d_o = mv.DeviceBuffer(nv * r_ * 4)
            mv.quantize(qt, d_x.ptr, c_, nv, c_, d_a.ptr)
            need = mv.mmq_split_workspace(qt, r_, c_, nv, r_)
            d_ws = mv.DeviceBuffer(max(need, 16))
            segs = [mv.make_segments([(c.ptr, d_o.ptr, r_, 0)]) for c in copies]
            state = {"i": 0}

            def run_dot():
                state["i"] += 1
                mv.gemv_segments(qt, segs[state["i"] % 6], c_, d_a.ptr, nv, r_)

            def run_tiles():
                state["i"] += 1
                mv.mmq(qt, copies[state["i"] % 6].ptr, r_, c_, d_a.ptr, nv, d_o.ptr, r_)

            def run_split():
                state["i"] += 1
                mv.mmq_split(qt, copies[state["i"] % 6].ptr, r_, c_, d_a.ptr, nv, d_o.ptr, r_, d_ws.ptr, need)

            row = {"one_workgroup_per_tile_us": round(timed(run_tiles, 24, mv), 1)}
            if nv <= 8:
                row["dot_kernel_us"] = round(timed(run_dot, 24, mv), 1)
            if need:
                row["columns_shared_us"] = round(timed(run_split, 24, mv), 1)
            per["batch%d" % nv] = row
            for b_ in (d_x, d_a, d_o, d_ws):
                b_.free()
        small[name] = per
        for c in copies:
            c.free()
    out["small_batches_few_rows"] = small
    # the Q6_K down projection in the two layouts the decode kernels read: the file layout and the
    # regrouped copy the decode set keeps (same bytes); eight distinct copies in turn (386 MB: from HBM)
    rows, cols = 4096, 14336
    w = synth.weights(Q6K, rows, cols, seed=0, stream=7)
    plain = [mv.DeviceBuffer.from_host(w) for _ in range(8)]
    grouped = []
    for c in plain:
        g = mv.DeviceBuffer(w.nbytes)
        mv.q6_k_group(c.ptr, rows, cols, g.ptr)
        grouped.append(g)
    mv.sync()
    d_x = mv.DeviceBuffer.from_host(synth.normal(cols, seed=0, stream=2006))
    d_o = mv.DeviceBuffer(rows * 4)
    seg_p = [mv.make_segments([(c.ptr, d_o.ptr, rows, 0)]) for c in plain]
    seg_g = [mv.make_segments([(c.ptr, d_o.ptr, rows, 0)]) for c in grouped]
    state = {"i": 0}

    def run_plain():
        state["i"] += 1
        mv.gemv_segments_f32(Q6K, seg_p[state["i"] % 8], cols, d_x.ptr, cols, None, 1, rows)

    def run_grouped():
        state["i"] += 1
        mv.gemv_segments_f32(mv.Q6_K_G8, seg_g[state["i"] % 8], cols, d_x.ptr, cols, None, 1, rows)

    nbytes = w.nbytes + 4 * cols + 4 * rows
    us_p, us_g = timed(run_plain, 64, mv), timed(run_grouped, 64, mv)
    out["q6k_down_4096x14336_layouts"] = {
        "file_layout": {"us": round(us_p, 2), "gbps": round(nbytes / us_p / 1e3, 1)},
        "regrouped_in_eights": {"us": round(us_g, 2), "gbps": round(nbytes / us_g / 1e3, 1)},
        "note": "k_gemv_q6_k against k_gemv_q6_kg, back-to-back launches, launch gaps included"}
    for c in plain + grouped:
        c.free()
    d_x.free()
    d_o.free()
    # Q8_0 lm_head (configuration 2), batch 1, 2, 4 and 8
    rows, cols = 151936, 896
    w = synth.weights(Q80, rows, cols, seed=0, stream=5)
    copies = [mv.DeviceBuffer.from_host(w) for _ in range(3)]
    # the same three copies rewritten tile-major once (oxh_tile16: the blocks as the matrix cores' operand
    # wants them; same bytes and bit-identical results)
    tiled = [mv.DeviceBuffer(mv.tile16_bytes(Q80, rows, cols)) for _ in range(3)]
    for c, t in zip(copies, tiled):
        mv.tile16(Q80, c.ptr, rows, cols, t.ptr)
    mv.sync()
    q8 = {}
    for nv in (1, 2, 4, 8, 16):
        xs = synth.normal(nv * cols, seed=0, stream=6)
        d_x = mv.DeviceBuffer.from_host(xs)
        d_o = mv.DeviceBuffer(nv * rows * 4)
        d_qa = mv.DeviceBuffer(nv * mv.act_bytes(Q80, cols))    # room for the quantised activations
        state = {"i": 0}
        nbytes = w.nbytes + nv * 4 * (cols + rows)
        leg = {}
        for label, qt, bufs in (("file_layout", Q80, copies), ("tile_major", mv.Q8_0_T16, tiled)):
            def run():
                state["i"] += 1
                segs = mv.make_segments([(bufs[state["i"] % 3].ptr, d_o.ptr, rows, 0)])
                mv.gemv_segments_f32(qt, segs, cols, d_x.ptr, cols, d_qa.ptr, nv, rows)

            us = timed(run, 12, mv)
            leg[label] = {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                          "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
        # the top-level figures of a batch are the file layout's (what a caller gets with no preparation)
        q8["batch%d" % nv] = dict(leg["file_layout"], tile_major=leg["tile_major"])
        d_x.free()
        d_o.free()
        d_qa.free()
    out["q8_0_lm_head_151936x896"] = q8
    for c in copies + tiled:
        c.free()
    # the feed-forward matrices of the same configuration (4864 x 896 and 896 x 4864, 4.6 MB each) at batch
    # 1, 2, 4 and 8: 48 distinct copies in turn (222 MB), single launches, launch gaps included
    ffn = {}
    for name, r_, c_ in (("gate_or_up_4864x896", 4864, 896), ("down_896x4864", 896, 4864)):
        w = synth.weights(Q80, r_, c_, seed=0, stream=9)
        copies = [mv.DeviceBuffer.from_host(w) for _ in range(48)]
        per = {}
        for nv in (1, 2, 4, 8):
            d_x = mv.DeviceBuffer.from_host(synth.normal(nv * c_, seed=0, stream=10))
            d_o = mv.DeviceBuffer(nv * r_ * 4)
            d_qa = mv.DeviceBuffer(nv * mv.act_bytes(Q80, c_))
            segs = [mv.make_segments([(c.ptr, d_o.ptr, r_, 0)]) for c in copies]
            state = {"i": 0}

            def run_ffn():
                state["i"] += 1
                mv.gemv_segments_f32(Q80, segs[state["i"] % 48], c_, d_x.ptr, c_, d_qa.ptr, nv, r_)

            us = timed(run_ffn, 96, mv)
            nbytes = w.nbytes + nv * 4 * (c_ + r_)
            per["batch%d" % nv] = {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                                   "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
            for b_ in (d_x, d_o, d_qa):
                b_.free()
        ffn[name] = per
        for c in copies:
            c.free()
    ffn["note"] = ("a launch over 4.6 MB is paced by its dependent chain (launch, input, quantise, one pass, row sums), "
                   "not by the bytes: the whole-step figure below is the one that streams")
    out["q8_0_ffn_shapes_batch_1_to_8"] = ffn
    # configuration 2 as a whole decode step: the Qwen2.5-0.5B-shaped Q8_0 set (24 layers x {q/k/v, o,
    # gate/up, down} + the head, every matmul quantising its own f32 input to Q8_0; matrices of 0.9-9 MB
    # and the 145 MB head) as ONE launch (a plan over a 32-value format: the rows of all 97 operations
    # cut into runs and dealt to the workgroups by bytes), and as a graph of 97 launches beside it
    from oxidize_amd.workloads import DecodeSet, QWEN2_5_0_5B
    qs = DecodeSet(qtypes=(Q80, Q80), seed=0, **QWEN2_5_0_5B)
    w = synth.weights(Q80, rows, cols, seed=0, stream=5)
    d_head = mv.DeviceBuffer.from_host(w)
    d_hx = mv.DeviceBuffer.from_host(synth.normal(cols, seed=0, stream=8))
    d_ho = mv.DeviceBuffer(rows * 4)
    head_seg = mv.make_segments([(d_head.ptr, d_ho.ptr, rows, 0)])

    def qwen_step():
        qs.launch_step()
        mv.gemv_segments_f32(Q80, head_seg, cols, d_hx.ptr, cols, None, 1, rows)

    qwen_step()
    mv.sync()
    graph = mv.Graph()
    with graph:
        qwen_step()
    us_graph = timed(graph.launch, 20, mv)
    graph.destroy()
    qplan = mv.Plan(qs.plan_ops() + [dict(qtype=Q80, segs=head_seg, cols=cols, d_x=d_hx.ptr, d_act_out=None)])
    us = timed(qplan.launch, 20, mv)
    assert qplan.status() == 0
    qplan.destroy()
    nbytes = qs.bytes_per_step + w.nbytes + 4 * (cols + rows)
    out["q8_0_decode_step_qwen2_5_0_5b"] = {
        "us_per_step": round(us, 1), "launches_per_step": 1, "operations_per_step": qs.layers * len(qs.ops) + 1,
        "bytes_per_step": nbytes, "gbps": round(nbytes / us / 1e3, 1),
        "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
        "as_graph_of_97_launches_us": round(us_graph, 1),
        "note": "independent operations (every input there when the launch starts); no workgroup waits for another"}
    # the same step for a batch of eight activations per matmul, as a graph of launches (a plan over a 32-value
    # format takes one activation per operation): the layers from the file layout (dot or matrix-core kernel by
    # launch size), the head from a tile-major copy
    nvb = 8
    bx, bo, ba, bsegs = [], [], [], []
    for layer in range(qs.layers):
        for op, (name, qt, rows_, cols_, _) in enumerate(qs.ops):
            tot = sum(rows_)
            x = mv.DeviceBuffer.from_host(synth.normal(nvb * cols_, seed=0, stream=500000 + layer * 8 + op))
            o = mv.DeviceBuffer(nvb * tot * 4)
            aq = mv.DeviceBuffer(nvb * mv.act_bytes(qt, cols_))
            items, off = [], 0
            for seg, r_ in enumerate(rows_):
                items.append((qs.weights[layer][op][seg].ptr, o.ptr + off * 4, r_, 0))
                off += r_
            bx.append(x); bo.append(o); ba.append(aq)
            bsegs.append((mv.make_segments(items), cols_, tot))
    d_head16 = mv.DeviceBuffer(mv.tile16_bytes(Q80, rows, cols))
    mv.tile16(Q80, d_head.ptr, rows, cols, d_head16.ptr)
    d_hx8 = mv.DeviceBuffer.from_host(synth.normal(nvb * cols, seed=0, stream=9))
    d_ho8 = mv.DeviceBuffer(nvb * rows * 4)
    d_ha8 = mv.DeviceBuffer(nvb * mv.act_bytes(Q80, cols))
    head16_seg = mv.make_segments([(d_head16.ptr, d_ho8.ptr, rows, 0)])

    def qwen_step_batch():
        for (segs, cols_, tot), x, aq in zip(bsegs, bx, ba):
            mv.gemv_segments_f32(Q80, segs, cols_, x.ptr, cols_, aq.ptr, nvb, tot)
        mv.gemv_segments_f32(mv.Q8_0_T16, head16_seg, cols, d_hx8.ptr, cols, d_ha8.ptr, nvb, rows)

    qwen_step_batch()
    mv.sync()
    graph = mv.Graph()
    with graph:
        qwen_step_batch()
    us_b = timed(graph.launch, 20, mv)
    graph.destroy()
    out["q8_0_decode_step_qwen2_5_0_5b"]["batch8_as_graph_of_launches_us"] = round(us_b, 1)
    out["q8_0_decode_step_qwen2_5_0_5b"]["batch8_note"] = (
        "eight activations per matmul, 97 operations as a graph (the layers' matrices from the file layout, the "
        "145 MB head from its tile-major copy); per activation %.1f us against %.1f us for the batch-1 step as one "
        "launch: launches over matrices of 0.9-9 MB are paced by their own dependent chain (8-18 us each at eight "
        "activations), so eight single-activation plan launches (%.0f us) beat one batched step of launches"
        % (us_b / nvb, us, nvb * us))
    # The same eight-activation step with EVERY matrix tile-major and the independent operations of one input
    # width grouped into launches of up to 32 segments (each segment its own run of eight activations): every
    # launch then has thousands of 16-row groups to deal to its waves, where a launch over one small matrix
    # has a few hundred.  Inputs are quantised by one launch per width.
    groups = {}
    for idx, ((segs_, cols_, tot), x) in enumerate(zip(bsegs, bx)):
        groups.setdefault(cols_, []).append(idx)
    tiled_keep, launches, t16_of = [], [], {}
    for cols_, idxs in groups.items():
        n_in = len(idxs) * nvb
        xin = mv.DeviceBuffer(n_in * cols_ * 4)
        for j, idx in enumerate(idxs):
            _lib_check_copy(xin.ptr + j * nvb * cols_ * 4, bx[idx].ptr, nvb * cols_ * 4)
        aq = mv.DeviceBuffer(n_in * mv.act_bytes(Q80, cols_))
        items = []
        for j, idx in enumerate(idxs):
            layer, op = divmod(idx, len(qs.ops))
            name, qt, rows_, _, _ = qs.ops[op]
            off = 0
            for seg, r_ in enumerate(rows_):
                t16 = mv.DeviceBuffer(mv.tile16_bytes(Q80, r_, cols_))
                mv.tile16(Q80, qs.weights[layer][op][seg].ptr, r_, cols_, t16.ptr)
                tiled_keep.append(t16)
                t16_of[(idx, seg)] = t16
                items.append((t16.ptr, bo[idx].ptr + off * 4, r_, j * nvb, nvb, sum(rows_)))
                off += r_
        tiled_keep += [xin, aq]
        # segments of one launch share the output stride: group them by it
        by_stride = {}
        for it in items:
            by_stride.setdefault(it[5], []).append(it[:5])
        for stride, its in by_stride.items():
            for k in range(0, len(its), 32):
                launches.append((mv.make_segments(its[k:k + 32]), cols_, aq, stride))
        launches.append(("quantize", cols_, xin, aq, n_in))
    mv.sync()

    def qwen_step_tiled():
        for l in launches:
            if l[0] == "quantize":
                mv.quantize(Q80, l[2].ptr, l[1], l[4], l[1], l[3].ptr)
        for l in launches:
            if l[0] != "quantize":
                mv.gemv_segments(mv.Q8_0_T16, l[0], l[1], l[2].ptr, nvb, l[3])
        mv.gemv_segments_f32(mv.Q8_0_T16, head16_seg, cols, d_hx8.ptr, cols, d_ha8.ptr, nvb, rows)

    import numpy as np
    probe_idx = (len(bo) - 1, 2, 0)                     # a down projection, a gate/up, a q/k/v
    before = [bo[i].download(np.uint32, bo[i].nbytes // 4).copy() for i in probe_idx]
    for i in probe_idx:
        _lib_check_memset(bo[i])
    qwen_step_tiled()
    mv.sync()
    for i, want in zip(probe_idx, before):              # the file layout's bits
        assert np.array_equal(bo[i].download(np.uint32, bo[i].nbytes // 4), want)
    graph = mv.Graph()
    with graph:
        qwen_step_tiled()
    us_t = timed(graph.launch, 20, mv)
    graph.destroy()
    n_l = sum(1 for l in launches) + 2
    out["q8_0_decode_step_qwen2_5_0_5b"]["batch8_tile_major_grouped_us"] = round(us_t, 1)
    out["q8_0_decode_step_qwen2_5_0_5b"]["batch8_tile_major_grouped_note"] = (
        "every matrix tile-major (oxh_tile16), the independent operations of one input width grouped into launches "
        "of up to 32 segments: %d launches per step, %.1f us per activation" % (n_l, us_t / nvb))
    # ... and as ONE launch: a plan over the tile-major matrices, eight activations per segment, every operation
    # quantising its own f32 input (the matrices cut into runs of whole row groups, dealt by units streamed)
    plan_ops = []
    for idx, (segs_, cols_, tot) in enumerate(bsegs):
        layer, op = divmod(idx, len(qs.ops))
        rows_ = qs.ops[op][2]
        items, off = [], 0
        for seg, r_ in enumerate(rows_):
            items.append((t16_of[(idx, seg)].ptr, bo[idx].ptr + off * 4, r_, 0, nvb))
            off += r_
        plan_ops.append(dict(qtype=mv.Q8_0_T16, segs=mv.make_segments(items), cols=cols_, d_x=bx[idx].ptr,
                             d_act_out=None, out_stride=tot))
    plan_ops.append(dict(qtype=mv.Q8_0_T16, segs=mv.make_segments([(d_head16.ptr, d_ho8.ptr, rows, 0, nvb)]), cols=cols,
                         d_x=d_hx8.ptr, d_act_out=None, out_stride=rows))
    tplan = mv.Plan(plan_ops)
    head_before = d_ho8.download(np.uint32, nvb * rows).copy()
    for i in probe_idx:
        _lib_check_memset(bo[i])
    _lib_check_memset(d_ho8)
    tplan.launch()
    assert tplan.status() == 0
    for i, want in zip(probe_idx, before):
        assert np.array_equal(bo[i].download(np.uint32, bo[i].nbytes // 4), want)
    assert np.array_equal(d_ho8.download(np.uint32, nvb * rows), head_before)
    us_p = timed(tplan.launch, 20, mv)
    t_info = tplan.info()
    tplan.destroy()
    step_bytes8 = qs.weight_bytes + w.nbytes
    out["q8_0_decode_step_qwen2_5_0_5b"]["batch8_tile_major_plan_us"] = round(us_p, 1)
    out["q8_0_decode_step_qwen2_5_0_5b"]["batch8_tile_major_plan_note"] = (
        "the same 97 operations at eight activations each as ONE launch (a plan over OXH_Q8_0_T16 operations, %d "
        "workgroups): %.1f us per activation, %.2f TB/s of weight bytes, bit-checked against the file-layout outputs"
        % (t_info["workgroups"], us_p / nvb, step_bytes8 / us_p / 1e6))
    for b_ in tiled_keep:
        b_.free()
    for b_ in bx + bo + ba + [d_head16, d_hx8, d_ho8, d_ha8]:
        b_.free()
    d_head.free()
    d_hx.free()
    d_ho.free()
    # What a kernel that only reads reaches on buffers the size of the decode set's matrices (launch
    # cost included; twelve distinct buffers in turn, 793 MB, so that nothing comes from the last-level
    # cache; one graph of twelve launches per replay): the ceiling the GEMV figures stand against here.
    ceiling = {}
    probe = [mv.DeviceBuffer(66060288) for _ in range(12)]
    for b in probe:
        _lib_check_memset(b)
    for name, nbytes in (("gate_up_66MB", 66060288), ("down_q6k_48MB", 48168960), ("qkv_14MB", 14155776),
                         ("o_9MB", 9437184)):
        graph = mv.Graph()                      # replayed as a graph, like the decode set
        with graph:
            for b in probe:
                mv.read_probe(b.ptr, nbytes)
        us = timed(graph.launch, 8, mv) / len(probe)
        graph.destroy()
        ceiling[name] = {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                         "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
    for b in probe:
        b.free()
    out["read_only_kernel_ceiling"] = ceiling
    # Mixtral-shaped expert GEMVs (configuration 4)
    ms_file = MoESet(seed=0)
    us_file = timed(ms_file.launch_step, 10, mv)
    for buf in list(ms_file.w.values()) + [ms_file.d_xg, ms_file.d_h, ms_file.d_gate, ms_file.d_up, ms_file.d_down,
                                           ms_file.d_act_x, ms_file.d_act_h]:
        buf.free()
    ms = MoESet(seed=0, tile_major=True)
    us = timed(ms.launch_step, 10, mv)
    out["moe_8x_top2_16tok_q4k"] = {
        "us": round(us, 2), "experts_hit": ms.hit, "gbps": round(ms.bytes_per_step / us / 1e3, 1),
        "frac_of_hbm_peak": round(ms.bytes_per_step / us / 1e3 / HBM_PEAK_GBPS, 4),
        "weights_layout": "tile-major (oxh_tile16: the same blocks, sixteen rows' blocks of one index adjacent; "
                          "rewritten once at load, results bit-identical)",
        "file_layout_us": round(us_file, 2),
        "note": "792.7 MB of expert weights fit the 256 MB last-level cache only in part; "
                "per step: Q8_K quantisation + one MFMA launch for all experts' gate+up, the same for "
                "all experts' down, each expert over its own tokens only"}
    # the same layer end to end with the routing on the device: router logits in, combined output out
    layer = mv.MoeLayer(mv.Q4_K_T16, mv.Q4_K_T16, ms.w["gate"].ptr, ms.w["up"].ptr, ms.w["down"].ptr, ms.n_expert, ms.top_k,
                        ms.hidden, ms.ffn, True, max_tok=ms.n_tok)
    d_logits = mv.DeviceBuffer.from_host(ms.logits)
    d_xt = mv.DeviceBuffer.from_host(ms.x_tok)
    d_yt = mv.DeviceBuffer(ms.n_tok * ms.hidden * 4)
    layer.forward(d_logits.ptr, d_xt.ptr, ms.n_tok, d_yt.ptr)
    mv.sync()
    # the six launches of oxh_moe_ffn as the call makes them, and replayed as a graph (whose replays cost about
    # 10 us each to start: timed in runs of fifty); five timings each, their median
    def forward():
        layer.forward(d_logits.ptr, d_xt.ptr, ms.n_tok, d_yt.ptr)

    runs = sorted(timed(forward, 20, mv) for _ in range(5))
    us = runs[2]
    graph = mv.Graph()
    with graph:
        forward()
    graph_runs = sorted(timed(graph.launch, 50, mv) for _ in range(5))
    graph.destroy()
    out["moe_layer_device_routed_8x_top2_16tok_q4k"] = {
        "us": round(us, 2), "gbps": round(ms.bytes_per_step / us / 1e3, 1),
        "frac_of_hbm_peak": round(ms.bytes_per_step / us / 1e3 / HBM_PEAK_GBPS, 4),
        "launches": 6, "weights_layout": "tile-major",
        "us_fastest_and_slowest_of_five_timings": [round(runs[0], 2), round(runs[-1], 2)],
        "as_graph_us": round(graph_runs[2], 2),
        "note": "oxh_moe_ffn, one call: route + group, gather + Q8_K, gate/up of all experts, "
                "silu(gate)*up + Q8_K, down of all experts, combine; no host step between them"}
    return out


def batched_step_figure(mv, synth, ds, single_us):
    """Configuration 1's set at eight and sixteen activations per matmul (a batch of sequences decoding
    together): not a launch per matmul (at that size q/k/v, o and down are launches of 64-96 row tiles on
    256 CUs) but the independent matmuls of one shape grouped into launches of up to 32 segments, each segment
    its own matrix and run of activations, Q4_K from tile-major copies: 7 matmul launches + 4 quantising
    launches per step."""
    import numpy as np
    Q4K, Q6K = 13, 16
    layers = ds.layers
    keep, w_run = [], {}
    for layer in range(layers):
        for op, (name, qt, rows_, cols_, _) in enumerate(ds.ops):
            for seg, r_ in enumerate(rows_):
                if qt == Q4K:
                    t = mv.DeviceBuffer(mv.tile16_bytes(Q4K, r_, cols_))
                    mv.tile16(Q4K, ds.weights[layer][op][seg].ptr, r_, cols_, t.ptr)
                elif ds.q6_grouped:                     # the tile kernel reads Q6_K in the file layout
                    t = mv.DeviceBuffer.from_host(synth.weights(Q6K, r_, cols_, seed=ds.seed, stream=layer * 7 + 6))
                else:
                    t = ds.weights[layer][op][seg]
                if t is not ds.weights[layer][op][seg]:
                    keep.append(t)
                w_run[(layer, op, seg)] = t
    mv.sync()
    res = {}
    for nv in (8, 16):
        bufs, launches, outs = [], [], {}
        for op, (name, qt, rows_, cols_, _) in enumerate(ds.ops):
            tot, n_in = sum(rows_), layers * nv
            xin = mv.DeviceBuffer.from_host(synth.normal(n_in * cols_, seed=0, stream=900 + op))
            aq = mv.DeviceBuffer(n_in * mv.act_bytes(qt, cols_))
            bufs += [xin, aq]
            items = []
            for layer in range(layers):
                o = mv.DeviceBuffer(nv * tot * 4)
                bufs.append(o)
                outs[(layer, op)] = (o, xin.ptr + layer * nv * cols_ * 4)
                off = 0
                for seg, r_ in enumerate(rows_):
                    items.append((w_run[(layer, op, seg)].ptr, o.ptr + off * 4, r_, layer * nv, nv))
                    off += r_
            # one call per shape: its 32-96 segments go out as launches of 32 over activations quantised once
            launches.append((mv.Q4_K_T16 if qt == Q4K else qt, mv.make_segments(items), cols_, xin, aq, tot))

        def step():
            for qt_, segs_, cols_, xin, aq, tot in launches:
                mv.gemv_segments_f32(qt_, segs_, cols_, xin.ptr, cols_, aq.ptr, nv, tot)

        step()
        mv.sync()
        if nv == 8:
            # the bits of a launch of its own over the file layout (which the tests hold to the oracle)
            for layer, op in ((layers - 1, 0), (0, 3)):
                name, qt, rows_, cols_, _ = ds.ops[op]
                o, x_ptr = outs[(layer, op)]
                tot = sum(rows_)
                ref, a_ref = mv.DeviceBuffer(nv * tot * 4), mv.DeviceBuffer(nv * mv.act_bytes(qt, cols_))
                items, off = [], 0
                for seg, r_ in enumerate(rows_):
                    w = ds.weights[layer][op][seg] if qt == Q4K else w_run[(layer, op, seg)]
                    items.append((w.ptr, ref.ptr + off * 4, r_, 0))
                    off += r_
                mv.gemv_segments_f32(qt, mv.make_segments(items), cols_, x_ptr, cols_, a_ref.ptr, nv, tot)
                mv.sync()
                assert np.array_equal(o.download(np.uint32, nv * tot), ref.download(np.uint32, nv * tot))
                ref.free()
                a_ref.free()
        graph = mv.Graph()
        with graph:
            step()
        us = timed(graph.launch, 10, mv)
        graph.destroy()
        res["batch%d" % nv] = {"us_per_step": round(us, 1), "us_per_activation": round(us / nv, 1),
                               "calls_per_step": len(launches),
                               "launches_per_step": sum(1 + (len(l[1]) + 31) // 32 for l in launches),
                               "weight_gbps": round(ds.weight_bytes / us / 1e3, 1),
                               "frac_of_hbm_peak": round(ds.weight_bytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
        for b_ in bufs:
            b_.free()
    for b_ in keep:
        b_.free()
    res["note"] = ("the 128 matmuls of a Llama-3-8B-shaped step with 8 / 16 activations each, the matmuls of one shape "
                   "in one oxh_gemv_segments_f32 call (32 segments to a launch, OXH_Q4_K_T16 copies and file-layout Q6_K, "
                   "one quantising launch per shape), replayed as a graph; two operations bit-checked against launches "
                   "of their own.  The single-activation step takes %.0f us as one launch: per activation this is "
                   "%.1fx / %.1fx less" % (single_us, single_us / res["batch8"]["us_per_activation"],
                                           single_us / res["batch16"]["us_per_activation"]))
    return res


def _lib_check_copy(dst, src, nbytes):
    import ctypes
    from oxidize_amd import _lib
    _lib.check(_lib.lib().oxh_memcpy_d2d(ctypes.c_void_p(dst), ctypes.c_void_p(src), nbytes, None))


def traffic_probe(mv, ds):
    """For `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` runs: three 256 MiB
    device-to-device copies (a kernel of known traffic to scale the counters
    by), then one gate/up GEMV per layer.  Prints nothing."""
    import ctypes
    from oxidize_amd import _lib
    n = 256 << 20
    a, b = mv.DeviceBuffer(n), mv.DeviceBuffer(n)
    _lib.check(_lib.lib().oxh_memset(ctypes.c_void_p(a.ptr), 1, n, None))
    for _ in range(3):
        _lib.check(_lib.lib().oxh_memcpy_d2d(ctypes.c_void_p(b.ptr), ctypes.c_void_p(a.ptr), n, None))
    mv.sync()
    for layer in range(ds.layers):
        ds.launch_op(layer, 2)
    mv.sync()
    plan = mv.Plan(ds.plan_ops())
    for _ in range(3):
        plan.launch()
    assert plan.status() == 0


def q80_step_probe(mv, synth):
    """For `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` runs on k_gemv_multi: three 256 MiB device-to-device
    copies (a kernel of known traffic to scale the counters by), then three launches of the
    Qwen2.5-0.5B-shaped Q8_0 decode step as one plan.  Prints nothing."""
    import ctypes
    from oxidize_amd import _lib
    from oxidize_amd.workloads import DecodeSet, QWEN2_5_0_5B
    Q80 = 7
    n = 256 << 20
    a, b = mv.DeviceBuffer(n), mv.DeviceBuffer(n)
    _lib.check(_lib.lib().oxh_memset(ctypes.c_void_p(a.ptr), 1, n, None))
    for _ in range(3):
        _lib.check(_lib.lib().oxh_memcpy_d2d(ctypes.c_void_p(b.ptr), ctypes.c_void_p(a.ptr), n, None))
    mv.sync()
    rows, cols = 151936, 896
    qs = DecodeSet(qtypes=(Q80, Q80), seed=0, **QWEN2_5_0_5B)
    d_head = mv.DeviceBuffer.from_host(synth.weights(Q80, rows, cols, seed=0, stream=5))
    d_hx = mv.DeviceBuffer.from_host(synth.normal(cols, seed=0, stream=8))
    d_ho = mv.DeviceBuffer(rows * 4)
    head_seg = mv.make_segments([(d_head.ptr, d_ho.ptr, rows, 0)])
    plan = mv.Plan(qs.plan_ops() + [dict(qtype=Q80, segs=head_seg, cols=cols, d_x=d_hx.ptr, d_act_out=None)])
    for _ in range(3):
        plan.launch()
    assert plan.status() == 0


def q80_batch_probe(mv, synth):
    """For `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` runs on k_q80t_multi: three 256 MiB device-to-device
    copies (known traffic), then three launches of the Qwen2.5-0.5B-shaped Q8_0 step at eight activations per
    matmul as one plan over tile-major copies.  Prints nothing."""
    import ctypes
    from oxidize_amd import _lib
    from oxidize_amd.workloads import DecodeSet, QWEN2_5_0_5B
    Q80, nvb = 7, 8
    n = 256 << 20
    a, b = mv.DeviceBuffer(n), mv.DeviceBuffer(n)
    _lib.check(_lib.lib().oxh_memset(ctypes.c_void_p(a.ptr), 1, n, None))
    for _ in range(3):
        _lib.check(_lib.lib().oxh_memcpy_d2d(ctypes.c_void_p(b.ptr), ctypes.c_void_p(a.ptr), n, None))
    mv.sync()
    rows, cols = 151936, 896
    qs = DecodeSet(qtypes=(Q80, Q80), seed=0, **QWEN2_5_0_5B)
    keep, ops = [], []

    def tiled(d_w, r_, c_):
        t = mv.DeviceBuffer(mv.tile16_bytes(Q80, r_, c_))
        mv.tile16(Q80, d_w.ptr, r_, c_, t.ptr)
        keep.append(t)
        return t

    for layer in range(qs.layers):
        for op, (name, qt, rows_, cols_, _) in enumerate(qs.ops):
            tot = sum(rows_)
            x = mv.DeviceBuffer.from_host(synth.normal(nvb * cols_, seed=0, stream=500000 + layer * 8 + op))
            o = mv.DeviceBuffer(nvb * tot * 4)
            keep += [x, o]
            items, off = [], 0
            for seg, r_ in enumerate(rows_):
                items.append((tiled(qs.weights[layer][op][seg], r_, cols_).ptr, o.ptr + off * 4, r_, 0, nvb))
                off += r_
            ops.append(dict(qtype=mv.Q8_0_T16, segs=mv.make_segments(items), cols=cols_, d_x=x.ptr, d_act_out=None,
                            out_stride=tot))
    d_head = mv.DeviceBuffer.from_host(synth.weights(Q80, rows, cols, seed=0, stream=5))
    hx = mv.DeviceBuffer.from_host(synth.normal(nvb * cols, seed=0, stream=9))
    ho = mv.DeviceBuffer(nvb * rows * 4)
    ops.append(dict(qtype=mv.Q8_0_T16, segs=mv.make_segments([(tiled(d_head, rows, cols).ptr, ho.ptr, rows, 0, nvb)]),
                    cols=cols, d_x=hx.ptr, d_act_out=None, out_stride=rows))
    mv.sync()
    plan = mv.Plan(ops)
    for _ in range(3):
        plan.launch()
    assert plan.status() == 0


def split_probe(mv, synth):
    """For `rocprofv3 --kernel-trace --stats` runs on the small-batch launches whose tiles share their
    columns between workgroups: a 4096 x 14336 Q6_K matrix under 16 activations, twelve launches of
    oxh_mmq and twelve of oxh_mmq_split over six copies of the weights in turn.  Prints nothing."""
    Q6K = 16
    rows, cols, n_vec = 4096, 14336, 16
    w = synth.weights(Q6K, rows, cols, seed=0, stream=12)
    copies = [mv.DeviceBuffer.from_host(w) for _ in range(6)]
    d_x = mv.DeviceBuffer.from_host(synth.normal(n_vec * cols, seed=0, stream=2011))
    d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(Q6K, cols))
    d_o = mv.DeviceBuffer(n_vec * rows * 4)
    mv.quantize(Q6K, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    need = mv.mmq_split_workspace(Q6K, rows, cols, n_vec, rows)
    assert need
    d_ws = mv.DeviceBuffer(need)
    for i in range(12):
        mv.mmq(Q6K, copies[i % 6].ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows)
    for i in range(12):
        mv.mmq_split(Q6K, copies[i % 6].ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows, d_ws.ptr, need)
    mv.sync()


def head_probe(mv, synth):
    """For `rocprofv3` runs on the Q8_0 kernels of 2-16 activations: the 151936 x 896 vocabulary head at
    eight activations, six launches from the file layout (k_mfma_q8_0_segments) and six from the tile-major
    copy (k_q80t_segments), three copies of the weights in turn.  Prints nothing."""
    Q80 = 7
    rows, cols, nv = 151936, 896, 8
    w = synth.weights(Q80, rows, cols, seed=0, stream=5)
    copies = [mv.DeviceBuffer.from_host(w) for _ in range(3)]
    tiled = [mv.DeviceBuffer(mv.tile16_bytes(Q80, rows, cols)) for _ in range(3)]
    for c, t in zip(copies, tiled):
        mv.tile16(Q80, c.ptr, rows, cols, t.ptr)
    d_x = mv.DeviceBuffer.from_host(synth.normal(nv * cols, seed=0, stream=6))
    d_o = mv.DeviceBuffer(nv * rows * 4)
    d_qa = mv.DeviceBuffer(nv * mv.act_bytes(Q80, cols))
    for qt, bufs in ((Q80, copies), (mv.Q8_0_T16, tiled)):
        for i in range(6):
            segs = mv.make_segments([(bufs[i % 3].ptr, d_o.ptr, rows, 0)])
            mv.gemv_segments_f32(qt, segs, cols, d_x.ptr, cols, d_qa.ptr, nv, rows)
    mv.sync()


def moe_probe(mv, synth):
    """For `rocprofv3` runs on the expert launches of configuration 4 (8 experts, top-2, 16 tokens, Q4_K):
    six steps from the file layout, then six from tile-major expert stacks.  Prints nothing."""
    from oxidize_amd.workloads import MoESet
    for tile_major in (False, True):
        ms = MoESet(seed=0, tile_major=tile_major)
        for _ in range(6):
            ms.launch_step()
        mv.sync()
        for buf in list(ms.w.values()) + [ms.d_xg, ms.d_h, ms.d_gate, ms.d_up, ms.d_down, ms.d_act_x, ms.d_act_h]:
            buf.free()


def mmq_probe(mv, synth):
    """For `rocprofv3 --pmc` runs on the MFMA kernel: quantise 512 activations
    of 4096 values, then three 14336 x 4096 x 512 launches.  Prints nothing."""
    Q4K = 13
    rows, cols, n_vec = 14336, 4096, 512
    d_w = mv.DeviceBuffer.from_host(synth.weights(Q4K, rows, cols, seed=0, stream=0))
    d_x = mv.DeviceBuffer.from_host(synth.normal(n_vec * cols, seed=0, stream=2000))
    d_a = mv.DeviceBuffer(n_vec * mv.act_bytes(Q4K, cols))
    d_o = mv.DeviceBuffer(n_vec * rows * 4)
    mv.quantize(Q4K, d_x.ptr, cols, n_vec, cols, d_a.ptr)
    for _ in range(3):
        mv.mmq(Q4K, d_w.ptr, rows, cols, d_a.ptr, n_vec, d_o.ptr, rows)
    mv.sync()


def host_cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(layers_sample=8, min_seconds=2.5, cores=None):
    """The reference CPU path on the host cores over `layers_sample` distinct
    layers of the same workload in turn (same shapes, same synthetic generator:
    138 MB a layer, so eight of them stream from DRAM rather than sit in the
    host's caches; layers_sample=1 gives the cache-resident figure); `cores` =
    worker threads (default: up to 16, the cap of the reference's own CLI)."""
    import numpy as np
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oxlibs
    from oxidize_amd import synth

    ref = oxlibs.ref()
    kind = "reference" if ref is not None else "port"
    if cores is None:
        cores = min(16, os.cpu_count() or 1)
    if ref is not None:
        ref.oc_parallel_set_threads(cores)
    else:
        os.environ.setdefault("OMP_NUM_THREADS", str(cores))
    orc = oxlibs.oracle()
    ops = [(13, [4096, 1024, 1024], 4096), (13, [4096], 4096), (13, [14336, 14336], 4096),
           (16, [4096], 14336)]
    layers = []
    nbytes = 0
    for layer in range(layers_sample):
        mats = []
        for i, (qt, rows, cols) in enumerate(ops):
            ws = [synth.weights(qt, r, cols, seed=0, stream=9000 + 100 * layer + 10 * i + k)
                  for k, r in enumerate(rows)]
            x = synth.normal(cols, seed=0, stream=9900 + i)
            outs = [np.zeros(r, np.float32) for r in rows]
            temp = np.zeros(cols, np.float32)
            mats.append((qt, rows, cols, ws, x, outs, temp))
            if layer == 0:
                nbytes += sum(w.nbytes for w in ws) + 4 * cols + 4 * sum(rows)
        layers.append(mats)
    fn = ref.oc_matvec_quantized_fused if ref is not None else orc.oxo_matvec_quantized_fused

    def one_layer(mats):
        for qt, rows, cols, ws, x, outs, temp in mats:
            rb = synth.row_bytes(qt, cols)
            n = len(rows)
            fn(oxlibs.u32_array([qt] * n), oxlibs.ptr_array(ws), oxlibs.size_array(rows), cols,
               oxlibs.size_array([rb] * n), n, x.ctypes.data, oxlibs.ptr_array(outs), temp.ctypes.data)

    one_layer(layers[0])
    reps, t0 = 0, time.perf_counter()
    while True:
        one_layer(layers[reps % layers_sample])
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds and reps >= 3:
            break
    gbps = nbytes * reps / dt / 1e9
    return {"value": round(gbps, 3), "unit": "GB/s", "cores": cores, "kind": kind,
            "sample": "%d layer passes over %d distinct layers of the same decode set in turn (qkv, o, gate/up "
                      "Q4_K; down Q6_K; %.1f MB per layer, %.0f MB in all) through oc_matvec_quantized_fused, "
                      "%.2f s wall; host CPU: %s" % (reps, layers_sample, nbytes / 1e6,
                                                     nbytes * layers_sample / 1e6, dt, host_cpu_model())}


def main():
    global LEG_SPINUP_MS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # a launch of the step kernel takes 0.8-1.1 ms for the first thirty or so launches after the device
    # was idle and settles after that (clock and memory power states), hence the long default warm-up
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--spinup-ms", type=float, default=60.0,
                    help="untimed milliseconds of the same step before the warm-up steps (device clocks settle)")
    ap.add_argument("--leg-spinup-ms", type=float, default=LEG_SPINUP_MS,
                    help="untimed milliseconds of the same calls in front of every other timed leg (0 under a tracing profiler)")
    ap.add_argument("--layers", type=int, default=32, help=argparse.SUPPRESS)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--mode", choices=["plan", "graph", "launches"], default="plan",
                    help="a step as one persistent launch (default), as a HIP graph of 128 launches, or as 128 launches")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary configurations")
    ap.add_argument("--probe", choices=["traffic", "mmq", "q80step", "q80batch", "split", "head", "moe"], help="run a counter-collection workload and exit")
    args = ap.parse_args()
    LEG_SPINUP_MS = max(0.0, args.leg_spinup_ms)
    if args.gpus != 1:
        print("bench.py: this path is built and measured on ONE GPU; --gpus %d is not supported "
              "(the work would shard by output rows across GPUs; nothing here launches a second rank)" % args.gpus, file=sys.stderr)
        return 2

    from oxidize_amd import _lib
    from oxidize_amd import matvec as mv
    from oxidize_amd.workloads import DecodeSet

    lib = _lib.lib()
    _lib.check(lib.oxh_init(0))
    info = mv.device_info()

    if args.probe == "mmq":
        from oxidize_amd import synth
        mmq_probe(mv, synth)
        return 0
    if args.probe == "split":
        from oxidize_amd import synth
        split_probe(mv, synth)
        return 0
    if args.probe in ("head", "moe"):
        from oxidize_amd import synth
        (head_probe if args.probe == "head" else moe_probe)(mv, synth)
        return 0
    if args.probe == "q80step":
        from oxidize_amd import synth
        q80_step_probe(mv, synth)
        return 0
    if args.probe == "q80batch":
        from oxidize_amd import synth
        q80_batch_probe(mv, synth)
        return 0

    ds = DecodeSet(layers=args.layers, seed=0)
    step_bytes = ds.bytes_per_step
    if args.probe == "traffic":
        traffic_probe(mv, ds)
        return 0

    graph = mv.Graph()
    with graph:
        ds.launch_step()
    plan = mv.Plan(ds.plan_ops())

    def step():
        if args.mode == "plan":
            plan.launch()
        elif args.mode == "graph":
            graph.launch()
        else:
            ds.launch_step()

    # The device's clocks take about thirty milliseconds of work to settle after an idle period (a launch
    # of the step kernel goes 0.79 -> 1.0 -> 0.73 ms over its first forty launches): run the step untimed
    # for --spinup-ms first, whatever the number of warm-up steps asked for.
    spun = 0
    t_spin = time.perf_counter()
    while (time.perf_counter() - t_spin) * 1e3 < args.spinup_ms:
        for _ in range(8):
            step()
        mv.sync()
        spun += 8
    for _ in range(args.warmup):
        step()
    mv.sync()

    e0, e1 = mv.Event(), mv.Event()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    mv.sync()
    wall = time.perf_counter() - t0
    if args.mode == "plan" and plan.status() != 0:
        print("bench.py: a plan launch gave up on a wait: " + lib.oxh_last_error().decode(), file=sys.stderr)
        return 1
    ev_ms = e1.ms_since(e0)
    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes * args.steps / wall / 1e9
    # the other two ways of running the same step, for the record
    other_modes = {"plan_one_launch_us": round(timed(plan.launch, args.steps, mv), 1),
                   "graph_of_128_launches_us": round(timed(graph.launch, args.steps, mv), 1)}

    # The four matmuls of a layer as single launches, each timed back to back over the 32 layers' distinct
    # weights (nothing is served from cache), HIP events on the launch stream: what a step costs when it is
    # launched kernel by kernel (their sum x 32 is the graph figure), and where the plan's gain comes from.
    sweeps = max(3, min(10, args.steps))
    per_launch = {}
    for op, (name, qt, rows, cols, _) in enumerate(ds.ops):
        nb = sum(w.nbytes for w in ds.weights[0][op]) + 4 * cols + 4 * sum(rows)
        for layer in range(ds.layers):
            ds.launch_op(layer, op)
        mv.sync()
        k0, k1 = mv.Event(), mv.Event()
        k0.record()
        for _ in range(sweeps):
            for layer in range(ds.layers):
                ds.launch_op(layer, op)
        k1.record()
        mv.sync()
        us = k1.ms_since(k0) * 1e3 / (sweeps * ds.layers)
        per_launch[name] = {"us": round(us, 3), "bytes": nb, "gbps": round(nb / us / 1e3, 1),
                            "frac_of_hbm_peak": round(nb / us / 1e3 / HBM_PEAK_GBPS, 4)}
    per_launch["sum_x_layers_ms"] = round(sum(v["us"] for v in per_launch.values()) * ds.layers / 1e3, 4)

    if args.mode == "plan":
        k_name = ("k_plan_ext" if plan.info()["prestaged"] else "k_plan") + " (one launch = one decode step of 128 matmuls)"
        k_bytes, k_us = step_bytes, ev_ms * 1e3 / args.steps
        k_traffic = PLAN_STEP_TRAFFIC_BYTES if ds.layers == 32 else None
    else:
        k_name, k_bytes, k_us = "k_gemv_q4_k (gate/up 28672x4096)", per_launch["gate_up"]["bytes"], per_launch["gate_up"]["us"]
        k_traffic = GATE_UP_TRAFFIC_BYTES
    achieved = k_bytes / k_us / 1e3   # GB/s

    out = {
        "metric": "q4k_gemv_hbm_gbps_llama3_8b_decode",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {"workload": "llama3-8b decode GEMV set, batch 1, 32 layers: qkv+o+gate/up Q4_K, "
                               "down Q6_K, Q8_K activations (the benchmark's configuration 1)",
                   "layers": ds.layers, "mode": args.mode,
                   "q6k_layout": "regrouped in runs of eight blocks when loaded (same bytes)" if ds.q6_grouped else "file",
                   "launches_per_step": 1 if args.mode == "plan" else 4 * ds.layers,
                   "operations_per_step": 4 * ds.layers,
                   "table_rows_per_step": plan.info()["table_rows"] if args.mode == "plan" else None,
                   "scheduling": ("the operations of this set do not depend on each other and the plan walks them in "
                                  "an order and grouping of its own: operations of one weight layout and vector length "
                                  "share table rows so that every wave has a whole number of 16-block passes "
                                  "(gate/up of a layer with o of the next, q/k/v of two layers, down of two layers); "
                                  "OXH_PLAN_MERGE=1 shares rows between neighbours only, 0 not at all; "
                                  "extra.decode_chain_fused is the same step with a layer's real dependencies")
                                 if args.mode == "plan" else None,
                   "untimed_steps_before_warmup": spun,
                   "bytes_per_step": step_bytes},
        "metric_scope": ("independent operations: the benchmark's configuration 1 gives every matmul its own N(0,1) "
                         "input, so nothing orders the 128 matmuls of a step; `dependent_chain` is the same 32 layers "
                         "as a model runs them"),
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "tokens_per_s_equiv": round(args.steps / wall, 1),
        "gpu_event_ms_per_step": round(ev_ms / args.steps, 4),
        "device": info,
        "roofline": {"bound": "hbm", "kernel": k_name,
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": k_traffic,
                     "traffic_source": ("historical: the rocprofv3 --pmc summary under profiles/ for this kernel and workload "
                                        "(a constant in bench.py, not measured in this run)"),
                     "bytes_per_launch": k_bytes, "us_per_launch": round(k_us, 3)},
        "step_other_modes": other_modes,
        "single_launches": per_launch,
    }
    # the same 32 layers with a layer's real dependencies (residual + RMSNorm and SwiGLU fused in), beside
    # the headline and not under `extra`: the headline's operations are independent, a model's are not
    # (a failure in a secondary leg is reported in its place: the line with the headline is printed regardless)
    def leg(fn, *a):
        try:
            return fn(*a)
        except Exception as e:                      # noqa: BLE001 - whatever it was, say so and go on
            print("bench.py: %s failed: %r" % (fn.__name__, e), file=sys.stderr)
            return {"error": "%s: %r" % (fn.__name__, e)}

    out["dependent_chain"] = leg(chain_figure, mv, ds, args.steps)
    if not args.no_extra:
        from oxidize_amd import synth
        out["extra"] = leg(secondary_figures, mv, synth)
        out["extra"]["decode_chain_fused"] = out["dependent_chain"]
        out["extra"]["decode_step_llama3_8b_batch_8_16"] = leg(batched_step_figure, mv, synth, ds, ev_ms * 1e3 / args.steps)
    out["cpu_baseline"] = None if args.no_cpu else cpu_baseline()
    if (not args.no_cpu and out["cpu_baseline"]["kind"] == "reference" and isinstance(out.get("extra"), dict)
            and "error" not in out["extra"]):
        one = cpu_baseline(layers_sample=2, min_seconds=1.5, cores=1)
        out["extra"]["cpu_baseline_1_thread"] = {"value": one["value"], "unit": one["unit"], "sample": one["sample"]}
        hot = cpu_baseline(layers_sample=1, min_seconds=1.5)
        out["extra"]["cpu_baseline_cache_resident"] = {"value": hot["value"], "unit": hot["unit"], "cores": hot["cores"],
                                                       "sample": hot["sample"]}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
