"""CPU tests of the shipped library's C ABI and host logic (no GPU needed):
every symbol include/oxhip.h declares is exported, the eligibility helpers
agree with the oracle's restatement of the reference's rules, declines happen
before any device work, and without a device the library fails loudly instead
of computing anything."""
import ctypes
import os
import re

import numpy as np

import oxlibs
from oxidize_amd import _lib, synth
from oxidize_amd import matvec as mv

ROOT = oxlibs.ROOT


def declared_functions():
    names = set()
    for header in ("oxhip.h", "oxhip_lab.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b((?:oxh|oc)_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    lib = _lib.lib()
    names = declared_functions()
    assert len(names) >= 40
    for n in names:
        assert hasattr(lib, n), "missing export: " + n
    assert set(_lib.SIGNATURES) == set(names)


def test_no_oracle_or_reference_symbols_in_the_product():
    out = os.popen("nm -D --defined-only %s" % _lib.LIB_PATH).read()
    assert "oxo_" not in out
    needed = os.popen("readelf -d %s" % _lib.LIB_PATH).read()
    assert "oxoracle" not in needed and "oxref" not in needed


def test_shape_helpers_match_the_reference_rules():
    lib = _lib.lib()
    o = oxlibs.oracle()
    handled = (3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20, 25, 36)
    for qt in tuple(range(0, 40)):
        for cols in (0, 32, 96, 256, 896, 900, 2816, 4096, 14336):
            want = o.oxo_act_kind(qt, cols) if qt in handled else 0      # every other id: declined
            assert lib.oxh_act_kind(qt, cols) == want
            assert (lib.oxh_act_kind(qt, cols) != 0) == (qt in handled and want != 0)
    assert lib.oxh_row_bytes(13, 4096) == 2304
    assert lib.oxh_row_bytes(16, 14336) == 11760
    assert lib.oxh_row_bytes(7, 896) == 952
    assert lib.oxh_row_bytes(13, 896) == 0
    assert lib.oxh_row_bytes(15, 4096) == 2816 and lib.oxh_row_bytes(14, 256) == 176
    assert [lib.oxh_row_bytes(q, 896) for q in (3, 4, 5, 6)] == [28 * 18, 28 * 20, 28 * 22, 28 * 24]
    assert [lib.oxh_row_bytes(q, 896) for q in (17, 18, 19, 20)] == [28 * 18, 28 * 14, 28 * 22, 28 * 34]
    assert [lib.oxh_row_bytes(q, 4096) for q in (8, 9, 10, 11)] == [16 * 84] + [16 * 110] * 3
    assert lib.oxh_act_bytes(13, 4096) == 4672
    assert lib.oxh_act_bytes(7, 896) == 952
    for cols in (0, 31, 256, 896, 4096, 14336, 1 << 20, 3 << 20):
        assert lib.oc_matvec_batch_scratch_bytes(cols) == o.oxo_matvec_batch_scratch_bytes(cols)


def test_fused_switch_and_counters():
    lib = _lib.lib()
    assert lib.oc_matvec_fused_enabled() is True
    lib.oc_matvec_set_fused(False)
    assert lib.oc_matvec_fused_enabled() is False
    lib.oc_matvec_set_fused(True)
    lib.oc_matvec_fused_test_reset()
    st = lib.oc_matvec_fused_test_stats()
    assert (st.activation_quantizations, st.parallel_dispatches, st.fallback_calls) == (0, 0, 0)


def test_declines_need_no_device():
    x = synth.normal(4096, seed=1)
    w = synth.weights(13, 2, 4096, seed=1)
    out = np.full(2, 9.0, np.float32)
    temp = np.zeros(4096, np.float32)
    assert mv.matvec_quantized(13, w, 2, 896, 504, x, out, temp) == mv.DECLINED
    assert mv.matvec_quantized(13, w, 2, 4096, 2320, x, out, temp) == mv.DECLINED
    assert mv.matvec_quantized(2, w, 2, 4096, 8192, x, out, temp) == mv.DECLINED
    assert b"declined" in _lib.lib().oxh_last_error()
    assert np.all(out == 9.0)


def test_without_a_device_the_library_reports_it():
    """In a GPU-less container the compute entry points must return an error
    (never a result): there is no CPU path behind them."""
    lib = _lib.lib()
    rc = lib.oxh_init(0)
    if rc == 0:
        return                                   # a GPU is present: covered by the gpu tests
    assert rc == _lib.ERR_NO_DEVICE
    assert b"no HIP device" in lib.oxh_last_error()
    x = synth.normal(256, seed=1)
    w = synth.weights(13, 4, 256, seed=1)
    out = np.full(4, 9.0, np.float32)
    temp = np.zeros(256, np.float32)
    try:
        mv.matvec_quantized(13, w, 4, 256, 144, x, out, temp)
    except mv.OxhError as e:
        assert e.status == _lib.ERR_NO_DEVICE
    else:
        raise AssertionError("expected an error without a device")
    assert np.all(out == 9.0)


def test_synthetic_generator_is_deterministic():
    a = synth.weights(13, 64, 1024, seed=5, stream=2)
    b = synth.weights(13, 64, 1024, seed=5, stream=2)
    c = synth.weights(13, 64, 1024, seed=6, stream=2)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    blk = a.reshape(-1, 144)
    d = blk[:, :2].copy().view(np.float16).astype(np.float32)
    assert np.all(np.isfinite(d)) and np.all(d >= 0) and 0.012 < d.mean() < 0.020
    x = synth.normal(1 << 16, seed=0)
    assert abs(float(x.mean())) < 0.02 and abs(float(x.std()) - 1.0) < 0.02
    q = synth.weights(7, 16, 896, seed=1).reshape(-1, 34)[:, 2:].copy().view(np.int8)
    assert q.min() >= -127 and q.max() <= 127
    s6 = synth.weights(16, 4, 512, seed=1).reshape(-1, 210)[:, 192:208].copy().view(np.int8)
    assert s6.min() >= -32 and s6.max() <= 31


def test_void_symbols_hand_declined_calls_to_the_cpu_fallback():
    """A link-time replacement must not kill the process on a shape the reference's own code handles
    (matvec.c:833-907 falls back to its dequantise path): with a CPU fallback installed the void
    oc_matvec_quantized* symbols forward the call with its original arguments."""
    lib = _lib.lib()
    o = oxlibs.oracle()
    seen = []

    ONE = ctypes.CFUNCTYPE(None, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t,
                           ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p)
    BATCH = ctypes.CFUNCTYPE(None, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t,
                             ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t,
                             ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t)

    def cpu_one(qt, data, rows, cols, rb, x, out, temp):
        seen.append(("one", qt, rows, cols, rb))
        # the caller's CPU path: here the oracle's integer path over the same arguments
        o.oxo_matvec_quantized(qt, data, rows, cols, rb, x, out, temp)

    def cpu_batch(qt, data, rows, cols, rb, xs, in_stride, outs, out_stride, n_vec, temp, scratch, nscratch):
        seen.append(("batch", qt, rows, cols, n_vec))

    class Table(ctypes.Structure):
        _fields_ = [("one", ONE), ("fused", ctypes.c_void_p), ("multi", ctypes.c_void_p), ("batch", BATCH)]

    table = Table(ONE(cpu_one), None, None, BATCH(cpu_batch))
    lib.oxh_set_cpu_fallback(ctypes.byref(table))
    try:
        before = lib.oxh_cpu_fallback_calls()
        rows, cols = 4, 512
        w = synth.weights(13, rows, cols, seed=3)
        x = synth.normal(cols, seed=3)
        out = np.full(rows, 9.0, np.float32)
        temp = np.zeros(cols, np.float32)
        lib.oc_matvec_set_fused(False)             # OC_NO_FUSED: every call is declined
        lib.oc_matvec_quantized(13, w.ctypes.data, rows, cols, 288, x.ctypes.data, out.ctypes.data,
                                temp.ctypes.data)
        lib.oc_matvec_set_fused(True)
        assert seen == [("one", 13, rows, cols, 288)]
        want = np.zeros(rows, np.float32)
        wtmp = np.zeros(cols, np.float32)
        o.oxo_matvec_quantized(13, w.ctypes.data, rows, cols, 288, x.ctypes.data, want.ctypes.data,
                               wtmp.ctypes.data)
        assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
        # a padded row stride is declined too (matvec.c:961-985) and goes to the batch fallback
        scratch = np.zeros(1 << 16, np.uint8)
        lib.oc_matvec_quantized_batch(13, w.ctypes.data, rows, cols, 304, x.ctypes.data, cols, out.ctypes.data,
                                      rows, 1, temp.ctypes.data, scratch.ctypes.data, scratch.size)
        assert seen[-1] == ("batch", 13, rows, cols, 1)
        assert lib.oxh_cpu_fallback_calls() == before + 2
    finally:
        lib.oxh_set_cpu_fallback(None)


def test_weight_stats_and_unregister_need_no_device():
    lib = _lib.lib()
    n = [ctypes.c_size_t(7) for _ in range(4)]
    assert lib.oxh_weight_stats(*[ctypes.byref(v) for v in n]) == 0
    assert lib.oxh_init(0) != 0 or True
    buf = np.zeros(64, np.uint8)
    assert lib.oxh_weight_unregister(buf.ctypes.data) == 0      # nothing there: not an error


def test_plan_deals_rows_within_the_grid():
    """How a plan spreads an operation's rows over the device is host arithmetic: never more workgroups
    than the grid, every segment served, no wave beyond 32 table rows."""
    lib = _lib.lib()

    def deal(rows, paired, grid):
        n = len(rows)
        r = (ctypes.c_size_t * n)(*rows)
        p = (ctypes.c_int * n)(*paired)
        wg = (ctypes.c_uint32 * n)()
        cap = ctypes.c_uint32()
        rc = lib.oxh_plan_deal(r, p, n, grid, wg, ctypes.byref(cap))
        return rc, list(wg), cap.value

    rc, wg, cap = deal([4096, 1024, 1024], [0, 0, 0], 256)       # q/k/v: plain rounding would take 257
    assert rc == 0 and sum(wg) <= 256 and wg[1] == wg[2] == 43 and wg[0] in (170, 171) and cap == 2
    rc, wg, cap = deal([14336], [1], 256)                        # gate/up pair: 3.5 rows per wave, both matrices
    assert rc == 0 and wg == [256] and cap == 8
    rc, wg, cap = deal([4096], [0], 256)
    assert rc == 0 and wg == [256] and cap == 1
    rc, wg, cap = deal([100], [0], 256)                          # fewer rows than waves: 7 workgroups are enough
    assert rc == 0 and wg == [7] and cap == 1
    rc, wg, cap = deal([7, 9000, 3], [0, 0, 0], 304)
    assert rc == 0 and sum(wg) <= 304 and min(wg) >= 1
    assert deal([1 << 20], [0], 256)[0] == _lib.ERR_TOO_WIDE     # 256 rows per wave: beyond the table
    assert deal([0], [0], 256)[0] == _lib.ERR_ARG


def test_mmq_tile_choice_is_host_arithmetic():
    """Which tile a matrix-core launch runs on depends on the launch and the number of compute units
    only: the benchmark's two prefill shapes take the big tiles on a 256-CU device, a device with fewer
    units takes them sooner, small batches take the small tiles (the smallest when that leaves no unit more
    than one), Q6_K has the 64 x 128 tile for matrices with few rows."""
    lib = _lib.lib()
    Q4K, Q5K, Q6K, Q80, WIDE2 = 13, 15, 16, 7, 0x1008

    def tile(qtype, rows, n_vec, n_cu=256):
        r, t = ctypes.c_uint32(), ctypes.c_uint32()
        rc = lib.oxh_mmq_tile(qtype, rows, n_vec, n_cu, ctypes.byref(r), ctypes.byref(t))
        return rc, r.value, t.value

    assert tile(Q4K, 14336, 512) == (0, 256, 128)        # 56 x 4 = 224 workgroups = 256 - 32
    assert tile(Q4K, 4096, 512) == (0, 128, 64)          # 16 x 4 = 64 big tiles would idle three quarters
    assert tile(Q4K, 4096, 512, n_cu=64) == (0, 256, 128)
    assert tile(Q4K, 14336, 16) == (0, 64, 16)
    assert tile(Q4K, 14336, 32) == (0, 64, 32)
    assert tile(Q4K, 1000, 100) == (0, 64, 16)           # neither larger tile fills the device; 16 x 7 small ones
    assert tile(Q4K, 7000, 40) == (0, 64, 32)            # 110 x 3 of the smallest would be more than one to a unit
    assert tile(Q4K, 4096, 64) == (0, 64, 16)            # 64 x 4 = one per unit
    assert tile(Q4K, 4096, 128) == (0, 64, 32)
    assert tile(Q5K, 28672, 512) == (0, 128, 128)        # one row chunk per wave: 128-row tiles
    assert tile(Q5K, 3600, 500) == (0, 128, 64)
    assert tile(Q6K, 4096, 512) == (0, 64, 128)          # 32 x 4 tiles of 128 x 128 are too few
    assert tile(Q6K, 14336, 512) == (0, 128, 128)
    assert tile(WIDE2, 14336, 512) == (0, 128, 128)
    # the rule itself, stated independently: the first of the candidates with at least 7/8 of the units busy
    def rule(qtype, rows, n_vec, n_cu):
        need = n_cu - n_cu // 8
        small = (64, 16) if -(-rows // 64) * -(-n_vec // 16) <= n_cu else (64, 32)
        if n_vec <= 16:
            return 64, 16
        if n_vec <= 32:
            return small
        cands = [(256, 128), (128, 64)] if qtype == Q4K else \
                [(128, 128), (128, 64)] if qtype == Q5K else [(128, 128), (64, 128), (128, 64)]
        for tr, tt in cands:
            if -(-rows // tr) * -(-n_vec // tt) >= need:
                return tr, tt
        return small
    for qtype in (Q4K, Q5K, Q6K):
        for rows in (1, 63, 64, 1000, 4096, 7165, 14336, 28672, 151936):
            for n_vec in (1, 16, 17, 32, 33, 64, 100, 128, 129, 512, 2048):
                for n_cu in (64, 256, 304):
                    assert tile(qtype, rows, n_vec, n_cu) == (0,) + rule(qtype, rows, n_vec, n_cu)
    # the 32-value formats have one tile; the codebook formats have no matrix-core kernel
    for qtype in (Q80, 3, 4, 5, 6, 17, 18, 19, 20):
        assert tile(qtype, 4096, 512) == (0, 128, 64)
    assert tile(25, 4096, 512)[0] == _lib.DECLINED
    assert tile(Q4K, 0, 512)[0] == _lib.DECLINED
    assert lib.oxh_mmq_tile(Q4K, 4096, 512, 256, None, None) == 0


def test_bindings_lay_the_structs_out_as_the_header_does(tmp_path):
    """The ctypes structures of the bindings against the C compiler's view of include/oxhip.h: size and
    the offset of every field (a field added to the header and not to the bindings would shift what
    follows it)."""
    import subprocess
    structs = {"OxhSegment": _lib.OxhSegment, "OxhPrologue": _lib.OxhPrologue, "OxhPlanOp": _lib.OxhPlanOp,
               "OxhMoe": _lib.OxhMoe, "OxhTensor": _lib.OxhTensor}
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "oxhip.h"', 'int main(void) {']
    for name, cls in structs.items():
        lines.append('printf("%s size %%zu\\n", sizeof(%s));' % (name, name))
        for field, _ in cls._fields_:
            lines.append('printf("%s %s %%zu\\n", offsetof(%s, %s));' % (name, field, name, field))
    lines += ['return 0; }']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), "-o", str(exe), str(src)], check=True)
    seen = {}
    for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines():
        name, field, value = line.split()
        seen[(name, field)] = int(value)
    for name, cls in structs.items():
        assert seen[(name, "size")] == ctypes.sizeof(cls), name
        for field, _ in cls._fields_:
            assert seen[(name, field)] == getattr(cls, field).offset, (name, field)
