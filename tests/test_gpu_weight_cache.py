"""The host-pointer entry points read caller-owned memory on every call
(oxidize-c/include/oxidize/matvec.h:45-52).  The library keeps device copies of matrices it has seen;
these tests reuse host memory in the ways a program does (a buffer refilled with another model's tensor,
a smaller tensor of another type inside an old one's range, free + malloc at the same address) WITHOUT
telling the library, and expect the oracle's bits every time."""
import ctypes

import numpy as np
import pytest

import oxlibs
from oxidize_amd import _lib, synth
from oxidize_amd import matvec as mv

pytestmark = pytest.mark.gpu


def oracle_matvec(qt, w, rows, cols, x):
    o = oxlibs.oracle()
    want = np.zeros(rows, np.float32)
    tmp = np.zeros(max(cols, 64), np.float32)
    assert o.oxo_matvec_quantized(qt, w.ctypes.data, rows, cols, synth.row_bytes(qt, cols), x.ctypes.data,
                                  want.ctypes.data, tmp.ctypes.data) == 0
    return want


def run(qt, w, rows, cols, x):
    out = np.zeros(rows, np.float32)
    temp = np.zeros(max(cols, 64), np.float32)
    assert mv.matvec_quantized(qt, w, rows, cols, synth.row_bytes(qt, cols), x, out, temp) == 0
    return out


def stats(lib):
    v = [ctypes.c_size_t(0) for _ in range(4)]
    assert lib.oxh_weight_stats(*[ctypes.byref(t) for t in v]) == 0
    return tuple(int(t.value) for t in v)


def test_same_buffer_refilled_with_other_matrices(oxh):
    """One numpy buffer, three tenants: a Q4_K matrix, another Q4_K matrix of the same size, then a smaller
    Q8_0 matrix inside the old range.  No oxh_weight_clear in between."""
    rows, cols = 512, 4096
    nbytes = rows * synth.row_bytes(13, cols)
    arena = np.zeros(nbytes, np.uint8)
    x = synth.normal(cols, seed=11)

    arena[:] = synth.weights(13, rows, cols, seed=1)
    a = run(13, arena, rows, cols, x)
    assert np.array_equal(a.view(np.uint32), oracle_matvec(13, arena, rows, cols, x).view(np.uint32))
    r0 = stats(oxh)[3]

    arena[:] = synth.weights(13, rows, cols, seed=2)          # same address, same size, other contents
    b = run(13, arena, rows, cols, x)
    assert np.array_equal(b.view(np.uint32), oracle_matvec(13, arena, rows, cols, x).view(np.uint32))
    assert not np.array_equal(a, b)
    assert stats(oxh)[3] == r0 + 1                            # noticed and refreshed, once

    b2 = run(13, arena, rows, cols, x)                        # unchanged bytes: served from the device copy
    assert np.array_equal(b2.view(np.uint32), b.view(np.uint32))
    assert stats(oxh)[3] == r0 + 1

    # a smaller matrix of another type at the same address, then one in the middle of the old range
    r8, c8 = 256, 896
    n8 = r8 * synth.row_bytes(7, c8)
    x8 = synth.normal(c8, seed=12)
    for at in (0, 300000 & ~1):
        view = arena[at:at + n8]
        view[:] = synth.weights(7, r8, c8, seed=3 + at)
        c = run(7, view, r8, c8, x8)
        want = np.zeros(r8, np.float32)
        tmp = np.zeros(c8, np.float32)
        assert oxlibs.oracle().oxo_matvec_quantized(7, view.ctypes.data, r8, c8, synth.row_bytes(7, c8),
                                                    x8.ctypes.data, want.ctypes.data, tmp.ctypes.data) == 0
        assert np.array_equal(c.view(np.uint32), want.view(np.uint32))

    # and the Q4_K tenant moves back in over all of it
    arena[:] = synth.weights(13, rows, cols, seed=4)
    d = run(13, arena, rows, cols, x)
    assert np.array_equal(d.view(np.uint32), oracle_matvec(13, arena, rows, cols, x).view(np.uint32))


def test_free_and_reallocate_like_a_model_reload(oxh):
    """The allocation pattern that turns an address-keyed cache into wrong answers: a large block is freed,
    then matrices are allocated, used and dropped one after the other, so that later ones land inside
    earlier ones' freed memory."""
    big = bytearray(8 << 20)
    del big
    for qt, rows, cols in ((13, 512, 4096), (16, 128, 14336), (7, 256, 896), (13, 256, 4096), (7, 256, 896)):
        w = synth.weights(qt, rows, cols, seed=0, stream=qt + rows)
        x = synth.normal(cols, seed=5)
        got = run(qt, w, rows, cols, x)
        assert np.array_equal(got.view(np.uint32), oracle_matvec(qt, w, rows, cols, x).view(np.uint32)), (qt, rows)
        del w


def test_grouped_and_batch_entries_see_refilled_buffers(oxh):
    rows, cols = 256, 2048
    rb = synth.row_bytes(13, cols)
    arena = [np.zeros(rows * rb, np.uint8) for _ in range(2)]
    x = synth.normal(cols, seed=21)
    xs = synth.normal(12 * cols, seed=22).reshape(12, cols)
    o = oxlibs.oracle()
    for seed in (1, 2):
        for k in range(2):
            arena[k][:] = synth.weights(13, rows, cols, seed=seed, stream=k)
        outs = [np.zeros(rows, np.float32) for _ in range(2)]
        temp = np.zeros(cols, np.float32)
        assert mv.matvec_quantized_fused([13, 13], arena, [rows, rows], cols, [rb, rb], x, outs, temp) == 0
        for k in range(2):
            assert np.array_equal(outs[k].view(np.uint32), oracle_matvec(13, arena[k], rows, cols, x).view(np.uint32))
        got = np.zeros((12, rows), np.float32)
        scratch = np.zeros(_lib.lib().oc_matvec_batch_scratch_bytes(cols), np.uint8)
        assert mv.matvec_quantized_batch(13, arena[0], rows, cols, rb, xs, cols, got, rows, 12, temp, scratch) == 0
        for v in range(12):
            assert np.array_equal(got[v].view(np.uint32),
                                  oracle_matvec(13, arena[0], rows, cols, xs[v]).view(np.uint32))


def test_registered_ranges_keep_their_contract_and_unregister_takes_inner_pointers(oxh):
    rows, cols = 64, 1024
    rb = synth.row_bytes(13, cols)
    stack = synth.weights(13, 4 * rows, cols, seed=9)          # four "experts"
    assert oxh.oxh_weight_register(stack.ctypes.data, stack.nbytes) == 0
    x = synth.normal(cols, seed=9)
    e2 = stack[2 * rows * rb:3 * rows * rb]
    got = run(13, e2, rows, cols, x)
    assert np.array_equal(got.view(np.uint32), oracle_matvec(13, e2, rows, cols, x).view(np.uint32))
    n_reg, n_cached = stats(oxh)[:2]
    assert n_reg >= 1
    # a slice resolved inside the registered tensor: nothing new was cached for it
    assert oxh.oxh_weight_device_ptr(e2.ctypes.data) is not None
    # unregister through a pointer in the middle of the range
    assert oxh.oxh_weight_unregister(e2.ctypes.data) == 0
    assert stats(oxh)[0] == n_reg - 1
    assert oxh.oxh_weight_device_ptr(stack.ctypes.data) is None
    # the same memory, now unregistered and changed, is picked up afresh
    stack[:] = synth.weights(13, 4 * rows, cols, seed=10)
    got = run(13, e2, rows, cols, x)
    assert np.array_equal(got.view(np.uint32), oracle_matvec(13, e2, rows, cols, x).view(np.uint32))


def test_cache_budget_evicts_least_recently_used(oxh):
    """Cached (never registered) matrices are bounded; the budget is read once per process, so this only checks
    that many distinct matrices do not pile up beyond it and still compute correctly."""
    rows, cols = 128, 1024
    x = synth.normal(cols, seed=31)
    keep = []
    for i in range(6):
        w = synth.weights(13, rows, cols, seed=40 + i)
        keep.append(w)
        got = run(13, w, rows, cols, x)
        assert np.array_equal(got.view(np.uint32), oracle_matvec(13, w, rows, cols, x).view(np.uint32))
    n_cached, cached_bytes = stats(oxh)[1:3]
    assert n_cached >= 1 and cached_bytes >= rows * synth.row_bytes(13, cols)
    assert oxh.oxh_weight_clear() == 0
    assert stats(oxh)[:3] == (0, 0, 0)


def test_a_few_bytes_patched_in_place_are_seen_within_the_stated_number_of_calls(oxh):
    """What the default cache mode guarantees for an UNREGISTERED matrix that is edited in place at the same
    address and size (a patched tensor, a merged adapter): 64 bytes in the middle of a 33 MB matrix, between
    the fingerprint's samples.  The per-call check re-hashes two 16 KiB slices in turn against the hashes
    taken at upload, so the edit is seen after at most ceil(bytes / 32 KiB) calls; until then the old copy
    may be served (the stated limit), and oxh_weight_unregister makes the very next call see it."""
    rows, cols = 14336, 4096
    rb = synth.row_bytes(13, cols)
    w = synth.weights(13, rows, cols, seed=77)
    x = synth.normal(cols, seed=78)
    first = run(13, w, rows, cols, x)
    assert np.array_equal(first.view(np.uint32), oracle_matvec(13, w, rows, cols, x).view(np.uint32))
    r0 = stats(oxh)[3]

    # nibble bytes of one block of row 7001 (neither in the first / last 4 KiB nor on a sample)
    row, at = 7001, 7001 * rb + 5 * 144 + 16 + 40
    w[at:at + 64] ^= 0x5A
    want = oracle_matvec(13, w, rows, cols, x)
    assert want[row] != first[row]
    limit = -(-w.nbytes // 32768)
    seen_after = None
    for call in range(1, limit + 1):
        got = run(13, w, rows, cols, x)
        if stats(oxh)[3] == r0 + 1:
            seen_after = call
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
            break
        assert np.array_equal(got.view(np.uint32), first.view(np.uint32))      # the old copy, whole
    assert seen_after is not None and seen_after <= limit

    # the invalidate call: a second edit, then unregister, and the next call is right
    w[at:at + 64] ^= 0x33
    assert oxh.oxh_weight_unregister(w.ctypes.data) == 0
    got = run(13, w, rows, cols, x)
    assert np.array_equal(got.view(np.uint32), oracle_matvec(13, w, rows, cols, x).view(np.uint32))


def test_rewritten_forms_count_towards_the_cache_and_go_with_their_entry(oxh):
    """A cached Q6_K matrix keeps a regrouped copy next to it: the bytes cached grow by both, and dropping the
    entry returns both."""
    rows, cols = 256, 2048
    w = synth.weights(16, rows, cols, seed=5)
    x = synth.normal(cols, seed=6)
    assert oxh.oxh_weight_clear() == 0
    got = run(16, w, rows, cols, x)
    assert np.array_equal(got.view(np.uint32), oracle_matvec(16, w, rows, cols, x).view(np.uint32))
    assert stats(oxh)[2] == 2 * w.nbytes
    assert oxh.oxh_weight_unregister(w.ctypes.data) == 0
    assert stats(oxh)[:3] == (0, 0, 0)
    free_b, total_b = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert oxh.oxh_mem_info(ctypes.byref(free_b), ctypes.byref(total_b)) == 0
    assert 0 < free_b.value <= total_b.value
