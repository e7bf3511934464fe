"""Host-side mirror of the reference's quantized-matvec interface over numpy
arrays, calling straight into liboxhip's C ABI.

Names and argument meaning follow oxidize-c/include/oxidize/matvec.h:
``matvec_quantized``, ``matvec_quantized_fused``,
``matvec_quantized_multi_input``, ``matvec_quantized_batch``.  Each returns the
library status (0 handled, 1 declined) and raises :class:`OxhError` on errors.
The ``Device*`` helpers wrap the device-resident layer for benchmarks.
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import DECLINED, OK, OxhError, OxhPrologue, OxhSegment, check, lib

Q8_0, Q4_K_S, Q4_K_M, Q5_K_S, Q5_K_M, Q6_K = 7, 12, 13, 14, 15, 16


def _p(a):
    return None if a is None else ctypes.c_void_p(a.ctypes.data)


def _status(rc):
    if rc in (OK, DECLINED):
        return rc
    return check(rc)


def _ptrs(arrays):
    return (ctypes.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])


def _sizes(values):
    return (ctypes.c_size_t * len(values))(*[int(v) for v in values])


def _u32s(values):
    return (ctypes.c_uint32 * len(values))(*[int(v) for v in values])


def matvec_quantized(qtype, data, rows, cols, row_bytes, x, out, temp):
    """out[r] = dot(W[r], Q8(x)); `temp` receives the quantised activation."""
    return _status(lib().oxh_matvec_quantized(qtype, _p(data), rows, cols, row_bytes,
                                              _p(x), _p(out), _p(temp)))


def matvec_quantized_fused(qtypes, datas, rows, cols, row_bytes, x, outs, temp):
    n = len(datas)
    return _status(lib().oxh_matvec_quantized_fused(
        _u32s(qtypes), _ptrs(datas), _sizes(rows), cols, _sizes(row_bytes), n, _p(x),
        _ptrs(outs), _p(temp)))


def matvec_quantized_multi_input(qtypes, datas, rows, cols, row_bytes, xs, outs, temp):
    n = len(datas)
    return _status(lib().oxh_matvec_quantized_multi_input(
        _u32s(qtypes), _ptrs(datas), _sizes(rows), cols, _sizes(row_bytes), n, _ptrs(xs),
        _ptrs(outs), _p(temp)))


def matvec_quantized_batch(qtype, data, rows, cols, row_bytes, xs, in_stride, outs,
                           out_stride, n_vec, temp, act_scratch):
    nbytes = 0 if act_scratch is None else act_scratch.nbytes
    return _status(lib().oxh_matvec_quantized_batch(
        qtype, _p(data), rows, cols, row_bytes, _p(xs), in_stride, _p(outs), out_stride,
        n_vec, _p(temp), _p(act_scratch), nbytes))


def batch_scratch_bytes(max_cols):
    return lib().oc_matvec_batch_scratch_bytes(max_cols)


# ─── device-resident layer ──────────────────────────────────────────────


class DeviceBuffer:
    """A hipMalloc'd range owned by this object."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        ptr = ctypes.c_void_p()
        check(lib().oxh_malloc(ctypes.byref(ptr), self.nbytes))
        self.ptr = ptr.value

    @classmethod
    def from_host(cls, array):
        array = np.ascontiguousarray(array)
        buf = cls(array.nbytes)
        buf.upload(array)
        return buf

    def upload(self, array, offset=0):
        array = np.ascontiguousarray(array)
        assert offset + array.nbytes <= self.nbytes
        check(lib().oxh_memcpy_h2d(ctypes.c_void_p(self.ptr + offset), _p(array),
                                   array.nbytes, None))
        check(lib().oxh_stream_sync(None))

    def download(self, dtype, count, offset=0):
        out = np.empty(count, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        check(lib().oxh_memcpy_d2h(_p(out), ctypes.c_void_p(self.ptr + offset), out.nbytes, None))
        check(lib().oxh_stream_sync(None))
        return out

    def free(self):
        if self.ptr:
            lib().oxh_stream_sync(None)
            lib().oxh_free(ctypes.c_void_p(self.ptr))
            self.ptr = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def copy_d2d(d_dst, d_src, nbytes, stream=None):
    check(lib().oxh_memcpy_d2d(ctypes.c_void_p(d_dst), ctypes.c_void_p(d_src), nbytes, stream))


def act_bytes(qtype, cols):
    return lib().oxh_act_bytes(qtype, cols)


def quantize(qtype, d_x, in_stride, n_vec, cols, d_act, stream=None):
    kind = lib().oxh_act_kind(qtype, cols)
    fn = lib().oxh_quantize_q8_k if kind == 2 else lib().oxh_quantize_q8_0
    check(fn(ctypes.c_void_p(d_x), in_stride, n_vec, cols, ctypes.c_void_p(d_act), stream))


def make_segments(items):
    """items: iterable of (d_w, d_out, rows, act_first[, n_vec[, d_w_pair]]) with
    integer addresses; n_vec 0/omitted = the launch's n_vec; d_w_pair = the second
    matrix of a gate/up pair (the segment then writes silu(gate) * up)."""
    items = list(items)
    segs = (OxhSegment * len(items))()
    for s, it in zip(segs, items):
        s.d_w, s.d_out, s.rows, s.act_first = it[0], it[1], it[2], it[3]
        s.n_vec = it[4] if len(it) > 4 else 0
        s.d_w_pair = it[5] if len(it) > 5 else None
    return segs


def gemv_segments(qtype, segs, cols, d_acts, n_vec=1, out_stride=0, stream=None):
    check(lib().oxh_gemv_segments(qtype, segs, len(segs), cols, ctypes.c_void_p(d_acts),
                                  n_vec, out_stride, stream))


def gemv_segments_f32(qtype, segs, cols, d_x, x_stride, d_act_out=None, n_vec=1, out_stride=0,
                      stream=None):
    """GEMV with the activation quantisation fused into the kernel."""
    check(lib().oxh_gemv_segments_f32(qtype, segs, len(segs), cols, ctypes.c_void_p(d_x), x_stride,
                                      None if d_act_out is None else ctypes.c_void_p(d_act_out),
                                      n_vec, out_stride, stream))


PRO_RMSNORM, PRO_SWIGLU = 1, 2


def gemv_segments_fused(qtype, segs, cols, d_x, x_stride, kind, d_b, eps=0.0, d_pro_out=None,
                        d_act_out=None, n_vec=1, out_stride=0, stream=None, d_add=None, d_sum_out=None):
    """GEMV with RMSNorm (d_b = norm weight; optionally of x + d_add, the sum
    stored to d_sum_out) or SwiGLU (d_x = gate, d_b = up) and the activation
    quantisation fused into the kernel."""
    def vp(a):
        return None if a is None else ctypes.c_void_p(a)
    pro = OxhPrologue(kind, eps, ctypes.c_void_p(d_b), vp(d_pro_out), vp(d_add), vp(d_sum_out))
    check(lib().oxh_gemv_segments_fused(qtype, segs, len(segs), cols, ctypes.c_void_p(d_x), x_stride,
                                        ctypes.byref(pro),
                                        None if d_act_out is None else ctypes.c_void_p(d_act_out),
                                        n_vec, out_stride, stream))


MMQ_RELAXED = 1


def mmq(qtype, d_w, rows, cols, d_acts, n_vec, d_out, out_stride, stream=None, flags=0):
    if flags:
        check(lib().oxh_mmq_ex(qtype, ctypes.c_void_p(d_w), rows, cols, ctypes.c_void_p(d_acts),
                               n_vec, ctypes.c_void_p(d_out), out_stride, flags, stream))
        return
    check(lib().oxh_mmq(qtype, ctypes.c_void_p(d_w), rows, cols, ctypes.c_void_p(d_acts),
                        n_vec, ctypes.c_void_p(d_out), out_stride, stream))


def mmq_split_workspace(qtype, rows, cols, n_vec, out_stride):
    """Bytes of workspace with which mmq_split shares a tile's columns between workgroups; 0 = it would not."""
    return int(lib().oxh_mmq_split_workspace(qtype, rows, cols, n_vec, out_stride))


def mmq_split(qtype, d_w, rows, cols, d_acts, n_vec, d_out, out_stride, d_ws, ws_bytes, stream=None):
    check(lib().oxh_mmq_split(qtype, ctypes.c_void_p(d_w), rows, cols, ctypes.c_void_p(d_acts), n_vec,
                              ctypes.c_void_p(d_out), out_stride, ctypes.c_void_p(d_ws) if d_ws else None, ws_bytes,
                              stream))


def mmq_tile(qtype, rows, n_vec, n_cu):
    """(rows, tokens) of the workgroup tile oxh_mmq would take; host arithmetic only."""
    r, t = ctypes.c_uint32(0), ctypes.c_uint32(0)
    check(lib().oxh_mmq_tile(qtype, rows, n_vec, n_cu, ctypes.byref(r), ctypes.byref(t)))
    return r.value, t.value


def get_rows(qtype, d_w, rows, cols, d_ids, n_ids, d_out, out_stride, stream=None):
    check(lib().oxh_get_rows(qtype, ctypes.c_void_p(d_w), rows, cols, ctypes.c_void_p(d_ids), n_ids,
                             ctypes.c_void_p(d_out), out_stride, stream))


def moe_route(d_logits, n_tok, n_expert, top_k, renorm, d_ids, d_wts, d_counts, d_offsets, d_perm, d_slot_pos,
              stream=None):
    vp = ctypes.c_void_p
    check(lib().oxh_moe_route(vp(d_logits), n_tok, n_expert, top_k, int(renorm), vp(d_ids), vp(d_wts),
                              vp(d_counts), vp(d_offsets), vp(d_perm), vp(d_slot_pos), stream))


class MoeLayer:
    """One mixture-of-experts feed-forward layer resident on the device
    (routing, grouping, expert matrices and combination as
    oxidize-c/src/model/llama.c:5965-6160); wraps oxh_moe_ffn and owns its
    workspace, sized for `max_tok` tokens."""

    PARTS = ("ids", "wts", "slot_pos", "perm", "counts", "offsets", "act_x", "gate", "up", "act_h", "y", "total")

    def __init__(self, qtype_gate_up, qtype_down, d_w_gate, d_w_up, d_w_down, n_expert, top_k, hidden, ffn,
                 renorm=True, max_tok=16):
        self.desc = _lib.OxhMoe(qtype_gate_up, qtype_down, d_w_gate, d_w_up, d_w_down, n_expert, top_k, hidden,
                                ffn, int(renorm))
        self.n_expert, self.top_k, self.hidden, self.ffn, self.max_tok = n_expert, top_k, hidden, ffn, max_tok
        need = ctypes.c_size_t()
        status = lib().oxh_moe_workspace_bytes(ctypes.byref(self.desc), max_tok, ctypes.byref(need))
        if status == DECLINED:
            raise OxhError(status, lib().oxh_last_error().decode())
        check(status)
        self.workspace = DeviceBuffer(need.value)

    def forward(self, d_logits, d_x, n_tok, d_out, x_stride=None, out_stride=None, stream=None):
        if n_tok > self.max_tok:
            raise ValueError("n_tok %d beyond the workspace's %d" % (n_tok, self.max_tok))
        check(lib().oxh_moe_ffn(ctypes.byref(self.desc), ctypes.c_void_p(d_logits), ctypes.c_void_p(d_x),
                                x_stride or self.hidden, n_tok, ctypes.c_void_p(d_out),
                                out_stride or self.hidden, ctypes.c_void_p(self.workspace.ptr),
                                self.workspace.nbytes, stream))

    def forward_static(self, d_logits, d_x, n_tok, d_out, x_stride=None, out_stride=None, stream=None):
        """The same layer through oxh_moe_ffn_static: no workspace argument, nothing allocated."""
        return lib().oxh_moe_ffn_static(ctypes.byref(self.desc), ctypes.c_void_p(d_logits), ctypes.c_void_p(d_x),
                                        x_stride or self.hidden, n_tok, ctypes.c_void_p(d_out),
                                        out_stride or self.hidden, stream)

    def parts(self, n_tok):
        """Offsets of the intermediates inside the workspace (test hook)."""
        v = (ctypes.c_size_t * 12)()
        check(_lib.lab().moe_workspace_parts(ctypes.byref(self.desc), n_tok, ctypes.byref(v)))
        return dict(zip(self.PARTS, [int(x) for x in v]))


def q3_k_as_q6_k(d_w, rows, cols, d_q6k, stream=None):
    """Rewrite a Q3_K matrix as a Q6_K one with bit-identical results (for oxh_mmq)."""
    check(lib().oxh_q3_k_as_q6_k(ctypes.c_void_p(d_w), rows, cols, ctypes.c_void_p(d_q6k), stream))


Q2_K_WIDE = 0x1008


def q2_k_widen(d_w, rows, cols, d_wide, stream=None):
    """Widen a Q2_K matrix to the 210-byte blocks oxh_mmq takes under Q2_K_WIDE."""
    check(lib().oxh_q2_k_widen(ctypes.c_void_p(d_w), rows, cols, ctypes.c_void_p(d_wide), stream))


Q6_K_G8 = 0x1009


def q6_k_group(d_w, rows, cols, d_g8, stream=None):
    """Q6_K regrouped in runs of eight blocks for the decode kernels (same size; cols % 2048 == 0)."""
    check(lib().oxh_q6_k_group(ctypes.c_void_p(d_w), rows, cols, ctypes.c_void_p(d_g8), stream))


Q4_K_T16, Q5_K_T16, Q8_0_T16 = 0x100A, 0x100B, 0x100C


def tile16_bytes(qtype, rows, cols):
    """Bytes of a Q4_K / Q5_K matrix stored tile-major (rows padded to whole sixteens); 0 = no such form."""
    return int(lib().oxh_tile16_bytes(qtype, rows, cols))


def tile16(qtype, d_w, rows, cols, d_t16, stream=None):
    """Rewrite a Q4_K / Q5_K matrix tile-major for the matrix-core tile kernels (Q4_K_T16 / Q5_K_T16)."""
    check(lib().oxh_tile16(qtype, ctypes.c_void_p(d_w), rows, cols, ctypes.c_void_p(d_t16), stream))


def read_probe(d_buf, nbytes, stream=None):
    """One launch that only reads `nbytes` at d_buf (measurement aid)."""
    check(_lib.lab().read_probe(ctypes.c_void_p(d_buf), nbytes, None, stream))


def debug_subblock_sums(qtype, d_w, rows, cols, d_act, d_sums, stream=None):
    check(_lib.lab().subblock_sums(qtype, ctypes.c_void_p(d_w), rows, cols,
                                        ctypes.c_void_p(d_act), ctypes.c_void_p(d_sums), stream))


class Plan:
    """A chain of decode matmuls compiled into one launch (oxh_plan_*).  `ops` is a list of dicts with the
    arguments of one gemv_segments_fused call each: qtype, segs (from make_segments), cols, d_x and
    optionally kind / d_b / eps / d_pro_out / d_add / d_sum_out (the prologue), d_act_out and out_stride
    (plans over Q8_0_T16 whose segments carry several activations)."""

    def __init__(self, ops):
        n = len(ops)
        self._keep = []
        arr = (_lib.OxhPlanOp * n)()

        def vp(a):
            return None if a is None else ctypes.c_void_p(a)
        for o, d in zip(arr, ops):
            o.qtype = d["qtype"]
            o.segs = ctypes.cast(d["segs"], ctypes.POINTER(OxhSegment))
            o.n_segs = len(d["segs"])
            o.cols = d["cols"]
            o.d_x = d["d_x"]
            if d.get("kind"):
                pro = OxhPrologue(d["kind"], d.get("eps", 0.0), vp(d.get("d_b")), vp(d.get("d_pro_out")),
                                  vp(d.get("d_add")), vp(d.get("d_sum_out")))
                self._keep.append(pro)
                o.pro = ctypes.pointer(pro)
            o.d_act_out = d.get("d_act_out")
            o.out_stride = d.get("out_stride", 0)
            self._keep.append(d["segs"])
        self.handle = ctypes.c_void_p()
        status = lib().oxh_plan_create(arr, n, ctypes.byref(self.handle))
        if status != OK:
            raise OxhError(status, lib().oxh_last_error().decode("utf-8", "replace"))

    def launch(self, stream=None):
        check(lib().oxh_plan_launch(self.handle, stream))

    def status(self, stream=None):
        """Waits for the stream; 0, or ERR_TIMEOUT when a launch gave up."""
        return lib().oxh_plan_status(self.handle, stream)

    def info(self):
        v = [ctypes.c_size_t() for _ in range(4)]
        check(lib().oxh_plan_info(self.handle, *[ctypes.byref(x) for x in v]))
        out = dict(zip(("n_ops", "n_waits", "workgroups", "lds_bytes"), [int(x.value) for x in v]))
        out["prestaged"] = bool(lib().oxh_plan_prestaged(self.handle))
        out["table_rows"] = lib().oxh_plan_table_rows(self.handle)
        return out

    def set_spin_limit(self, polls, phantom_workgroup=False):
        check(lib().oxh_plan_set_spin_limit(self.handle, polls))
        check(_lib.lab().plan_phantom(self.handle, int(phantom_workgroup)))

    def destroy(self):
        if self.handle:
            lib().oxh_plan_destroy(self.handle)
            self.handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def sync(stream=None):
    check(lib().oxh_stream_sync(stream))


def device_info():
    name = ctypes.create_string_buffer(256)
    n_cu, mhz, mem = ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
    check(lib().oxh_device_info(name, 256, ctypes.byref(n_cu), ctypes.byref(mhz), ctypes.byref(mem)))
    return {"name": name.value.decode(), "n_cu": n_cu.value, "clock_mhz": mhz.value,
            "mem_bytes": mem.value}


class Graph:
    """Capture of everything launched on `stream` inside the with-block."""

    def __init__(self, stream=None):
        self.stream = stream
        self.exec = ctypes.c_void_p()

    def __enter__(self):
        check(lib().oxh_graph_begin(self.stream))
        return self

    def __exit__(self, exc_type, exc, tb):
        rc = lib().oxh_graph_end(self.stream, ctypes.byref(self.exec))
        if exc_type is None:
            check(rc)
        return False

    def launch(self):
        check(lib().oxh_graph_launch(self.exec, self.stream))

    def destroy(self):
        if self.exec:
            lib().oxh_graph_destroy(self.exec)
            self.exec = ctypes.c_void_p()


class Event:
    def __init__(self):
        self.handle = ctypes.c_void_p()
        check(lib().oxh_event_create(ctypes.byref(self.handle)))

    def record(self, stream=None):
        check(lib().oxh_event_record(self.handle, stream))

    def sync(self):
        check(lib().oxh_event_sync(self.handle))

    def ms_since(self, start):
        ms = ctypes.c_float()
        check(lib().oxh_event_elapsed_ms(start.handle, self.handle, ctypes.byref(ms)))
        return ms.value
