"""ctypes binding of liboxhip.so (the C ABI declared in include/oxhip.h).

Loading fails loudly when the library has not been built: there is no Python
or CPU implementation behind these calls.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboxhip.so")

OK, DECLINED = 0, 1
ERR_HIP, ERR_ARG, ERR_NO_DEVICE, ERR_TOO_WIDE, ERR_NOMEM, ERR_FORMAT, ERR_IO, ERR_TIMEOUT = -1, -2, -3, -4, -5, -6, -7, -8

V = ctypes.c_void_p
Z = ctypes.c_size_t
U32 = ctypes.c_uint32
I = ctypes.c_int


class OxhSegment(ctypes.Structure):
    _fields_ = [("d_w", V), ("d_out", V), ("rows", Z), ("act_first", Z), ("n_vec", Z),
                ("d_w_pair", V)]


class OxhPrologue(ctypes.Structure):
    _fields_ = [("kind", U32), ("eps", ctypes.c_float), ("d_b", V), ("d_out", V), ("d_add", V),
                ("d_sum_out", V)]


class OxhPlanOp(ctypes.Structure):
    _fields_ = [("qtype", U32), ("segs", ctypes.POINTER(OxhSegment)), ("n_segs", Z), ("cols", Z), ("d_x", V),
                ("pro", ctypes.POINTER(OxhPrologue)), ("d_act_out", V), ("out_stride", Z)]


class OxhMoe(ctypes.Structure):
    _fields_ = [("qtype_gate_up", U32), ("qtype_down", U32), ("d_w_gate", V), ("d_w_up", V), ("d_w_down", V),
                ("n_expert", Z), ("top_k", Z), ("hidden", Z), ("ffn", Z), ("renorm", I)]


class OxhTensor(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("qtype", U32), ("ggml_type", U32), ("n_dims", U32),
                ("dims", ctypes.c_uint64 * 8), ("offset", ctypes.c_uint64), ("data", V), ("nbytes", Z),
                ("rows", Z), ("cols", Z), ("row_bytes", Z), ("resident", I)]


class OcMatvecFusedTestStats(ctypes.Structure):
    _fields_ = [("activation_quantizations", Z), ("parallel_dispatches", Z),
                ("fallback_calls", Z)]


class OxhLab(ctypes.Structure):
    """include/oxhip_lab.h: test hooks and measurement aids, reached through oxh_lab()."""
    _fields_ = [("plan_stamps", ctypes.CFUNCTYPE(I, V, V)),
                ("plan_phantom", ctypes.CFUNCTYPE(I, V, I)),
                ("moe_workspace_parts", ctypes.CFUNCTYPE(I, ctypes.POINTER(OxhMoe), Z, ctypes.POINTER(Z * 12))),
                ("read_probe", ctypes.CFUNCTYPE(I, V, Z, V, V)),
                ("mfma_probe", ctypes.CFUNCTYPE(I, I, I, ctypes.POINTER(ctypes.c_double))),
                ("subblock_sums", ctypes.CFUNCTYPE(I, U32, V, Z, Z, V, V, V))]


# name -> (restype, argtypes); every symbol include/oxhip.h and include/oxhip_lab.h declare
SIGNATURES = {
    "oxh_lab": (ctypes.POINTER(OxhLab), []),
    "oxh_last_error": (ctypes.c_char_p, []),
    "oxh_init": (I, [I]),
    "oxh_shutdown": (None, []),
    "oxh_act_kind": (I, [U32, Z]),
    "oxh_row_bytes": (Z, [U32, Z]),
    "oxh_act_bytes": (Z, [U32, Z]),
    "oxh_f32_path_row_bytes": (Z, [U32, Z]),
    "oxh_quantize_q8_k": (I, [V, Z, Z, Z, V, V]),
    "oxh_quantize_q8_0": (I, [V, Z, Z, Z, V, V]),
    "oxh_gemv_segments": (I, [U32, ctypes.POINTER(OxhSegment), Z, Z, V, Z, Z, V]),
    "oxh_gemv_segments_f32": (I, [U32, ctypes.POINTER(OxhSegment), Z, Z, V, Z, V, Z, Z, V]),
    "oxh_gemv_segments_fused": (I, [U32, ctypes.POINTER(OxhSegment), Z, Z, V, Z,
                                    ctypes.POINTER(OxhPrologue), V, Z, Z, V]),
    "oxh_plan_create": (I, [ctypes.POINTER(OxhPlanOp), Z, ctypes.POINTER(V)]),
    "oxh_plan_launch": (I, [V, V]),
    "oxh_plan_status": (I, [V, V]),
    "oxh_plan_info": (I, [V, ctypes.POINTER(Z), ctypes.POINTER(Z), ctypes.POINTER(Z), ctypes.POINTER(Z)]),
    "oxh_plan_prestaged": (I, [V]),
    "oxh_plan_table_rows": (I, [V]),
    "oxh_q6_k_group": (I, [V, Z, Z, V, V]),
    "oxh_tile16_bytes": (Z, [U32, Z, Z]),
    "oxh_tile16": (I, [U32, V, Z, Z, V, V]),
    "oxh_plan_set_spin_limit": (I, [V, U32]),
    "oxh_plan_destroy": (I, [V]),
    "oxh_plan_deal": (I, [ctypes.POINTER(Z), ctypes.POINTER(I), Z, U32, ctypes.POINTER(U32), ctypes.POINTER(U32)]),
    "oxh_mmq": (I, [U32, V, Z, Z, V, Z, V, Z, V]),
    "oxh_mmq_ex": (I, [U32, V, Z, Z, V, Z, V, Z, U32, V]),
    "oxh_mmq_tile": (I, [U32, Z, Z, Z, ctypes.POINTER(U32), ctypes.POINTER(U32)]),
    "oxh_mmq_split_workspace": (Z, [U32, Z, Z, Z, Z]),
    "oxh_mmq_split": (I, [U32, V, Z, Z, V, Z, V, Z, V, Z, V]),
    "oxh_get_rows": (I, [U32, V, Z, Z, V, Z, V, Z, V]),
    "oxh_q3_k_as_q6_k": (I, [V, Z, Z, V, V]),
    "oxh_q2_k_widen": (I, [V, Z, Z, V, V]),
    "oxh_moe_workspace_bytes": (I, [ctypes.POINTER(OxhMoe), Z, ctypes.POINTER(Z)]),
    "oxh_moe_ffn": (I, [ctypes.POINTER(OxhMoe), V, V, Z, Z, V, Z, V, Z, V]),
    "oxh_moe_ffn_static": (I, [ctypes.POINTER(OxhMoe), V, V, Z, Z, V, Z, V]),
    "oxh_moe_route": (I, [V, Z, Z, Z, I, V, V, V, V, V, V, V]),
    "oxh_malloc": (I, [ctypes.POINTER(V), Z]),
    "oxh_host_alloc": (I, [ctypes.POINTER(V), Z]),
    "oxh_host_free": (I, [V]),
    "oxh_free": (I, [V]),
    "oxh_memcpy_h2d": (I, [V, V, Z, V]),
    "oxh_memcpy_d2h": (I, [V, V, Z, V]),
    "oxh_memcpy_d2d": (I, [V, V, Z, V]),
    "oxh_memcpy2d_h2d": (I, [V, Z, V, Z, Z, Z, V]),
    "oxh_memcpy2d_d2h": (I, [V, Z, V, Z, Z, Z, V]),
    "oxh_memset": (I, [V, I, Z, V]),
    "oxh_stream_create": (I, [ctypes.POINTER(V)]),
    "oxh_stream_destroy": (I, [V]),
    "oxh_stream_sync": (I, [V]),
    "oxh_event_create": (I, [ctypes.POINTER(V)]),
    "oxh_event_destroy": (I, [V]),
    "oxh_event_record": (I, [V, V]),
    "oxh_event_sync": (I, [V]),
    "oxh_event_elapsed_ms": (I, [V, V, ctypes.POINTER(ctypes.c_float)]),
    "oxh_graph_begin": (I, [V]),
    "oxh_graph_end": (I, [V, ctypes.POINTER(V)]),
    "oxh_graph_launch": (I, [V, V]),
    "oxh_graph_destroy": (I, [V]),
    "oxh_device_info": (I, [ctypes.c_char_p, Z, ctypes.POINTER(I), ctypes.POINTER(I),
                            ctypes.POINTER(Z)]),
    "oxh_mem_info": (I, [ctypes.POINTER(Z), ctypes.POINTER(Z)]),
    "oxh_gguf_open": (I, [ctypes.c_char_p, ctypes.POINTER(V)]),
    "oxh_gguf_close": (None, [V]),
    "oxh_gguf_info": (I, [V, ctypes.POINTER(U32), ctypes.POINTER(ctypes.c_uint64),
                          ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(Z), ctypes.POINTER(Z)]),
    "oxh_gguf_tensor_at": (I, [V, Z, ctypes.POINTER(OxhTensor)]),
    "oxh_gguf_tensor_find": (I, [V, ctypes.c_char_p, ctypes.POINTER(OxhTensor)]),
    "oxh_gguf_meta_u64": (I, [V, ctypes.c_char_p, ctypes.POINTER(ctypes.c_uint64)]),
    "oxh_gguf_meta_f64": (I, [V, ctypes.c_char_p, ctypes.POINTER(ctypes.c_double)]),
    "oxh_gguf_meta_str": (I, [V, ctypes.c_char_p, ctypes.POINTER(V), ctypes.POINTER(Z)]),
    "oxh_gguf_register_all": (I, [V, ctypes.POINTER(Z), ctypes.POINTER(Z)]),
    "oxh_qtype_from_ggml_id": (U32, [U32]),
    "oxh_weight_register": (I, [V, Z]),
    "oxh_weight_unregister": (I, [V]),
    "oxh_weight_clear": (I, []),
    "oxh_weight_device_ptr": (V, [V]),
    "oxh_weight_stats": (I, [ctypes.POINTER(Z), ctypes.POINTER(Z), ctypes.POINTER(Z), ctypes.POINTER(Z)]),
    "oxh_weight_evictions": (Z, []),
    "oxh_matvec_quantized": (I, [U32, V, Z, Z, Z, V, V, V]),
    "oxh_matvec_quantized_fused": (I, [V, V, V, Z, V, Z, V, V, V]),
    "oxh_matvec_quantized_multi_input": (I, [V, V, V, Z, V, Z, V, V, V]),
    "oxh_matvec_quantized_batch": (I, [U32, V, Z, Z, Z, V, Z, V, Z, Z, V, V, Z]),
    "oc_matvec_quantized": (None, [U32, V, Z, Z, Z, V, V, V]),
    "oc_matvec_quantized_fused": (None, [V, V, V, Z, V, Z, V, V, V]),
    "oc_matvec_quantized_multi_input": (None, [V, V, V, Z, V, Z, V, V, V]),
    "oc_matvec_quantized_batch": (None, [U32, V, Z, Z, Z, V, Z, V, Z, Z, V, V, Z]),
    "oc_matvec_batch_scratch_bytes": (Z, [Z]),
    "oc_matvec_set_fused": (None, [ctypes.c_bool]),
    "oc_matvec_fused_enabled": (ctypes.c_bool, []),
    "oc_matvec_fused_test_reset": (None, []),
    "oc_matvec_fused_test_stats": (OcMatvecFusedTestStats, []),
    "oxh_set_decline_handler": (None, [V, V]),
    "oxh_set_cpu_fallback": (None, [V]),
    "oxh_cpu_fallback_calls": (Z, []),
}

_LIB = None


class OxhError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("liboxhip status %d: %s" % (status, message))
        self.status = status


def lib():
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "liboxhip.so has not been built (expected %s); run "
                "`python -c 'import __graft_entry__ as g; g.build()'`" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _LIB = handle
    return _LIB


def lab():
    """The table of test hooks and measurement aids (include/oxhip_lab.h)."""
    return lib().oxh_lab().contents


def check(status):
    """Raise on anything but OXH_OK."""
    if status != OK:
        raise OxhError(status, lib().oxh_last_error().decode("utf-8", "replace"))
    return status
