"""ctypes handles on the two CPU checkers used by the tests.

``oracle()``  -> oracle/liboxoracle.so, our scalar restatement (always built).
``ref()``     -> oracle/_ref/liboxref.so, the reference's own sources compiled
                 as a shared object (None when it was never built).
Neither is ever loaded by the shipped package.
"""
import ctypes
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
c_u8p = ctypes.POINTER(ctypes.c_uint8)
c_f32p = ctypes.POINTER(ctypes.c_float)
c_i32p = ctypes.POINTER(ctypes.c_int32)

_ORACLE = None
_REF = False


def ptr(a, ty=ctypes.c_void_p):
    if a is None:
        return None
    return ctypes.cast(a.ctypes.data, ty) if ty is not ctypes.c_void_p else ctypes.c_void_p(a.ctypes.data)


def oracle():
    global _ORACLE
    if _ORACLE is None:
        path = os.path.join(ROOT, "oracle", "liboxoracle.so")
        if not os.path.exists(path):
            raise RuntimeError("oracle/liboxoracle.so missing: run `make -C oracle`")
        lib = ctypes.CDLL(path)
        V, Z, U32, F = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32, ctypes.c_float
        lib.oxo_f16_to_f32.argtypes = [ctypes.c_uint16]; lib.oxo_f16_to_f32.restype = F
        lib.oxo_f32_to_f16_bits.argtypes = [F]; lib.oxo_f32_to_f16_bits.restype = ctypes.c_uint16
        lib.oxo_scale_min_k4.argtypes = [ctypes.c_uint, V, V, V]; lib.oxo_scale_min_k4.restype = None
        lib.oxo_quantize_q8_k.argtypes = [V, Z, V]; lib.oxo_quantize_q8_k.restype = None
        lib.oxo_quantize_q8_0.argtypes = [V, Z, V]; lib.oxo_quantize_q8_0.restype = None
        lib.oxo_dot_q4_k_q8_k.argtypes = [V, Z, V, V, V]; lib.oxo_dot_q4_k_q8_k.restype = F
        lib.oxo_dot_q5_k_q8_k.argtypes = [V, Z, V, V, V]; lib.oxo_dot_q5_k_q8_k.restype = F
        lib.oxo_dot_q6_k_q8_k.argtypes = [V, Z, V, V]; lib.oxo_dot_q6_k_q8_k.restype = F
        lib.oxo_dot_q8_0_q8_0.argtypes = [V, Z, V, V]; lib.oxo_dot_q8_0_q8_0.restype = F
        lib.oxo_dot_q2_k_q8_k.argtypes = [V, Z, V, V]; lib.oxo_dot_q2_k_q8_k.restype = F
        lib.oxo_dot_iq3_s_q8_k.argtypes = [V, Z, V, V]; lib.oxo_dot_iq3_s_q8_k.restype = F
        lib.oxo_dot_iq1_xxxs_q8_k.argtypes = [V, Z, V, V]; lib.oxo_dot_iq1_xxxs_q8_k.restype = F
        lib.oxo_dot_q3_k_q8_k.argtypes = [V, Z, V, V]; lib.oxo_dot_q3_k_q8_k.restype = F
        for n in ("q4_0", "q4_1", "q5_0", "q5_1", "al5_xs"):
            f = getattr(lib, "oxo_dot_%s_q8_0" % n)
            f.argtypes = [V, Z, V, V]; f.restype = F
        lib.oxo_act_kind.argtypes = [U32, Z]; lib.oxo_act_kind.restype = ctypes.c_int
        lib.oxo_stride_ok.argtypes = [U32, Z, Z]; lib.oxo_stride_ok.restype = ctypes.c_int
        lib.oxo_matvec_quantized.argtypes = [U32, V, Z, Z, Z, V, V, V]
        lib.oxo_matvec_quantized.restype = ctypes.c_int
        lib.oxo_matvec_quantized_fused.argtypes = [V, V, V, Z, V, Z, V, V, V]
        lib.oxo_matvec_quantized_fused.restype = ctypes.c_int
        lib.oxo_matvec_quantized_multi_input.argtypes = [V, V, V, Z, V, Z, V, V, V]
        lib.oxo_matvec_quantized_multi_input.restype = ctypes.c_int
        lib.oxo_matvec_quantized_batch.argtypes = [U32, V, Z, Z, Z, V, Z, V, Z, Z, V, Z]
        lib.oxo_matvec_quantized_batch.restype = ctypes.c_int
        lib.oxo_matvec_batch_scratch_bytes.argtypes = [Z]
        lib.oxo_matvec_batch_scratch_bytes.restype = Z
        lib.oxo_moe_route.argtypes = [V, Z, Z, Z, ctypes.c_int, V, V]; lib.oxo_moe_route.restype = None
        lib.oxo_moe_ffn.argtypes = [U32, U32, V, V, V, Z, Z, Z, Z, ctypes.c_int, V, V, Z, V]
        lib.oxo_moe_ffn.restype = ctypes.c_int
        lib.oxo_dequant_row.argtypes = [U32, V, Z, V]; lib.oxo_dequant_row.restype = ctypes.c_int
        lib.oxo_matvec_dequant.argtypes = [U32, V, Z, Z, Z, V, V, V]; lib.oxo_matvec_dequant.restype = ctypes.c_int
        lib.oxo_dequant_path_row_bytes.argtypes = [U32, Z]; lib.oxo_dequant_path_row_bytes.restype = Z
        lib.oxo_rms_norm_f32.argtypes = [V, V, V, Z, F]; lib.oxo_rms_norm_f32.restype = None
        lib.oxo_swiglu_f32.argtypes = [V, V, V, Z]; lib.oxo_swiglu_f32.restype = None
        _ORACLE = lib
    return _ORACLE


def ref():
    """The compiled reference, or None.  Symbols keep the reference's names."""
    global _REF
    if _REF is False:
        path = os.path.join(ROOT, "oracle", "_ref", "liboxref.so")
        if not os.path.exists(path):
            _REF = None
            return None
        lib = ctypes.CDLL(path)
        V, Z, U32, F = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32, ctypes.c_float
        lib.oc_oxk_f16_le_to_f32.argtypes = [V]; lib.oc_oxk_f16_le_to_f32.restype = F
        lib.oc_f32_to_f16_bits.argtypes = [F]; lib.oc_f32_to_f16_bits.restype = ctypes.c_uint16
        lib.oc_oxk_get_scale_min_k4.argtypes = [ctypes.c_uint, V, V, V]
        lib.oc_oxk_get_scale_min_k4.restype = None
        for n in ("q2_k_q8_k", "q3_k_q8_k", "q4_k_q8_k", "q5_k_q8_k", "q6_k_q8_k", "q8_0_q8_0", "q4_0_q8_0", "q4_1_q8_0", "q5_0_q8_0",
                  "q5_1_q8_0", "al5_xs_q8_0"):
            for suf in ("", "_scalar"):
                f = getattr(lib, "oc_oxk_dot_" + n + suf)
                f.argtypes = [V, Z, V]; f.restype = F
        lib.oc_matvec_quantized.argtypes = [U32, V, Z, Z, Z, V, V, V]
        lib.oc_matvec_quantized.restype = None
        lib.oc_matvec_quantized_fused.argtypes = [V, V, V, Z, V, Z, V, V, V]
        lib.oc_matvec_quantized_fused.restype = None
        lib.oc_matvec_quantized_multi_input.argtypes = [V, V, V, Z, V, Z, V, V, V]
        lib.oc_matvec_quantized_multi_input.restype = None
        lib.oc_matvec_quantized_batch.argtypes = [U32, V, Z, Z, Z, V, Z, V, Z, Z, V, V, Z]
        lib.oc_matvec_quantized_batch.restype = None
        lib.oc_matvec_batch_scratch_bytes.argtypes = [Z]
        lib.oc_matvec_batch_scratch_bytes.restype = Z
        lib.oc_parallel_set_threads.argtypes = [Z]; lib.oc_parallel_set_threads.restype = ctypes.c_int
        lib.oc_parallel_n_threads.restype = Z
        lib.oc_quant_dequant_row.argtypes = [U32, V, Z, V, Z]; lib.oc_quant_dequant_row.restype = ctypes.c_int
        if hasattr(lib, "oc_rms_norm_f32"):
            lib.oc_rms_norm_f32.argtypes = [V, V, V, Z, F]; lib.oc_rms_norm_f32.restype = None
            lib.oc_swiglu_inplace_f32.argtypes = [V, V, Z]; lib.oc_swiglu_inplace_f32.restype = None
        _REF = lib
    return _REF


def ptr_array(arrays):
    """void*[] over a list of numpy arrays (kept alive by the caller)."""
    return (ctypes.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])


def size_array(values):
    return (ctypes.c_size_t * len(values))(*values)


def u32_array(values):
    return (ctypes.c_uint32 * len(values))(*values)
