"""Seeded synthetic tensors (raw Q4_K / Q5_K / Q6_K / Q8_0 blocks, f32 activations).

Thin ctypes wrapper over ``liboxsynth.so`` (built from ``csrc/synth.c``).  The
generator is integer-only, so the same seed gives the same bytes everywhere.
Shapes and distributions follow the benchmark configurations: Q4_K d/dmin
~ |N(0,0.02)|, 6-bit scales/mins uniform, nibbles uniform (Q5_K: the same plus a
uniform fifth-bit plane); Q6_K int8 scales in
[-32,31], codes uniform; Q8_0 int8 in [-127,127], d ~ |N(0,0.01)|.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q4_K, Q5_K, Q6_K = 3, 4, 5, 6, 7, 13, 15, 16
Q2_K, Q3_K = 8, 10                      # Q3_K also under ids 9 and 11 (the _S and _L variants)
AL5_XS = 18
IQ3_S, IQ1_XXXS = 25, 36                # codebook formats: f16 d, every other byte uniform
IQ4_NL, IQ4_XS = 26, 27                 # 4-bit codebook formats: f16 d, every other byte uniform
BLOCK_BYTES = {Q4_0: 18, Q4_1: 20, Q5_0: 22, Q5_1: 24, Q8_0: 34, Q4_K: 144, 12: 144, Q5_K: 176, 14: 176,
               Q6_K: 210, Q2_K: 84, 9: 110, Q3_K: 110, 11: 110, AL5_XS: 14, IQ3_S: 110, IQ1_XXXS: 38, IQ4_NL: 18, IQ4_XS: 136}
BLOCK_ELEMS = {Q4_0: 32, Q4_1: 32, Q5_0: 32, Q5_1: 32, Q8_0: 32, Q4_K: 256, 12: 256, Q5_K: 256, 14: 256,
               Q6_K: 256, Q2_K: 256, 9: 256, Q3_K: 256, 11: 256, AL5_XS: 32, IQ3_S: 256, IQ1_XXXS: 256, IQ4_NL: 32, IQ4_XS: 256}


def _lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboxsynth.so")
        if not os.path.exists(path):
            raise RuntimeError(
                "liboxsynth.so is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
        lib = ctypes.CDLL(path)
        for name in ("oxs_fill_q4_k", "oxs_fill_q5_k", "oxs_fill_q6_k", "oxs_fill_q8_0"):
            getattr(lib, name).argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint64,
                                           ctypes.c_uint64, ctypes.c_float]
            getattr(lib, name).restype = None
        lib.oxs_fill_legacy.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint64, ctypes.c_uint64,
                                        ctypes.c_float, ctypes.c_uint32, ctypes.c_int]
        lib.oxs_fill_legacy.restype = None
        lib.oxs_fill_q23_k.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint64, ctypes.c_uint64,
                                       ctypes.c_float, ctypes.c_int]
        lib.oxs_fill_q23_k.restype = None
        lib.oxs_fill_normal_f32.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint64,
                                            ctypes.c_uint64, ctypes.c_float]
        lib.oxs_fill_normal_f32.restype = None
        _LIB = lib
    return _LIB


def row_bytes(qtype, cols):
    return cols // BLOCK_ELEMS[qtype] * BLOCK_BYTES[qtype]


def weights(qtype, rows, cols, seed=0, stream=0, sigma=None, out=None):
    """rows x cols matrix of raw blocks of `qtype`, as a flat uint8 array."""
    if cols % BLOCK_ELEMS[qtype]:
        raise ValueError("cols must be a whole number of blocks")
    n_blocks = rows * (cols // BLOCK_ELEMS[qtype])
    nbytes = n_blocks * BLOCK_BYTES[qtype]
    if out is None:
        out = np.empty(nbytes, dtype=np.uint8)
    assert out.dtype == np.uint8 and out.size == nbytes and out.flags.c_contiguous
    if qtype in (Q4_0, Q4_1, Q5_0, Q5_1, AL5_XS, IQ3_S, IQ1_XXXS, IQ4_NL, IQ4_XS):
        _lib().oxs_fill_legacy(out.ctypes.data, n_blocks, seed, stream, 0.02 if sigma is None else sigma,
                               BLOCK_BYTES[qtype], int(qtype in (Q4_1, Q5_1)))
        return out
    if qtype in (Q2_K, 9, Q3_K, 11):
        _lib().oxs_fill_q23_k(out.ctypes.data, n_blocks, seed, stream, 0.02 if sigma is None else sigma,
                              int(qtype != Q2_K))
        return out
    fn = {Q8_0: "oxs_fill_q8_0", Q4_K: "oxs_fill_q4_k", 12: "oxs_fill_q4_k",
          Q5_K: "oxs_fill_q5_k", 14: "oxs_fill_q5_k", Q6_K: "oxs_fill_q6_k"}[qtype]
    if sigma is None:
        sigma = 0.01 if qtype == Q8_0 else 0.02
    getattr(_lib(), fn)(out.ctypes.data, n_blocks, seed, stream, sigma)
    return out


def normal(n, seed=0, stream=1000, scale=1.0):
    """n float32 values ~ N(0,1)*scale."""
    out = np.empty(n, dtype=np.float32)
    _lib().oxs_fill_normal_f32(out.ctypes.data, n, seed, stream, scale)
    return out
