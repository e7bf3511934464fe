"""GPU test of the model-file path: a GGUF file written by the test is mapped,
its quantized tensors are made resident, and the host-pointer matvec entry
points run straight from the mapped tensor views -- results against the CPU
oracle on the same bytes (bit-exact for the K-quants, the Q8_0 chain for
Q8_0)."""
import ctypes

import numpy as np
import pytest

import gguf_writer as gw
import oxlibs
from oxidize_amd import matvec as mv
from oxidize_amd import synth
from oxidize_amd.gguf import GgufFile

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def host_view(t):
    """The mapped tensor as a numpy array (no copy)."""
    buf = (ctypes.c_uint8 * t.nbytes).from_address(t.data)
    return np.frombuffer(buf, dtype=np.uint8)


def test_matvec_straight_from_a_mapped_model_file(oxh, tmp_path):
    specs = [("blk.0.attn_q.weight", 13, 12, 512, 1024), ("blk.0.attn_k.weight", 13, 12, 128, 1024),
             ("blk.0.ffn_down.weight", 16, 14, 256, 2816), ("blk.0.attn_v.weight", 15, 13, 128, 1024),
             ("output.weight", 7, 8, 1000, 896)]
    tensors = [(n, [c, r], ggml, gw.as_bytes(synth.weights(q, r, c, seed=5, stream=i)))
               for i, (n, q, ggml, r, c) in enumerate(specs)]
    n_exp, e_rows, e_cols = 4, 96, 512
    tensors.append(("blk.0.ffn_up_exps.weight", [e_cols, e_rows, n_exp], 12,
                    gw.as_bytes(synth.weights(13, n_exp * e_rows, e_cols, seed=6))))
    tensors.append(("blk.0.attn_norm.weight", [1024], 0, gw.as_bytes(synth.normal(1024, seed=5))))
    path = tmp_path / "model.gguf"
    path.write_bytes(gw.build([("general.architecture", gw.STRING, "llama")], tensors, alignment=64))
    o = oxlibs.oracle()
    with GgufFile(path) as g:
        n, nbytes = g.register_all()
        assert n == 6 and nbytes == sum(len(t[3]) for t in tensors[:6])     # every matrix, not the f32 norm
        assert g.find("blk.0.attn_norm.weight").resident == 0
        for name, q, ggml, rows, cols in specs:
            t = g.find(name)
            assert t.resident == 1 and (t.qtype, t.rows, t.cols) == (q, rows, cols)
            assert oxh.oxh_weight_device_ptr(ctypes.c_void_p(t.data)) is not None
            w = host_view(t)
            x = synth.normal(cols, seed=7, stream=rows)
            out = np.zeros(rows, np.float32)
            temp = np.zeros(cols, np.float32)
            assert mv.matvec_quantized(t.qtype, w, rows, cols, t.row_bytes, x, out, temp) == 0
            want = np.zeros(rows, np.float32)
            wtemp = np.zeros(cols, np.float32)
            assert o.oxo_matvec_quantized(t.qtype, w.ctypes.data, rows, cols, t.row_bytes, x.ctypes.data,
                                          want.ctypes.data, wtemp.ctypes.data) == 0
            assert np.array_equal(bits(out), bits(want)), name
        # expert slices of the stacked tensor resolve inside its one device copy
        t = g.find("blk.0.ffn_up_exps.weight")
        assert (t.rows, t.cols, t.row_bytes) == (n_exp * e_rows, e_cols, 288)
        base = oxh.oxh_weight_device_ptr(ctypes.c_void_p(t.data))
        w = host_view(t)
        x = synth.normal(e_cols, seed=8)
        for e in (3, 0, 2):
            sl = w[e * e_rows * t.row_bytes:(e + 1) * e_rows * t.row_bytes]
            assert oxh.oxh_weight_device_ptr(ctypes.c_void_p(sl.ctypes.data)) == base + e * e_rows * t.row_bytes
            out = np.zeros(e_rows, np.float32)
            temp = np.zeros(e_cols, np.float32)
            assert mv.matvec_quantized(13, sl, e_rows, e_cols, t.row_bytes, x, out, temp) == 0
            want = np.zeros(e_rows, np.float32)
            assert o.oxo_matvec_quantized(13, sl.ctypes.data, e_rows, e_cols, t.row_bytes, x.ctypes.data,
                                          want.ctypes.data, temp.ctypes.data) == 0
            assert np.array_equal(bits(out), bits(want))
        q_ptr = g.find("blk.0.attn_q.weight").data
    # closing the file dropped the device copies
    assert not oxh.oxh_weight_device_ptr(ctypes.c_void_p(q_ptr))
