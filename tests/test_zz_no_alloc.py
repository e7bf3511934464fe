"""oxh_moe_ffn_static: the mixture-of-experts layer for callers that cannot allocate.  Its workspace is a
device array built into the library; its results must be oxh_moe_ffn's, bit for bit, also when a call
follows a larger one whose intermediates still fill that array."""
import ctypes

import numpy as np
import pytest

from oxidize_amd import _lib, synth
from oxidize_amd import matvec as mv

pytestmark = pytest.mark.gpu
Q4K, Q6K = 13, 16


def layer(qt_gu, qt_dn, n_expert, top_k, hidden, ffn, seed):
    w = {}
    for name, qt, rows, cols in (("gate", qt_gu, n_expert * ffn, hidden), ("up", qt_gu, n_expert * ffn, hidden),
                                 ("down", qt_dn, n_expert * hidden, ffn)):
        w[name] = mv.DeviceBuffer.from_host(synth.weights(qt, rows, cols, seed=seed, stream=len(name)))
    moe = mv.MoeLayer(qt_gu, qt_dn, w["gate"].ptr, w["up"].ptr, w["down"].ptr, n_expert, top_k, hidden, ffn,
                      renorm=True, max_tok=64)
    return moe, w


def both(moe, n_tok, n_expert, hidden, seed):
    logits = synth.normal(n_tok * n_expert, seed=seed, stream=1).reshape(n_tok, n_expert)
    x = synth.normal(n_tok * hidden, seed=seed, stream=2).reshape(n_tok, hidden)
    d_l, d_x = mv.DeviceBuffer.from_host(logits), mv.DeviceBuffer.from_host(x)
    d_a, d_b = mv.DeviceBuffer(4 * n_tok * hidden), mv.DeviceBuffer(4 * n_tok * hidden)
    moe.forward(d_l.ptr, d_x.ptr, n_tok, d_a.ptr)
    mv.sync()
    assert moe.forward_static(d_l.ptr, d_x.ptr, n_tok, d_b.ptr) == 0
    mv.sync()
    a = d_a.download(np.float32, n_tok * hidden)
    b = d_b.download(np.float32, n_tok * hidden)
    assert np.all(np.isfinite(a)) and float(np.abs(a).max()) > 0.0
    return a.view(np.uint32), b.view(np.uint32)


@pytest.mark.parametrize("qt_gu,qt_dn", [(Q4K, Q4K), (Q4K, Q6K)])
def test_static_workspace_matches_the_caller_workspace_entry(oxh, qt_gu, qt_dn):
    n_expert, top_k, hidden, ffn = 8, 2, 512, 1024
    moe, keep = layer(qt_gu, qt_dn, n_expert, top_k, hidden, ffn, seed=5)
    # two calls in a row on the one built-in array, the second smaller than the first
    for n_tok, seed in ((40, 1), (7, 2), (1, 3)):
        a, b = both(moe, n_tok, n_expert, hidden, seed)
        assert np.array_equal(a, b), n_tok
    del keep


def test_static_workspace_limit_and_arguments(oxh):
    n_expert, top_k, hidden, ffn = 8, 2, 4096, 14336
    # weights are never touched by a refused call: any non-NULL pointer will do
    dummy = mv.DeviceBuffer(256)
    moe = mv.MoeLayer(Q4K, Q4K, dummy.ptr, dummy.ptr, dummy.ptr, n_expert, top_k, hidden, ffn, max_tok=1)
    need = ctypes.c_size_t()
    assert oxh.oxh_moe_workspace_bytes(ctypes.byref(moe.desc), 64, ctypes.byref(need)) == 0
    assert need.value > (8 << 20)
    assert moe.forward_static(dummy.ptr, dummy.ptr, 64, dummy.ptr) == _lib.ERR_TOO_WIDE
    assert b"workspace" in oxh.oxh_last_error()
    assert oxh.oxh_moe_workspace_bytes(ctypes.byref(moe.desc), 16, ctypes.byref(need)) == 0
    assert need.value <= (8 << 20)                      # the Mixtral-shaped decode batch fits
    assert moe.forward_static(None, dummy.ptr, 16, dummy.ptr) == _lib.ERR_ARG
