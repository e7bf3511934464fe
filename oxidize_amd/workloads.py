"""Device-resident benchmark workloads built from synthetic tensors.

``DecodeSet`` is the Llama-3-8B-shaped decode GEMV set: per layer a fused
q/k/v projection (4096+1024+1024 rows x 4096, Q4_K), the o projection
(4096 x 4096, Q4_K), a fused gate/up projection (2 x 14336 x 4096, Q4_K) and
the down projection (4096 x 14336, Q6_K), 32 layers with distinct weights,
each GEMV preceded by the quantisation of its own f32 input vector — the
launch sequence a decode step of the reference issues through
oc_matvec_quantized_fused / oc_matvec_quantized (llama.c:4702, :3926, :3234).
"""
import numpy as np

from . import matvec as mv
from . import synth

Q80, Q4K, Q6K = 7, 13, 16

LLAMA3_8B = dict(hidden=4096, kv=1024, ffn=14336, layers=32)
QWEN2_5_0_5B = dict(hidden=896, kv=128, ffn=4864, layers=24)


class DecodeSet:
    def __init__(self, hidden=4096, kv=1024, ffn=14336, layers=32, seed=0, keep_host=(), q6_grouped=None,
                 qtypes=(Q4K, Q6K)):
        """q6_grouped: keep the Q6_K matrices resident in the regrouped layout the decode kernels read
        fastest (oxh_q6_k_group; same bytes, made once when the weights are loaded, as the host layer
        does for registered weights).  Default: wherever the shape allows it (ffn % 2048 == 0).
        qtypes: weight types of (q/k/v, o, gate/up) and of the down projection; (Q80, Q80) with
        QWEN2_5_0_5B's shapes is the reference's Q8_0 configuration."""
        self.hidden, self.kv, self.ffn, self.layers = hidden, kv, ffn, layers
        self.seed = seed
        qt_main, qt_down = qtypes
        if q6_grouped is None:
            q6_grouped = qt_down == Q6K and ffn % 2048 == 0
        elif q6_grouped and (ffn % 2048 or qt_down != Q6K):
            raise ValueError("the regrouped Q6_K layout needs Q6_K weights and ffn a multiple of 2048")
        self.q6_grouped = q6_grouped
        self.qtype_run = {qt_main: qt_main, qt_down: qt_down}
        if qt_down == Q6K:
            self.qtype_run[Q6K] = mv.Q6_K_G8 if q6_grouped else Q6K
        staging = None
        # (name, qtype, [rows...], cols, input index)
        self.ops = [
            ("qkv", qt_main, [hidden, kv, kv], hidden, 0),
            ("o", qt_main, [hidden], hidden, 1),
            ("gate_up", qt_main, [ffn, ffn], hidden, 2),
            ("down", qt_down, [hidden], ffn, 3),
        ]
        self.weights = []      # [layer][op] -> list of DeviceBuffer (one per segment)
        self.host = {}         # (layer, op, seg) -> numpy, for layers in keep_host
        self.weight_bytes = 0
        stream_id = 0
        for layer in range(layers):
            per_layer = []
            for op, (name, qt, rows, cols, _) in enumerate(self.ops):
                bufs = []
                for seg, r in enumerate(rows):
                    w = synth.weights(qt, r, cols, seed=seed, stream=stream_id)
                    stream_id += 1
                    if qt == Q6K and q6_grouped:
                        if staging is None or staging.nbytes < w.nbytes:
                            staging = mv.DeviceBuffer(w.nbytes)
                        staging.upload(w)
                        buf = mv.DeviceBuffer(w.nbytes)
                        mv.q6_k_group(staging.ptr, r, cols, buf.ptr)
                        mv.sync()
                        bufs.append(buf)
                    else:
                        bufs.append(mv.DeviceBuffer.from_host(w))
                    self.weight_bytes += w.nbytes
                    if layer in keep_host:
                        self.host[(layer, op, seg)] = w
                per_layer.append(bufs)
            self.weights.append(per_layer)
        # one f32 input per (layer, op): N(0,1)
        self.x_host = {}
        self.x, self.act, self.out = [], [], []
        self.io_bytes = 0
        for layer in range(layers):
            xs, acts, outs = [], [], []
            for op, (name, qt, rows, cols, _) in enumerate(self.ops):
                x = synth.normal(cols, seed=seed, stream=100000 + layer * 8 + op)
                if layer in keep_host:
                    self.x_host[(layer, op)] = x
                xs.append(mv.DeviceBuffer.from_host(x))
                acts.append(mv.DeviceBuffer(mv.act_bytes(qt, cols)))
                outs.append(mv.DeviceBuffer(sum(rows) * 4))
                self.io_bytes += cols * 4 + sum(rows) * 4
            self.x.append(xs)
            self.act.append(acts)
            self.out.append(outs)
        self.segments = []
        for layer in range(layers):
            per_layer = []
            for op, (name, qt, rows, cols, _) in enumerate(self.ops):
                items, off = [], 0
                for seg, r in enumerate(rows):
                    items.append((self.weights[layer][op][seg].ptr, self.out[layer][op].ptr + off * 4, r, 0))
                    off += r
                per_layer.append(mv.make_segments(items))
            self.segments.append(per_layer)

    @property
    def bytes_per_step(self):
        """Algorithmic bytes of one decode step: packed weights at their on-disk
        size plus the f32 activation read and f32 output written per GEMV."""
        return self.weight_bytes + self.io_bytes

    @property
    def ops_per_step(self):
        return sum(2 * sum(rows) * cols for _, _, rows, cols, _ in self.ops) * self.layers

    def launch_op(self, layer, op, stream=None, fused=True):
        """One decode matmul from its f32 input: a single launch that quantises
        the activation inside the GEMV kernel (fused=True, what the host API
        does), or the stand-alone quantiser followed by the GEMV."""
        name, qt, rows, cols, _ = self.ops[op]
        run = self.qtype_run[qt]
        if fused:
            mv.gemv_segments_f32(run, self.segments[layer][op], cols, self.x[layer][op].ptr, cols,
                                 self.act[layer][op].ptr, 1, 0, stream)
        else:
            mv.quantize(qt, self.x[layer][op].ptr, cols, 1, cols, self.act[layer][op].ptr, stream)
            mv.gemv_segments(run, self.segments[layer][op], cols, self.act[layer][op].ptr, 1, 0, stream)

    def launch_step(self, stream=None, fused=True):
        for layer in range(self.layers):
            for op in range(len(self.ops)):
                self.launch_op(layer, op, stream, fused)

    def plan_ops(self):
        """The step as the operation list of one persistent launch (mv.Plan): the same calls as
        launch_step(fused=True), in the same order."""
        ops = []
        for layer in range(self.layers):
            for op, (name, qt, rows, cols, _) in enumerate(self.ops):
                ops.append(dict(qtype=self.qtype_run[qt], segs=self.segments[layer][op], cols=cols,
                                d_x=self.x[layer][op].ptr, d_act_out=self.act[layer][op].ptr))
        return ops

    def output(self, layer, op):
        rows = sum(self.ops[op][2])
        return self.out[layer][op].download(np.float32, rows)

    def activation(self, layer, op):
        _, qt, _, cols, _ = self.ops[op]
        return self.act[layer][op].download(np.uint8, mv.act_bytes(qt, cols))


class DecodeChain:
    """The same matrices as a ``DecodeSet``, launched as the dependent chain a
    decode step really is, with the float steps between the matmuls fused into
    the GEMV launches (four launches per layer, nothing leaves the device):

      1. q/k/v = W_qkv . Q8K(rmsnorm(x + f) * g_attn)      x <- x + f   (f: the previous
                                                            layer's feed-forward output)
      2. o     = W_o . Q8K(a)                               a: attention output
      3. h     = silu(W_gate . n) * (W_up . n),  n = Q8K(rmsnorm(x + o) * g_ffn),  x <- x + o
      4. f     = W_down . Q8K(h)

    Attention itself (RoPE, KV cache, softmax) is not part of this library; its
    output is stood in for by the q projection so that every launch still
    depends on the one before it.  The residual stream alternates between two
    buffers because a launch may not store over a vector it reads."""

    def __init__(self, dset, eps=1e-5, seed=0, capture=False):
        self.d = dset
        self.eps = eps
        h, ffn, layers = dset.hidden, dset.ffn, dset.layers
        self.g_attn_host = [(synth.normal(h, seed=seed, stream=300000 + l) * np.float32(0.1) + np.float32(1.0))
                            .astype(np.float32) for l in range(layers)]
        self.g_ffn_host = [(synth.normal(h, seed=seed, stream=310000 + l) * np.float32(0.1) + np.float32(1.0))
                           .astype(np.float32) for l in range(layers)]
        self.g_attn = [mv.DeviceBuffer.from_host(g) for g in self.g_attn_host]
        self.g_ffn = [mv.DeviceBuffer.from_host(g) for g in self.g_ffn_host]
        self.x0_host = synth.normal(h, seed=seed, stream=320000)
        self.f0_host = np.zeros(h, np.float32)
        self.x0 = mv.DeviceBuffer.from_host(self.x0_host)
        self.f0 = mv.DeviceBuffer.from_host(self.f0_host)
        self.res = [mv.DeviceBuffer(h * 4) for _ in range(3)]     # residual stream, rotating
        self.qkv = mv.DeviceBuffer((h + 2 * dset.kv) * 4)
        self.o = mv.DeviceBuffer(h * 4)
        self.h = mv.DeviceBuffer(ffn * 4)
        self.f = mv.DeviceBuffer(h * 4)
        # per-stage copies for the parity test: [layer] -> dict of DeviceBuffers
        self.capture = capture
        self.cap = [dict(n1=mv.DeviceBuffer(h * 4), x1=mv.DeviceBuffer(h * 4), qkv=mv.DeviceBuffer((h + 2 * dset.kv) * 4),
                         o=mv.DeviceBuffer(h * 4), n2=mv.DeviceBuffer(h * 4), x2=mv.DeviceBuffer(h * 4),
                         h=mv.DeviceBuffer(ffn * 4), f=mv.DeviceBuffer(h * 4))
                    for _ in range(layers)] if capture else None
        self.segs = []
        for l in range(layers):
            w = dset.weights[l]
            off, qkv_items = 0, []
            for seg, r in enumerate(dset.ops[0][2]):
                qkv_items.append((w[0][seg].ptr, self.qkv.ptr + off * 4, r, 0))
                off += r
            self.segs.append(dict(
                qkv=mv.make_segments(qkv_items),
                o=mv.make_segments([(w[1][0].ptr, self.o.ptr, h, 0)]),
                gate_up=mv.make_segments([(w[2][0].ptr, self.h.ptr, ffn, 0, 0, w[2][1].ptr)]),
                down=mv.make_segments([(w[3][0].ptr, self.f.ptr, h, 0)])))

    @property
    def bytes_per_step(self):
        """Packed weights once, plus what the four launches of a layer read and
        write in f32: x, f, g, x' / q,k,v out; a in, o out; x, o, g in, x', h
        out; h in, f out."""
        d = self.d
        h, kv, ffn = d.hidden, d.kv, d.ffn
        per_layer = 4 * ((3 * h + h + (h + 2 * kv)) + (h + h) + (3 * h + h + ffn) + (ffn + h))
        return d.weight_bytes + d.layers * per_layer

    def plan_ops(self):
        """launch_step's calls as the operation list of one persistent launch (mv.Plan); no per-stage
        copies (capture must be off)."""
        assert not self.capture
        d = self.d
        h = d.hidden
        x, f = self.x0, self.f0
        turn = 0
        ops = []
        for l in range(d.layers):
            sg = self.segs[l]
            x1, x2 = self.res[turn % 3], self.res[(turn + 1) % 3]
            turn += 2
            ops.append(dict(qtype=Q4K, segs=sg["qkv"], cols=h, d_x=x.ptr, kind=mv.PRO_RMSNORM, d_b=self.g_attn[l].ptr,
                            eps=self.eps, d_add=f.ptr, d_sum_out=x1.ptr))
            ops.append(dict(qtype=Q4K, segs=sg["o"], cols=h, d_x=self.qkv.ptr))
            ops.append(dict(qtype=Q4K, segs=sg["gate_up"], cols=h, d_x=x1.ptr, kind=mv.PRO_RMSNORM,
                            d_b=self.g_ffn[l].ptr, eps=self.eps, d_add=self.o.ptr, d_sum_out=x2.ptr))
            ops.append(dict(qtype=d.qtype_run[Q6K], segs=sg["down"], cols=d.ffn, d_x=self.h.ptr))
            x, f = x2, self.f
        self.last_x = x
        return ops

    def launch_step(self, stream=None):
        d = self.d
        h = d.hidden
        x, f = self.x0, self.f0
        turn = 0
        for l in range(d.layers):
            sg = self.segs[l]
            cap = self.cap[l] if self.capture else None
            # three buffers in rotation: a launch never stores over a vector it reads
            x1, x2 = self.res[turn % 3], self.res[(turn + 1) % 3]
            turn += 2
            mv.gemv_segments_fused(Q4K, sg["qkv"], h, x.ptr, h, mv.PRO_RMSNORM, self.g_attn[l].ptr, self.eps,
                                   cap["n1"].ptr if cap else None, None, 1, 0, stream, d_add=f.ptr,
                                   d_sum_out=x1.ptr)
            mv.gemv_segments_f32(Q4K, sg["o"], h, self.qkv.ptr, h, None, 1, 0, stream)
            mv.gemv_segments_fused(Q4K, sg["gate_up"], h, x1.ptr, h, mv.PRO_RMSNORM, self.g_ffn[l].ptr, self.eps,
                                   cap["n2"].ptr if cap else None, None, 1, 0, stream, d_add=self.o.ptr,
                                   d_sum_out=x2.ptr)
            mv.gemv_segments_f32(d.qtype_run[Q6K], sg["down"], d.ffn, self.h.ptr, d.ffn, None, 1, 0, stream)
            if cap:
                for name, src in (("x1", x1), ("qkv", self.qkv), ("o", self.o), ("x2", x2), ("h", self.h),
                                  ("f", self.f)):
                    mv.copy_d2d(cap[name].ptr, src.ptr, cap[name].nbytes, stream)
            x, f = x2, self.f
        self.last_x = x


def route_top_k(logits, k=2, renorm=True):
    """Token -> expert routing as the reference's MoE layers do it
    (llama.c:5965-6031): softmax over the expert logits, the k largest
    probabilities by repeated strict-greater scan (ties keep the lower index),
    gate weights renormalised over the selected experts.  Host-side caller
    logic, not part of the matmul path; it only decides which GEMVs run."""
    logits = np.asarray(logits, dtype=np.float32)
    n_tok, n_exp = logits.shape
    ids = np.zeros((n_tok, k), np.int32)
    wts = np.zeros((n_tok, k), np.float32)
    for t in range(n_tok):
        p = np.exp(logits[t] - logits[t].max()).astype(np.float32)
        p = (p * np.float32(1.0 / float(p.astype(np.float64).sum()))).astype(np.float32)
        order = list(range(n_exp))
        for i in range(k):
            best = i
            for c in range(i + 1, n_exp):
                if p[order[c]] > p[order[best]]:
                    best = c
            order[i], order[best] = order[best], order[i]
            ids[t, i] = order[i]
        sel = p[ids[t]].astype(np.float64)
        norm = sel.sum() if renorm else 1.0
        wts[t] = (sel / (norm if norm > 0 else 1.0)).astype(np.float32)
    return ids, wts


def group_by_expert(ids, n_expert):
    """Counting sort of the (token, slot) pairs by expert, token order kept
    inside an expert (llama.c:6060-6069).  Returns (offsets[n_expert+1],
    token index per sorted pair)."""
    pairs = [(int(e), t) for t in range(ids.shape[0]) for e in ids[t]]
    counts = np.bincount([e for e, _ in pairs], minlength=n_expert)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    fill = offsets[:-1].copy()
    tok = np.zeros(len(pairs), np.int64)
    for e, t in pairs:
        tok[fill[e]] = t
        fill[e] += 1
    return offsets, tok


class MoESet:
    """Mixtral-8x7B-shaped expert GEMVs: 8 experts, top-2 routing of 16 decode
    tokens; gate/up 14336 x 4096 and down 4096 x 14336 per expert, all Q4_K,
    stacked expert-major as the reference stores them (llama.c:4248-4251).
    Every expert's matrices are applied only to the tokens routed to it: ONE
    launch for all experts' gate+up, ONE for all experts' down, each expert a
    segment with its own activation count.  tile_major: the stacks are rewritten
    once with oxh_tile16 and the launches read that form (same results, to the bit)."""

    def __init__(self, n_expert=8, top_k=2, n_tok=16, hidden=4096, ffn=14336, seed=0, keep_host=False,
                 tile_major=False):
        self.n_expert, self.top_k, self.n_tok = n_expert, top_k, n_tok
        self.hidden, self.ffn = hidden, ffn
        self.qtype_run = mv.Q4_K_T16 if tile_major else Q4K
        self.logits = synth.normal(n_tok * n_expert, seed=seed, stream=4242).reshape(n_tok, n_expert)
        self.ids, self.gate_w = route_top_k(self.logits, top_k)
        self.offsets, self.pair_tok = group_by_expert(self.ids, n_expert)
        n_pairs = n_tok * top_k
        rb_gu, rb_dn = synth.row_bytes(Q4K, hidden), synth.row_bytes(Q4K, ffn)
        self.host = {}
        self.w = {}
        for name, rows, cols, stream in (("gate", ffn, hidden, 700), ("up", ffn, hidden, 701),
                                         ("down", hidden, ffn, 702)):
            w = synth.weights(Q4K, n_expert * rows, cols, seed=seed, stream=stream)
            self.w[name] = mv.DeviceBuffer.from_host(w)
            if tile_major:
                assert rows % 16 == 0
                tiled = mv.DeviceBuffer(mv.tile16_bytes(Q4K, n_expert * rows, cols))
                mv.tile16(Q4K, self.w[name].ptr, n_expert * rows, cols, tiled.ptr)
                mv.sync()
                self.w[name].free()
                self.w[name] = tiled
            if keep_host:
                self.host[name] = w
        self.x_tok = synth.normal(n_tok * hidden, seed=seed, stream=4300).reshape(n_tok, hidden)
        self.xg = np.ascontiguousarray(self.x_tok[self.pair_tok])            # gathered per pair
        self.h = synth.normal(n_pairs * ffn, seed=seed, stream=4301).reshape(n_pairs, ffn)
        self.d_xg = mv.DeviceBuffer.from_host(self.xg)
        self.d_h = mv.DeviceBuffer.from_host(self.h)
        self.d_gate = mv.DeviceBuffer(n_pairs * ffn * 4)
        self.d_up = mv.DeviceBuffer(n_pairs * ffn * 4)
        self.d_down = mv.DeviceBuffer(n_pairs * hidden * 4)
        # room for the quantised activations: with it, launches of three or more
        # activations per expert run on the matrix cores
        self.d_act_x = mv.DeviceBuffer(n_pairs * mv.act_bytes(Q4K, hidden))
        self.d_act_h = mv.DeviceBuffer(n_pairs * mv.act_bytes(Q4K, ffn))
        gu, dn = [], []
        self.hit = 0
        for e in range(n_expert):
            lo, hi = int(self.offsets[e]), int(self.offsets[e + 1])
            if hi > lo:
                self.hit += 1
            for c0 in range(lo, hi, 8):
                m = min(8, hi - c0)
                gu.append((self.w["gate"].ptr + e * ffn * rb_gu, self.d_gate.ptr + c0 * ffn * 4, ffn, c0, m))
                gu.append((self.w["up"].ptr + e * ffn * rb_gu, self.d_up.ptr + c0 * ffn * 4, ffn, c0, m))
                dn.append((self.w["down"].ptr + e * hidden * rb_dn, self.d_down.ptr + c0 * hidden * 4, hidden, c0, m))
        self.seg_gu = [mv.make_segments(gu[i:i + 32]) for i in range(0, len(gu), 32)]
        self.seg_dn = [mv.make_segments(dn[i:i + 32]) for i in range(0, len(dn), 32)]
        per_expert = (2 * ffn * rb_gu + hidden * rb_dn)
        self.bytes_per_step = self.hit * per_expert + n_pairs * 4 * (hidden + 2 * ffn + ffn + hidden)
        self.ops_per_step = n_pairs * 2 * 3 * ffn * hidden

    def launch_step(self, stream=None):
        for segs in self.seg_gu:
            mv.gemv_segments_f32(self.qtype_run, segs, self.hidden, self.d_xg.ptr, self.hidden, self.d_act_x.ptr, 1,
                                 self.ffn, stream)
        for segs in self.seg_dn:
            mv.gemv_segments_f32(self.qtype_run, segs, self.ffn, self.d_h.ptr, self.ffn, self.d_act_h.ptr, 1,
                                 self.hidden, stream)

    def outputs(self):
        n_pairs = self.n_tok * self.top_k
        return (self.d_gate.download(np.float32, n_pairs * self.ffn).reshape(n_pairs, self.ffn),
                self.d_up.download(np.float32, n_pairs * self.ffn).reshape(n_pairs, self.ffn),
                self.d_down.download(np.float32, n_pairs * self.hidden).reshape(n_pairs, self.hidden))
