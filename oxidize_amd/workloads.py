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


class DecodeSet:
    def __init__(self, hidden=4096, kv=1024, ffn=14336, layers=32, seed=0, keep_host=()):
        self.hidden, self.kv, self.ffn, self.layers = hidden, kv, ffn, layers
        self.seed = seed
        # (name, qtype, [rows...], cols, input index)
        self.ops = [
            ("qkv", Q4K, [hidden, kv, kv], hidden, 0),
            ("o", Q4K, [hidden], hidden, 1),
            ("gate_up", Q4K, [ffn, ffn], hidden, 2),
            ("down", Q6K, [hidden], ffn, 3),
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
        if fused:
            mv.gemv_segments_f32(qt, self.segments[layer][op], cols, self.x[layer][op].ptr, cols,
                                 self.act[layer][op].ptr, 1, 0, stream)
        else:
            mv.quantize(qt, self.x[layer][op].ptr, cols, 1, cols, self.act[layer][op].ptr, stream)
            mv.gemv_segments(qt, self.segments[layer][op], cols, self.act[layer][op].ptr, 1, 0, stream)

    def launch_step(self, stream=None, fused=True):
        for layer in range(self.layers):
            for op in range(len(self.ops)):
                self.launch_op(layer, op, stream, fused)

    def output(self, layer, op):
        rows = sum(self.ops[op][2])
        return self.out[layer][op].download(np.float32, rows)

    def activation(self, layer, op):
        _, qt, _, cols, _ = self.ops[op]
        return self.act[layer][op].download(np.uint8, mv.act_bytes(qt, cols))
