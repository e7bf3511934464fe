"""Weights and inputs at the formats' integer bounds, shared by the oracle's own
check against the compiled reference and by the GPU parity test."""
import numpy as np

from oxidize_amd import synth

# type id -> (layout id for the generator tables, offsets of the f16 fields)
TYPES = {13: (13, (0, 2)), 15: (15, (0, 2)), 16: (16, (208,)), 8: (8, (80, 82)), 10: (10, (108,)),
         7: (7, (0,)), 3: (3, (0,)), 4: (4, (0, 2)), 5: (5, (0,)), 6: (6, (0, 2)), 18: (18, (0,))}
F16 = (0x1400, 0x9400, 0x1800, 0x0400)          # 2^-10, -2^-10, 2^-9, 2^-14: finite results at any integer


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def extreme_weights(layout, fields, rows, cols):
    bsz, per = synth.BLOCK_BYTES[layout], synth.BLOCK_ELEMS[layout]
    nblk = rows * (cols // per)
    fills = np.array([0xFF, 0x00, 0x7F, 0x80, 0xF0, 0x0F, 0xAA, 0x55], np.uint8)
    blk = np.empty((nblk, bsz), np.uint8)
    blk[:] = fills[(np.arange(nblk) // 3) % fills.size][:, None]          # runs of three blocks per fill
    # a few blocks mix the fills bytewise, so that maxima sit next to minima inside a block
    mix = np.arange(nblk) % 5 == 4
    blk[mix] = fills[(np.arange(bsz)[None, :] + np.arange(nblk)[mix, None]) % fills.size]
    for i, off in enumerate(fields):
        v = np.array(F16, np.uint16)[(np.arange(nblk) + i) % len(F16)]
        blk[:, off] = v & 0xFF
        blk[:, off + 1] = v >> 8
    return blk.reshape(-1)


def extreme_inputs(n_vec, cols):
    x = np.empty((n_vec, cols), np.float32)
    e = np.arange(cols)
    pats = [np.full(cols, 3.0), np.full(cols, -3.0), np.where((e // 16) % 2 == 0, 3.0, -3.0),
            np.where(e % 2 == 0, 3.0, -3.0), np.where((e // 32) % 2 == 0, 3.0, -3.0),
            np.where(e % 7 == 0, -3.0, 3.0)]
    for v in range(n_vec):
        x[v] = pats[v % len(pats)]
    return x


def quantiser_edge_inputs(n):
    e = np.arange(n, dtype=np.float32)
    c = {}
    t = (e % 127) + 0.5
    t[0] = 127.0
    c["ties, positive"] = t.copy()                       # x / d lands on k + 0.5: round half to even
    c["ties, negative"] = -t
    t = ((e % 250) - 125) * 0.5
    t[1] = 127.0
    c["half steps"] = t.copy()
    c["near the largest float"] = np.where(e % 3 == 0, 3.0e38, -1.7e38).astype(np.float32)
    c["the largest float"] = np.full(n, np.finfo(np.float32).max, np.float32)
    c["negative zeros"] = np.full(n, -0.0, np.float32)
    c["subnormal scale"] = (np.float32(1.4e-36) * ((e % 5) - 2) / 2).astype(np.float32)      # d = 1.1e-38
    c["smallest normal scale"] = (np.float32(1.6e-36) * ((e % 5) - 2) / 2).astype(np.float32)
    c["smallest scale whose reciprocal is finite"] = (np.float32(3.8e-37) * ((e % 5) - 2) / 2).astype(np.float32)
    c["one value among zeros"] = np.where(e % 256 == 200, -5.0, 0.0).astype(np.float32)
    return c
