"""Numpy statement of the exact rewrite of Q3_K blocks as Q6_K blocks, element by
element from the two layouts (no bit tricks), used to check the device kernel.

Q3_K (oxidize-c/src/compute/oxk.c:624-652): 32 bytes of third bits, 64 bytes of
2-bit codes, sixteen 6-bit scales in 12 bytes (oxk.c:556-573), f16 d.  Element
e = 128n + 32k + l has code bits 2k of qs[32n + l] plus 4 when bit 4n + k of
hmask[l] is set, weight d * (sc[e // 16] - 32) * (code - 4).
Q6_K (oxk.c:913-964): 128 bytes of low nibbles, 64 bytes of upper bit pairs,
sixteen int8 scales, f16 d; weight d * sc[e // 16] * (code6 - 32).
code6 = code + 28 and sc6 = sc - 32 make the two weights the same.
"""
import numpy as np


def q3k_scales(sc12):
    """(n, 12) packed bytes -> (n, 16) values 0..63"""
    a = sc12.astype(np.int32)
    out = np.zeros((a.shape[0], 16), np.int32)
    for j in range(16):
        low = (a[:, j] & 15) if j < 8 else (a[:, j - 8] >> 4)
        out[:, j] = low | (((a[:, 8 + j % 4] >> (2 * (j // 4))) & 3) << 4)
    return out


def q3k_codes(blk):
    """(n, 110) Q3_K blocks -> (n, 256) codes 0..7 in element order"""
    hm, qs = blk[:, :32].astype(np.int32), blk[:, 32:96].astype(np.int32)
    out = np.zeros((blk.shape[0], 256), np.int32)
    for n in range(2):
        for k in range(4):
            for l in range(32):
                out[:, 128 * n + 32 * k + l] = ((qs[:, 32 * n + l] >> (2 * k)) & 3) + \
                    4 * ((hm[:, l] >> (4 * n + k)) & 1)
    return out


def q3k_as_q6k(w):
    """flat uint8 array of Q3_K blocks -> flat uint8 array of Q6_K blocks"""
    blk = np.ascontiguousarray(w, dtype=np.uint8).reshape(-1, 110)
    c6 = q3k_codes(blk) + 28
    out = np.zeros((blk.shape[0], 210), np.uint8)
    for n in range(2):
        for l in range(32):
            e = [128 * n + 32 * k + l for k in range(4)]
            out[:, 64 * n + l] = (c6[:, e[0]] & 15) | ((c6[:, e[2]] & 15) << 4)
            out[:, 64 * n + 32 + l] = (c6[:, e[1]] & 15) | ((c6[:, e[3]] & 15) << 4)
            out[:, 128 + 32 * n + l] = sum((c6[:, e[k]] >> 4) << (2 * k) for k in range(4))
    out[:, 192:208] = (q3k_scales(blk[:, 96:108]) - 32).astype(np.int8).view(np.uint8)
    out[:, 208:210] = blk[:, 108:110]
    return out.reshape(-1)


def q2k_widen(w):
    """flat uint8 array of Q2_K blocks (oxk.c:592-622: 16 scale|min bytes, 64 bytes of 2-bit codes in
    the element order above, f16 d, f16 dmin) -> the 210-byte blocks of the tile kernel's Q2 mode:
    scale * code in the 6-bit fields of the Q6_K layout, minima as nibbles in bytes 192..199, dmin in
    200..201, zeros to 207, d in 208..209"""
    blk = np.ascontiguousarray(w, dtype=np.uint8).reshape(-1, 84)
    sm, qs = blk[:, :16].astype(np.int32), blk[:, 16:80].astype(np.int32)
    c6 = np.zeros((blk.shape[0], 256), np.int32)
    for n in range(2):
        for k in range(4):
            for l in range(32):
                e = 128 * n + 32 * k + l
                c6[:, e] = ((qs[:, 32 * n + l] >> (2 * k)) & 3) * (sm[:, e // 16] & 15)
    out = np.zeros((blk.shape[0], 210), np.uint8)
    for n in range(2):
        for l in range(32):
            e = [128 * n + 32 * k + l for k in range(4)]
            out[:, 64 * n + l] = (c6[:, e[0]] & 15) | ((c6[:, e[2]] & 15) << 4)
            out[:, 64 * n + 32 + l] = (c6[:, e[1]] & 15) | ((c6[:, e[3]] & 15) << 4)
            out[:, 128 + 32 * n + l] = sum((c6[:, e[k]] >> 4) << (2 * k) for k in range(4))
    for g in range(0, 16, 2):
        out[:, 192 + g // 2] = (sm[:, g] >> 4) | ((sm[:, g + 1] >> 4) << 4)
    out[:, 200:202] = blk[:, 82:84]
    out[:, 208:210] = blk[:, 80:82]
    return out.reshape(-1)
