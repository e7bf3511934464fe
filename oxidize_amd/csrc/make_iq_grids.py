#!/usr/bin/env python3
"""Writes iq_grids.inc: the two codebooks the IQ3_S and IQ1_XXXS kernels (and the oracle) look codes up
in.  They are constant data of the formats themselves (ggml's iq3s_grid and iq1s_grid; the reference
keeps its copies in oxidize-c/src/compute/quant_tables.h:23, :381 and the IQ1_XXXS index table in
oxidize-c/src/compute/quantization.c:891), read here from a reference checkout and written out as
numbers only:

    OXH_IQ3S_GRID[512]      uint32: four magnitudes (one per byte) per 9-bit code
    OXH_IQ1XXXS_GRID[256]   uint64: eight values in {-1, 0, +1} (one int8 per byte) per 8-bit code,
                            i.e. iq1s_grid composed with the IQ1_XXXS index table

    python oxidize_amd/csrc/make_iq_grids.py /root/reference > oxidize_amd/csrc/iq_grids.inc
"""
import re
import sys


def table(text, name):
    m = re.search(r"%s\[\d+\]\s*=\s*\{(.*?)\};" % re.escape(name), text, re.S)
    body = re.sub(r"/\*.*?\*/", "", m.group(1), flags=re.S)
    return [int(t.rstrip("uUlL"), 0) for t in re.findall(r"0[xX][0-9a-fA-F]+[uUlL]*|\d+[uUlL]*", body)]


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    tables = open(root + "/oxidize-c/src/compute/quant_tables.h").read()
    quant = open(root + "/oxidize-c/src/compute/quantization.c").read()
    iq3s = table(tables, "IQ3S_GRID")
    iq1s = table(tables, "IQ1S_GRID")
    index = table(quant, "IQ1_XXXS_TO_IQ1S")
    assert len(iq3s) == 512 and len(iq1s) == 2048 and len(index) == 256
    iq1x = [iq1s[i] for i in index]
    for v in iq1x:
        assert all(((v >> (8 * j)) & 0xFF) in (0x00, 0x01, 0xFF) for j in range(8))
    out = ["/* iq_grids.inc -- codebooks of the IQ3_S and IQ1_XXXS formats; data only.  Written by",
           " * make_iq_grids.py (see there for where the numbers come from); do not edit.",
           " * OXH_IQ_TABLE_ATTR: what a device translation unit puts in front (__device__); empty otherwise. */",
           "#ifndef OXH_IQ_TABLE_ATTR",
           "#define OXH_IQ_TABLE_ATTR",
           "#endif",
           "OXH_IQ_TABLE_ATTR static const uint32_t OXH_IQ3S_GRID[512] = {"]
    for i in range(0, 512, 8):
        out.append("    " + ", ".join("0x%08xu" % v for v in iq3s[i:i + 8]) + ",")
    out.append("};")
    out.append("OXH_IQ_TABLE_ATTR static const uint64_t OXH_IQ1XXXS_GRID[256] = {")
    for i in range(0, 256, 4):
        out.append("    " + ", ".join("0x%016xull" % v for v in iq1x[i:i + 4]) + ",")
    out.append("};")
    print("\n".join(out))


if __name__ == "__main__":
    main()
