#!/usr/bin/env python3
"""Provenance script for qtip_tables.h (run once, in the build container).

Reads the +-1 Hadamard factor matrices and the default HYB tlut that the
reference carries as data (src/qtip_constants.hpp) and re-encodes them in this
library's own compact form: each Hadamard row is bit-packed (bit k of the row
word array set <=> entry +1), the tlut is kept as fp32 bit patterns.

It sits beside the other provenance scripts of committed data (the make_ref_* scripts of this folder); the header it
writes lives with the library, behemoth-qtip_amd/csrc/data/qtip_tables.h.

usage: make_qtip_tables.py /root/reference/src/qtip_constants.hpp > behemoth-qtip_amd/csrc/data/qtip_tables.h
"""
import re
import sys


def main():
    src = open(sys.argv[1]).read()
    order = [int(v) for v in re.search(r"kHadOrder\[\d+\]\s*=\s*\{([^}]*)\}", src).group(1).split(",")]
    out = []
    out.append("/* Hadamard factor matrices (bit-packed rows, bit set = +1) and the default HYB tlut")
    out.append(" * (fp32 bit patterns, [512][2]).  Data only; written by tests/golden/make_qtip_tables.py. */")
    out.append("#ifndef QTIP_TABLES_H_")
    out.append("#define QTIP_TABLES_H_")
    out.append("#include <stdint.h>")
    out.append("#define QTIP_NUM_HAD %d" % len(order))
    out.append("/* in C++ the tables can be read in constant expressions */")
    out.append("#ifdef __cplusplus")
    out.append("#define QTIP_TABLE static constexpr")
    out.append("#else")
    out.append("#define QTIP_TABLE static const")
    out.append("#endif")
    out.append("QTIP_TABLE int qtip_had_order[QTIP_NUM_HAD] = {%s};" % ",".join(map(str, order)))
    for K in order:
        body = re.search(r"kHad%d\[\d+\]\s*=\s*\{([^}]*)\}" % K, src).group(1)
        vals = [int(v) for v in body.split(",")]
        assert len(vals) == K * K and all(v in (1, -1) for v in vals)
        wpr = (K + 31) // 32
        words = []
        for r in range(K):
            for w in range(wpr):
                x = 0
                for b in range(32):
                    k = w * 32 + b
                    if k < K and vals[r * K + k] > 0:
                        x |= 1 << b
                words.append("0x%08xu" % x)
        out.append("QTIP_TABLE uint32_t qtip_had%d_bits[%d] = {" % (K, len(words)))
        for i in range(0, len(words), 8):
            out.append("  " + ",".join(words[i:i + 8]) + ",")
        out.append("};")
    out.append("static inline const uint32_t* qtip_had_bits(int K) {")
    out.append("  switch (K) {")
    for K in order:
        out.append("    case %d: return qtip_had%d_bits;" % (K, K))
    out.append("    default: return 0;")
    out.append("  }")
    out.append("}")
    out.append("/* entry (r, k) of the K x K factor: +1 or -1 */")
    out.append("static inline int qtip_had_entry(const uint32_t* bits, int K, int r, int k) {")
    out.append("  int wpr = (K + 31) / 32;")
    out.append("  return ((bits[r * wpr + (k >> 5)] >> (k & 31)) & 1u) ? 1 : -1;")
    out.append("}")
    body = re.search(r"kTlutF32Bits\[1024\]\s*=\s*\{([^}]*)\}", src).group(1)
    vals = [v.strip() for v in body.split(",") if v.strip()]
    assert len(vals) == 1024
    out.append("QTIP_TABLE uint32_t qtip_hyb_tlut_bits[1024] = {")
    for i in range(0, 1024, 8):
        out.append("  " + ",".join(v + "u" for v in vals[i:i + 8]) + ",")
    out.append("};")
    out.append("#endif")
    print("\n".join(out))


if __name__ == "__main__":
    main()
