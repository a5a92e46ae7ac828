#!/usr/bin/env python3
"""Writes the golden vectors of the NVFP4 block loop, which only the reference's device path can pin: run on a machine
with a gfx950 GPU and oracle/_ref/libqtip_ref_gpu.so (the reference's src/nvfp4_gpu.hip compiled in place by
oracle/Makefile).  Inputs are the two 96 x 256 weight matrices of ref_nvfp4.json and one 256 x 256 Hessian.

  ref_nvfp4_gpu_H.bin        the Hessian (f32 [256][256]); stored because a BLAS product is not reproducible to the bit
  ref_nvfp4_gpu_<name>.bin   for each option combination of ref_nvfp4_gpu.json, in order: packed (u8 [96][128]) then
                             scales (u8 [96][16]) returned by nvfp4_quantize_group
  ref_nvfp4_gpu.json         the combinations: [hessian given, scale_search, calibrate], and the global scales

usage: make_ref_nvfp4_gpu_vectors.py [output directory, default: this directory]
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
from oracle import binding as ob  # noqa: E402
from test_oracle_nvfp4 import _hessian, _weights  # noqa: E402

COMBOS = [[0, 0, 0], [0, 1, 1], [1, 1, 0], [1, 0, 1], [1, 1, 1]]


def main():
    out = sys.argv[1] if len(sys.argv) > 1 else HERE
    os.makedirs(out, exist_ok=True)
    assert ob.ref_gpu_lib() is not None, "build oracle/_ref first (make -C oracle ref)"
    H = _hessian(ob, 256, 21)
    H.tofile(os.path.join(out, "ref_nvfp4_gpu_H.bin"))
    meta = {"combos": COMBOS, "global": {}}
    for name in ("gauss", "heavy"):
        w, _ = _weights(ob, name)
        blob = b""
        for (h, s, c) in COMBOS:
            ((pk, sc, g),), used = ob.ref_gpu_nvfp4_quantize_group([w], 256, H if h else None, scale_search=bool(s), calibrate=bool(c))
            assert used == bool(h and c)
            blob += pk.tobytes() + sc.tobytes()
            meta["global"][name] = float.hex(g)
        open(os.path.join(out, "ref_nvfp4_gpu_%s.bin" % name), "wb").write(blob)
    json.dump(meta, open(os.path.join(out, "ref_nvfp4_gpu.json"), "w"))
    print("wrote NVFP4 device-path vectors to", out)


if __name__ == "__main__":
    main()
