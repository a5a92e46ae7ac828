#!/usr/bin/env python3
"""Writes golden vectors of the fp32 Hadamard transform as the reference's device kernels compute it
(k_hadamard_rows, src/kernels.hip:293-313): run on a machine with a gfx950 GPU and
oracle/_ref/libqtip_ref_gpu.so (those kernels compiled in place by oracle/Makefile).

  ref_hadamard_gpu.json   the cases: [n, rows, transpose, seed]; the input of a case is rng_normal(seed, rows * n) as
                          fp32, rows of length n without padding
  ref_hadamard_gpu.bin    the transformed rows of every case, fp32, in the order of the json

usage: make_ref_hadamard_gpu_vectors.py [output directory, default: this directory]
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from oracle import binding as ob  # noqa: E402

CASES = [[n, rows, tr, 4000 + n] for n, rows in ((12, 3), (80, 3), (96, 3), (448, 2), (864, 2), (1024, 2), (2304, 2),
                                                (8192, 1), (12288, 1), (28672, 1)) for tr in (0, 1)]


def main():
    out = sys.argv[1] if len(sys.argv) > 1 else HERE
    os.makedirs(out, exist_ok=True)
    assert ob.ref_gpu_lib() is not None, "build oracle/_ref first (make -C oracle ref)"
    blob = b""
    for n, rows, tr, seed in CASES:
        x = ob.rng_normal(seed, rows * n).astype(np.float32).reshape(rows, n)
        blob += ob.ref_gpu_hadamard_rows(x, n, tr).tobytes()
    open(os.path.join(out, "ref_hadamard_gpu.bin"), "wb").write(blob)
    json.dump({"cases": CASES}, open(os.path.join(out, "ref_hadamard_gpu.json"), "w"))
    print("wrote %d bytes of device Hadamard vectors to %s" % (len(blob), out))


if __name__ == "__main__":
    main()
