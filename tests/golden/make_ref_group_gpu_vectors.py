#!/usr/bin/env python3
"""Writes group-level golden vectors from the reference's own device path: run on a machine with a gfx950 GPU and
oracle/_ref/libqtip_ref_gpu.so (the reference's quantizer.cpp, viterbi.hip, kernels.hip, gemm.cpp compiled in place by
oracle/Makefile).  They pin what only the whole call shows: the seeds of SU / SV, the Wscale formula, the proxy
formulas and the order of the packed words per linear (src/quantizer.cpp:176-346).

Inputs come from group_case() below and are reproducible to the bit on any machine: the weights from the splitmix
stream, the Hessian as X^T X / 512 of small integers (every partial sum is exact in fp32, whatever the order).

  ref_group_gpu_<case>.bin  per linear, in order: trellis (u16, kernel layout), su_bf16 (u16 [n]), sv (i8 [m], +-1)
  ref_group_gpu.json        per case: shapes, seed, and per linear wscale (hex float), proxy, proxy_rot_reg

usage: make_ref_group_gpu_vectors.py [output directory, default: this directory]
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from oracle import binding as ob  # noqa: E402

CASES = {"a": dict(n=256, ms=(64, 32), seed=7), "b": dict(n=1024, ms=(128,), seed=9)}


def group_case(name):
    """(list of W, H, seed) of a case; integers make H exact."""
    c = CASES[name]
    n, rows = c["n"], 512
    e = np.rint(ob.rng_normal(100 + c["seed"], rows * (n + 2)).reshape(rows, n + 2) * 2.5).clip(-8, 8)
    x = e[:, 2:] + e[:, 1:-1] + e[:, :-2]                  # correlated neighbouring channels, |x| <= 24
    x[:, ::97] *= 4                                        # a few channels of large scale
    H = (x.T @ x / rows).astype(np.float32)                # sums of integer products below 2^24: exact
    Ws = [(ob.rng_normal(200 + c["seed"] + i, m * n).reshape(m, n) * s).astype(np.float32)
          for i, (m, s) in enumerate(zip(c["ms"], (0.02, 0.05)))]
    return Ws, H, c["seed"]


def main():
    out = sys.argv[1] if len(sys.argv) > 1 else HERE
    os.makedirs(out, exist_ok=True)
    assert ob.ref_gpu_lib() is not None, "build oracle/_ref first (make -C oracle ref)"
    meta = {}
    for name, c in CASES.items():
        Ws, H, seed = group_case(name)
        r = ob.ref_gpu_quantize_group(Ws, H, seed, ldl_threads=8)
        blob = b""
        for k in range(len(Ws)):
            sv = r["sv"][k]
            assert np.all(np.abs(sv) == 1)
            blob += r["trellis"][k].tobytes() + r["su_bf16"][k].tobytes() + sv.astype(np.int8).tobytes()
        open(os.path.join(out, "ref_group_gpu_%s.bin" % name), "wb").write(blob)
        meta[name] = dict(n=c["n"], ms=list(c["ms"]), seed=seed,
                          wscale=[float(v).hex() for v in r["wscale"]], proxy=[float(v) for v in r["proxy"]],
                          proxy_rot_reg=[float(v) for v in r["proxy_rot_reg"]])
    json.dump(meta, open(os.path.join(out, "ref_group_gpu.json"), "w"), indent=1)
    print("wrote group vectors of the reference's device path to", out)


if __name__ == "__main__":
    main()
