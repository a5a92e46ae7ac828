#!/usr/bin/env python3
"""Writes the golden vectors that only the compiled reference can pin (run in the build container, where
oracle/_ref/libqtip_ref.so exists; the GPU box only reads the committed outputs).

  ref_rng.json            first 64 next() / sign() / normal() of the splitmix stream for seeds 0 and 7
  ref_vit_raw_x.bin       64 tiles of raw (not fp16-representable) fp32 N(0,1), seed 1234 (first 64 of config 1)
  ref_vit_raw_hyb.bin     their states under the built-in HYB tlut            (u16 [64][128])
  ref_vit_raw_syn.bin     their states under the synthetic unit-rms tlut, seed 1 (u16 [64][128])
  ref_vit_raw_cost.bin    pass-2 path metrics returned by the reference (f64 [2][64]: hyb, syn)
  ref_config1.json        FNV-1a 64 of the packed words of all 4096 config-1 tiles (synthetic tlut)
  ref_config1_packed.bin  those packed words (u16 [4096][32], pack_trellis layout, not swizzled)
  ref_ldl_1024.bin        rows 1000..1007 of L (fp32) from block_ldl_to_L on a seeded n=1024 SPD matrix
  ref_ldl_2560_f32.bin    rows 255, 256, 257, 1279, 1280, 2558, 2559 of L (fp32) from block_ldl_to_L on a seeded
                          n=2560 SPD matrix rounded to fp32 first (the input type of ldl_hessian): ten 256-column
                          panels deep, so the rows carry the blocked code's order of operations
  ref_chol_528_rows.bin   rows 255, 256, 300, 511, 512, 527 of the fp64 Cholesky factor (cholesky_inplace) of a seeded
                          n=528 SPD matrix: every bit of the factor, not only what survives the rounding to fp32
                          (`python make_ref_vectors.py ldl` writes the three LDL files only)
  ref_ldlq_L.bin          a block-LDL factor (f32 [256][256]) and
  ref_ldlq_Q.bin          the states (u16 [64][128]) ldlq_ref of the reference's GPU test program (CPU code,
                          tests/test_gpu.cpp:180-225, compiled into oracle/_ref/libqtip_ref_gpu.so) returns for it and
                          the seeded 64 x 256 Wr of ref_ldlq.json, which also holds the FNV-1a 64 of the returned hatWr
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import binding as ob  # noqa: E402


def fnv1a64(buf):
    h = 0xcbf29ce484222325
    for b in bytes(buf):
        h = ((h ^ b) * 0x100000001b3) & 0xffffffffffffffff
    return h


def ref_quantize(R, X):
    st = np.zeros((X.shape[0], 128), np.uint16)
    cost = np.zeros(X.shape[0])
    hat = np.zeros(256, np.float32)
    for b in range(X.shape[0]):
        cost[b] = R.ref_quantize_seq(X[b], st[b], hat)
    return st, cost


def ldl_case(n=1024, seed=3):
    g = ob.rng_normal(seed, n * 64).reshape(n, 64)
    H = g @ g.T / 64 + 0.05 * np.eye(n)
    return H


LDL_2560_ROWS = (255, 256, 257, 1279, 1280, 2558, 2559)
CHOL_528_ROWS = (255, 256, 300, 511, 512, 527)


def ldl_vectors(R):
    H = ldl_case()
    A = H.copy()
    L = np.zeros((1024, 1024), np.float32)
    assert R.ref_block_ldl(A.reshape(-1), 1024, L.reshape(-1), 8) == 1
    L[1000:1008].tofile(os.path.join(HERE, "ref_ldl_1024.bin"))
    n = 2560
    H32 = ldl_case(n, 5).astype(np.float32)
    A = np.tril(0.5 * (H32.astype(np.float64) + H32.astype(np.float64).T))
    L = np.zeros((n, n), np.float32)
    assert R.ref_block_ldl(A.reshape(-1), n, L.reshape(-1), 8) == 1
    L[list(LDL_2560_ROWS)].tofile(os.path.join(HERE, "ref_ldl_2560_f32.bin"))
    n = 528
    A = np.tril(ldl_case(n, 6))
    assert R.ref_cholesky(A.reshape(-1), n, 4) == 1
    np.tril(A)[list(CHOL_528_ROWS)].tofile(os.path.join(HERE, "ref_chol_528_rows.bin"))


def main():
    R = ob.ref_lib()
    assert R is not None, "build oracle/_ref first (make -C oracle ref)"
    if sys.argv[1:] == ["ldl"]:
        ldl_vectors(R)
        return
    out = {}
    for seed in (0, 7):
        u = np.zeros(64, np.uint64)
        f = np.zeros(64)
        g = np.zeros(64)
        R.ref_rng(seed, 0, 64, None, u.ctypes.data)
        R.ref_rng(seed, 3, 64, f.ctypes.data, None)
        R.ref_rng(seed, 2, 64, g.ctypes.data, None)
        out[str(seed)] = {"next": [int(v) for v in u], "sign": [int(v) for v in f], "normal": [float.hex(float(v)) for v in g]}
    json.dump(out, open(os.path.join(HERE, "ref_rng.json"), "w"))

    X = ob.rng_normal(1234, 4096 * 256).astype(np.float32).reshape(4096, 256)
    X[:64].tofile(os.path.join(HERE, "ref_vit_raw_x.bin"))
    hyb = ob.Codebook()
    syn = ob.Codebook(ob.synthetic_tlut(1))
    st_h, c_h = ref_quantize(R, X[:64])
    R.ref_override_codebook(syn.lut0, syn.lut1, syn.lut_h2, syn.lut_rms)
    st_s, c_s = ref_quantize(R, X[:64])
    st_h.tofile(os.path.join(HERE, "ref_vit_raw_hyb.bin"))
    st_s.tofile(os.path.join(HERE, "ref_vit_raw_syn.bin"))
    np.stack([c_h, c_s]).tofile(os.path.join(HERE, "ref_vit_raw_cost.bin"))

    # all of config 1 under the synthetic tlut, the reference's code on 8 threads through a process pool-free loop
    import concurrent.futures as cf
    def chunk(lo):
        return ref_quantize(R, X[lo:lo + 128])[0]
    with cf.ThreadPoolExecutor(8) as ex:   # ctypes releases the GIL
        parts = list(ex.map(chunk, range(0, 4096, 128)))
    st_all = np.concatenate(parts)
    packed = np.zeros((4096, 32), np.uint16)
    R.ref_pack_trellis(st_all.reshape(-1), 4096, packed.reshape(-1))
    packed.tofile(os.path.join(HERE, "ref_config1_packed.bin"))
    json.dump({"tiles": 4096, "x_seed": 1234, "tlut_seed": 1, "fnv1a64_packed": "%016x" % fnv1a64(packed.tobytes()),
               "fnv1a64_states": "%016x" % fnv1a64(st_all.tobytes())},
              open(os.path.join(HERE, "ref_config1.json"), "w"))

    ldl_vectors(R)
    # LDLQ with 128-column buffers: the reference's own CPU restatement of ldlq.LDLQ, two buffers, four tile rows
    if ob.ref_gpu_lib() is not None:
        m, n = 64, 256
        Wr = ob.rng_normal(31, m * n).astype(np.float32).reshape(m, n)
        g = ob.rng_normal(32, n * 2 * n).reshape(n, 2 * n) * (1.0 + (np.arange(2 * n) % 7))
        Lq = ob.block_ldl(g @ g.T / (2 * n) + 0.05 * np.eye(n))
        hat, Q = ob.ref_ldlq(Wr, Lq)
        Lq.tofile(os.path.join(HERE, "ref_ldlq_L.bin"))
        Q.tofile(os.path.join(HERE, "ref_ldlq_Q.bin"))
        json.dump({"m": m, "n": n, "w_seed": 31, "fnv1a64_hat": "%016x" % fnv1a64(hat.tobytes())},
                  open(os.path.join(HERE, "ref_ldlq.json"), "w"))
    # NVFP4: the reference's plain quantizer (src/nvfp4.cpp) on gaussian and heavy-tailed weights (the two cases of
    # tests/test_nvfp4.cpp:47-57, same shapes, this repo's generator), plus the E4M3 encoder on a sweep of values
    nv = {}
    for name, seed, heavy in (("gauss", 5, False), ("heavy", 11, True)):
        m, n = 96, 256
        w = ob.rng_normal(seed, m * n) * 0.02
        if heavy:
            w = w * np.exp(1.2 * ob.rng_normal(seed + 100, m * n))
        w = w.astype(np.float32).reshape(m, n)
        w[3, 16:32] = 0.0                      # an all-zero block
        packed = np.zeros((m, n // 2), np.uint8)
        scales = np.zeros((m, n // 16), np.uint8)
        g = R.ref_nvfp4_quantize(w.reshape(-1), m, n, packed.reshape(-1), scales.reshape(-1))
        dq = np.zeros((m, n), np.float32)
        R.ref_nvfp4_dequantize(packed.reshape(-1), scales.reshape(-1), g, m, n, dq.reshape(-1))
        np.concatenate([packed.reshape(-1), scales.reshape(-1)]).tofile(os.path.join(HERE, "ref_nvfp4_%s.bin" % name))
        nv[name] = {"m": m, "n": n, "seed": seed, "global": float.hex(float(g)),
                    "fnv1a64_dequant": "%016x" % fnv1a64(dq.tobytes()),
                    "mse": float.hex(R.ref_nvfp4_proxy_error(w.reshape(-1), dq.reshape(-1), m, n, None))}
    xs = np.concatenate([np.float32(2.0) ** np.arange(-12, 10, dtype=np.float32) * s for s in (1.0, 1.0625, 1.25, 1.4375, 1.9375)]
                        + [np.array([0.0, 448.0, 500.0, 1e-9, 0.015625, 0.0146484375], np.float32)]).astype(np.float32)
    nv["fp8_inputs"] = [float.hex(float(v)) for v in xs]
    nv["fp8_codes"] = [int(R.ref_f32_to_fp8e4m3(float(v))) for v in xs]
    json.dump(nv, open(os.path.join(HERE, "ref_nvfp4.json"), "w"))
    print("wrote golden vectors to", HERE)


if __name__ == "__main__":
    main()
