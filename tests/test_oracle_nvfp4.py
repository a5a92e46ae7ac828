"""Pins the oracle's NVFP4 restatement (no GPU): the plain quantizer and the E4M3 encoder against vectors written by
the reference's own src/nvfp4.cpp compiled in place (tests/golden/make_ref_vectors.py) and against that library
directly where it is present; the scale search and the calibrated rounding (a restatement of the reference's GPU
kernels, src/nvfp4_gpu.hip:66-228) against the bytes the reference's own device path returned on a gfx950 GPU
(tests/golden/make_ref_nvfp4_gpu_vectors.py) and the criteria of its test, tests/test_nvfp4.cpp:59-105."""
import json
import os

import numpy as np
import pytest

from conftest import GOLDEN


def _fnv1a64(b):
    h = 0xcbf29ce484222325
    for x in np.frombuffer(b, np.uint8).reshape(-1, 1 << 16 if len(b) % (1 << 16) == 0 else 1).reshape(-1):
        h = ((h ^ int(x)) * 0x100000001b3) & 0xffffffffffffffff
    return h


def _weights(oracle, name):
    meta = json.load(open(os.path.join(GOLDEN, "ref_nvfp4.json")))[name]
    m, n, seed = meta["m"], meta["n"], meta["seed"]
    w = oracle.rng_normal(seed, m * n) * 0.02
    if name == "heavy":
        w = w * np.exp(1.2 * oracle.rng_normal(seed + 100, m * n))
    w = w.astype(np.float32).reshape(m, n)
    w[3, 16:32] = 0.0
    return w, meta


def _hessian(oracle, n, seed, samples=600):
    """Correlated, unevenly scaled input channels (the construction of tests/test_nvfp4.cpp:25-45)."""
    g = oracle.rng_normal(seed, n + n * 8 + samples * n * 9)
    colscale = np.exp(0.8 * g[:n])
    mix = g[n:n + 8 * n].reshape(n, 8)
    rest = g[n + 8 * n:].reshape(samples, n, 9)
    X = (0.5 * rest[:, :, 0] + 0.4 * np.einsum("jk,sjk->sj", mix, rest[:, :, 1:])) * colscale[None, :]
    return (X.T @ X / samples).astype(np.float32)


def test_fp8_e4m3_encoder_golden(oracle):
    meta = json.load(open(os.path.join(GOLDEN, "ref_nvfp4.json")))
    xs = [float.fromhex(v) for v in meta["fp8_inputs"]]
    got = [int(oracle.lib().qo_f32_to_fp8e4m3(x)) for x in xs]
    assert got == meta["fp8_codes"]
    assert got[xs.index(448.0)] == 126 and got[xs.index(500.0)] == 126 and got[xs.index(0.0)] == 0
    for code in range(127):   # every finite code decodes to a value that encodes back to itself
        assert oracle.lib().qo_f32_to_fp8e4m3(oracle.lib().qo_fp8e4m3_to_f32(code)) == code
        assert oracle.lib().qo_f32_to_fp8e4m3(-oracle.lib().qo_fp8e4m3_to_f32(code)) == (code | 128)


@pytest.mark.parametrize("name", ["gauss", "heavy"])
def test_plain_quantizer_golden(oracle, name):
    w, meta = _weights(oracle, name)
    m, n = w.shape
    packed, scales, g = oracle.nvfp4_quantize(w)
    want = np.fromfile(os.path.join(GOLDEN, "ref_nvfp4_%s.bin" % name), np.uint8)
    assert np.array_equal(packed.reshape(-1), want[:m * n // 2])
    assert np.array_equal(scales.reshape(-1), want[m * n // 2:])
    assert g == float.fromhex(meta["global"])
    dq = oracle.nvfp4_dequantize(packed, scales, g, m, n)
    assert "%016x" % _fnv1a64(dq.tobytes()) == meta["fnv1a64_dequant"]
    # the sum over rows is an OpenMP reduction in the reference too: its last bits depend on the thread count
    assert abs(oracle.nvfp4_proxy_error(w, dq) / float.fromhex(meta["mse"]) - 1) < 1e-13
    assert np.all(packed[3, 8:16] & 0x77 == 0) and scales[3, 1] == 0      # the all-zero block
    assert np.all((scales & 0x7f) <= 126)


def test_plain_quantizer_against_compiled_reference(oracle):
    R = oracle.ref_lib()
    if R is None or not hasattr(R, "ref_nvfp4_quantize"):
        pytest.skip("oracle/_ref not built here")
    rng = np.random.default_rng(4)
    for m, n, scale in ((7, 16, 1.0), (33, 304, 1e-3), (64, 1024, 30.0)):
        w = (rng.standard_normal((m, n)) * scale * np.exp(rng.standard_normal((m, n)))).astype(np.float32)
        p0, s0, g0 = oracle.nvfp4_quantize(w)
        p1 = np.zeros_like(p0)
        s1 = np.zeros_like(s0)
        g1 = R.ref_nvfp4_quantize(w.reshape(-1), m, n, p1.reshape(-1), s1.reshape(-1))
        assert g0 == g1 and np.array_equal(p0, p1) and np.array_equal(s0, s1)
        d0 = oracle.nvfp4_dequantize(p0, s0, g0, m, n)
        d1 = np.zeros_like(d0)
        R.ref_nvfp4_dequantize(p1.reshape(-1), s1.reshape(-1), g1, m, n, d1.reshape(-1))
        assert np.array_equal(d0, d1)
        H = _hessian(oracle, n, 9, samples=40) if n <= 304 else None
        e0 = oracle.nvfp4_proxy_error(w, d0, H)
        e1 = R.ref_nvfp4_proxy_error(w.reshape(-1), d1.reshape(-1), m, n, None if H is None else H.ctypes.data)
        assert abs(e0 - e1) <= 1e-12 * abs(e1)


@pytest.mark.parametrize("name", ["gauss", "heavy"])
def test_block_loop_meets_the_reference_test_criteria(oracle, name):
    """tests/test_nvfp4.cpp:59-105 on the oracle's restatement of the GPU block loop."""
    w, _ = _weights(oracle, name)
    m, n = w.shape
    H = _hessian(oracle, n, 21)
    naive = oracle.nvfp4_quantize(w)
    g = naive[2]

    def dq(t):
        return oracle.nvfp4_dequantize(t[0], t[1], g, m, n)

    off = oracle.nvfp4_blocks(w, None, None, g, False, False)
    assert np.array_equal(off[0], naive[0]) and np.array_equal(off[1], naive[1])      # upgrades off == plain quantizer
    search_plain = oracle.nvfp4_blocks(w, None, None, g, False, True)
    L, D = oracle.nvfp4_prepare(H, 1e-2, True)
    _, dH = oracle.nvfp4_prepare(H, 1e-2, False)
    cal = oracle.nvfp4_blocks(w, L, D, g, True, True)
    cal_only = oracle.nvfp4_blocks(w, L, D, g, True, False)
    search_h = oracle.nvfp4_blocks(w, None, dH, g, False, True)
    mse_naive, mse_search = oracle.nvfp4_proxy_error(w, dq(naive)), oracle.nvfp4_proxy_error(w, dq(search_plain))
    p_naive, p_search = oracle.nvfp4_proxy_error(w, dq(naive), H), oracle.nvfp4_proxy_error(w, dq(search_h), H)
    p_cal, p_cal_only = oracle.nvfp4_proxy_error(w, dq(cal), H), oracle.nvfp4_proxy_error(w, dq(cal_only), H)
    assert mse_search <= mse_naive * (1 + 1e-9)
    assert p_search <= p_naive * 1.02
    assert p_cal < 0.9 * p_naive and p_cal_only <= p_naive
    for t in (cal, cal_only, search_h, search_plain):
        assert np.all((t[1] & 0x7f) <= 126) and np.all(np.isfinite(dq(t)))
    # the factor used for the feedback reproduces the regularised Hessian: L diag(D) L^T = sym(H) + creg I
    Lu = L.astype(np.float64) + np.eye(n)
    Hr = 0.5 * (H.astype(np.float64) + H.T) + 1e-2 * np.trace(H.astype(np.float64)) / n * np.eye(n)
    assert np.max(np.abs(Lu @ np.diag(D.astype(np.float64)) @ Lu.T - Hr)) < 1e-5 * np.max(np.abs(Hr))


def device_path_vectors(name):
    """(H, [(hessian given, search, calibrate, packed, scales)], global) of tests/golden/ref_nvfp4_gpu_*."""
    meta = json.load(open(os.path.join(GOLDEN, "ref_nvfp4_gpu.json")))
    H = np.fromfile(os.path.join(GOLDEN, "ref_nvfp4_gpu_H.bin"), np.float32).reshape(256, 256)
    blob = np.fromfile(os.path.join(GOLDEN, "ref_nvfp4_gpu_%s.bin" % name), np.uint8)
    per = 96 * 128 + 96 * 16
    cases = []
    for k, (h, s, c) in enumerate(meta["combos"]):
        b = blob[k * per:(k + 1) * per]
        cases.append((bool(h), bool(s), bool(c), b[:96 * 128].reshape(96, 128), b[96 * 128:].reshape(96, 16)))
    return H, cases, float.fromhex(meta["global"][name])


@pytest.mark.parametrize("name", ["gauss", "heavy"])
def test_block_loop_equals_the_reference_device_path(oracle, name):
    """Every byte nvfp4_quantize_group of the reference returned on the GPU, for all five option combinations."""
    w, _ = _weights(oracle, name)
    m, n = w.shape
    H, cases, g = device_path_vectors(name)
    assert g == oracle.nvfp4_quantize(w)[2]
    L, D = oracle.nvfp4_prepare(H, 1e-2, True)
    _, dH = oracle.nvfp4_prepare(H, 1e-2, False)
    for (h, s, c, pk, sc) in cases:
        cal = h and c
        got = oracle.nvfp4_blocks(w, L if cal else None, (D if cal else dH) if h else None, g, cal, s)
        assert np.array_equal(got[0], pk) and np.array_equal(got[1], sc), (h, s, c)
    assert np.allclose(H, _hessian(oracle, n, 21), rtol=1e-5, atol=1e-7)      # the stored Hessian is the seeded one
