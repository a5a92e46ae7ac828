"""Host part of the NVFP4 fallback quantizer through the C ABI (no GPU): E4M3 encoder, plain quantizer, dequantizer and
the Hessian preparation, against the golden vectors written by the reference's compiled src/nvfp4.cpp and the oracle."""
import json
import os

import numpy as np
import pytest

from conftest import GOLDEN
from test_oracle_nvfp4 import _hessian, _weights


def test_fp8_encoder_through_the_abi(pkg, oracle):
    meta = json.load(open(os.path.join(GOLDEN, "ref_nvfp4.json")))
    xs = [float.fromhex(v) for v in meta["fp8_inputs"]]
    assert [pkg.f32_to_fp8e4m3(x) for x in xs] == meta["fp8_codes"]
    assert pkg.f32_to_fp8e4m3(float("nan")) & 127 == 127 and pkg.f32_to_fp8e4m3(-0.5) == oracle.lib().qo_f32_to_fp8e4m3(-0.5)


@pytest.mark.parametrize("name", ["gauss", "heavy"])
def test_plain_quantizer_and_dequantizer(pkg, oracle, name):
    w, meta = _weights(oracle, name)
    m, n = w.shape
    t = pkg.nvfp4_quantize(w)
    want = np.fromfile(os.path.join(GOLDEN, "ref_nvfp4_%s.bin" % name), np.uint8)
    assert np.array_equal(t.packed.reshape(-1), want[:m * n // 2]) and np.array_equal(t.scales.reshape(-1), want[m * n // 2:])
    assert t.global_scale == float.fromhex(meta["global"])
    dq = pkg.nvfp4_dequantize(t)
    assert np.array_equal(dq, oracle.nvfp4_dequantize(t.packed, t.scales, t.global_scale, m, n))
    # proxy error: the golden mean squared error of the reference's own code, and a Hessian-weighted case
    assert abs(pkg.nvfp4_proxy_error(w, dq) / float.fromhex(meta["mse"]) - 1) < 1e-13
    H = _hessian(oracle, n, 9, samples=40)
    assert abs(pkg.nvfp4_proxy_error(w, dq, H) / oracle.nvfp4_proxy_error(w, dq, H) - 1) < 1e-12


def test_errors(pkg):
    with pytest.raises(pkg.QtipError):
        pkg.nvfp4_quantize(np.zeros((4, 24), np.float32))                 # n % 16
    bad = np.zeros((2, 16), np.float32)
    bad[1, 3] = np.inf
    with pytest.raises(pkg.QtipError):
        pkg.nvfp4_quantize(bad)                                           # nonfinite input
    t = pkg.nvfp4_quantize(np.ones((2, 16), np.float32))
    t.scales[0, 0] = 0x7f                                                 # NaN scale code
    with pytest.raises(pkg.QtipError):
        pkg.nvfp4_dequantize(t)
    z = pkg.nvfp4_quantize(np.zeros((2, 32), np.float32))                 # all zero: global 1, everything decodes to 0
    assert z.global_scale == 1.0 and not z.packed.any() and not pkg.nvfp4_dequantize(z).any()


def test_prepare_matches_oracle(pkg, oracle):
    n = 256
    H = _hessian(oracle, n, 21)
    L, D = pkg.nvfp4_prepare(H, 1e-2, True, threads=4)
    Lo, Do = oracle.nvfp4_prepare(H, 1e-2, True)
    # same factor up to the summation order of two fp64 Cholesky codes, rounded to fp32
    assert np.max(np.abs(L - Lo)) <= 4e-7 * np.max(np.abs(Lo)) and np.max(np.abs(D - Do) / Do) < 1e-6
    assert np.all(np.triu(L) == 0)
    _, dh = pkg.nvfp4_prepare(H, 1e-2, False)
    _, dho = oracle.nvfp4_prepare(H, 1e-2, False)
    assert np.array_equal(dh, dho)
    G = np.random.default_rng(0).standard_normal((n, 8)).astype(np.float32)
    with pytest.raises(pkg.QtipError) as e:
        pkg.nvfp4_prepare(G @ G.T, 0.0, True)
    assert e.value.code == pkg.QTIP_E_NOT_PD
