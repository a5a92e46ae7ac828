"""Pins oracle/ against the reference's own CPU core compiled in place (oracle/_ref, built only where
/root/reference exists) and against the vectors that build wrote into tests/golden.  No GPU."""
import json
import os

import numpy as np
import pytest

from conftest import GOLDEN


def g(name, dt):
    return np.fromfile(os.path.join(GOLDEN, name), dtype=dt)


# ------------------------------------------------------------------ committed vectors (run everywhere)
def test_rng_golden(oracle):
    want = json.load(open(os.path.join(GOLDEN, "ref_rng.json")))
    for seed in (0, 7):
        w = want[str(seed)]
        assert [int(v) for v in oracle.rng_next(seed, 64)] == w["next"]
        assert [int(v) for v in oracle.rng_sign(seed, 64)] == w["sign"]
        assert [float.hex(float(v)) for v in oracle.rng_normal(seed, 64)] == w["normal"]


def test_viterbi_raw_inputs_golden(oracle, hyb, syn):
    X = g("ref_vit_raw_x.bin", np.float32).reshape(64, 256)
    assert np.array_equal(X, oracle.rng_normal(1234, 64 * 256).astype(np.float32).reshape(64, 256))
    assert not np.array_equal(X, X.astype(np.float16).astype(np.float32))   # inputs are NOT fp16-representable
    cost = g("ref_vit_raw_cost.bin", np.float64).reshape(2, 64)
    for k, (cb, name) in enumerate(((hyb, "ref_vit_raw_hyb.bin"), (syn, "ref_vit_raw_syn.bin"))):
        want = g(name, np.uint16).reshape(64, 128)
        for fast in (True, False):
            got = oracle.quantize_tiles(cb, X, fast=fast)
            assert np.array_equal(got, want)
        st = np.zeros(128, np.uint16)
        hat = np.zeros(256, np.float32)
        for b in range(0, 64, 7):   # returned path metric, bit for bit
            c = oracle.lib().qo_quantize_seq(cb.lut0, cb.lut1, X[b], st, hat)
            assert c == cost[k, b]


def test_ldl_1024_golden(oracle):
    n = 1024
    gm = oracle.rng_normal(3, n * 64).reshape(n, 64)
    H = gm @ gm.T / 64 + 0.05 * np.eye(n)
    L = oracle.block_ldl(H)
    want = g("ref_ldl_1024.bin", np.float32).reshape(8, n)
    got = L[1000:1008]
    # same order of operations as the blocked reference: the same bits
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_cholesky_528_fp64_golden(oracle):
    """Every bit of the fp64 factor (two 256-column panels and a ragged third): rows written by the compiled
    reference's cholesky_inplace."""
    n = 528
    gm = oracle.rng_normal(6, n * 64).reshape(n, 64)
    A = np.tril(gm @ gm.T / 64 + 0.05 * np.eye(n))
    assert oracle.lib().qo_cholesky(A.reshape(-1), n) == 1
    rows = [255, 256, 300, 511, 512, 527]
    want = g("ref_chol_528_rows.bin", np.uint64).reshape(len(rows), n)
    assert np.array_equal(np.tril(A)[rows].view(np.uint64), want)


def test_ldl_2560_f32_golden(oracle):
    n = 2560
    gm = oracle.rng_normal(5, n * 64).reshape(n, 64)
    H32 = (gm @ gm.T / 64 + 0.05 * np.eye(n)).astype(np.float32)
    rows = [255, 256, 257, 1279, 1280, 2558, 2559]
    want = g("ref_ldl_2560_f32.bin", np.uint32).reshape(len(rows), n)
    L = np.zeros((n, n), np.float32)
    assert oracle.lib().qo_ldl_hessian(H32.reshape(-1), n, L.reshape(-1)) == 0
    assert np.array_equal(L[rows].view(np.uint32), want)


# ------------------------------------------------------------------ live comparison (build container only)
@pytest.fixture(scope="module")
def ref(oracle):
    R = oracle.ref_lib()
    if R is None:
        pytest.skip("oracle/_ref not built (the reference tree is absent here)")
    return R


def test_ref_codebook_perm_formats(oracle, ref, hyb):
    l0 = np.zeros(65536, np.float32)
    l1 = np.zeros(65536, np.float32)
    h2 = np.zeros(65536, np.uint32)
    import ctypes
    rms = ctypes.c_double()
    tl = np.zeros(1024, np.float32)
    ref.ref_codebook(l0.ctypes.data, l1.ctypes.data, h2.ctypes.data, ctypes.addressof(rms), tl.ctypes.data)
    assert np.array_equal(l0, hyb.lut0) and np.array_equal(l1, hyb.lut1) and np.array_equal(h2, hyb.lut_h2)
    assert rms.value == hyb.lut_rms
    assert np.array_equal(tl, hyb.tlut.reshape(-1))
    p = np.zeros(256, np.int32)
    q = np.zeros(256, np.int32)
    ref.ref_perm256(p, q)
    op, oq = oracle.perm256()
    assert np.array_equal(p, op) and np.array_equal(q, oq)
    rng = np.random.default_rng(0)
    vals = np.concatenate([rng.normal(size=3000), rng.normal(size=1000) * 1e-6, rng.normal(size=300) * 1e5]).astype(np.float32)
    L = oracle.lib()
    for v in vals:
        assert L.qo_f32_to_fp16(float(v)) == ref.ref_f32_to_fp16(float(v))
        assert L.qo_f32_to_bf16(float(v)) == ref.ref_f32_to_bf16(float(v))
    for n in (96, 1024, 3000, 12288, 28672, 57344, 2304, 100, 640):
        assert L.qo_had_K(n) == ref.ref_had_K(n)


def test_ref_viterbi_live(oracle, ref, hyb):
    # single passes with and without the constraint, returned metrics bit for bit, raw fp32 inputs
    X = oracle.rng_normal(77, 6 * 256).astype(np.float32).reshape(6, 256) * np.float32(1.3)
    L = oracle.lib()
    for b in range(6):
        for ov in (-1, 17, 4000):
            s1 = np.zeros(128, np.uint16)
            s2 = np.zeros(128, np.uint16)
            c1 = ref.ref_viterbi(X[b], ov, s1)
            c2 = L.qo_viterbi(hyb.lut0, hyb.lut1, X[b], ov, s2)
            assert c1 == c2 and np.array_equal(s1, s2)
            assert ref.ref_path_cost(X[b], s1) == L.qo_path_cost(hyb.lut0, hyb.lut1, X[b], s2)


def test_ref_hadamard_pack_ldl_live(oracle, ref):
    rng = np.random.default_rng(1)
    L = oracle.lib()
    for n in (96, 1024, 12288):
        x = rng.normal(size=(2, n + 8))
        for t in (0, 1):
            a = x.reshape(-1).copy()
            b = x.reshape(-1).copy()
            ref.ref_hadamard_rows(a, 2, n, n + 8, t)
            L.qo_hadamard_rows(b, 2, n, n + 8, t)
            assert np.array_equal(a, b)
    st = rng.integers(0, 65536, (24, 128)).astype(np.uint16)
    a = np.zeros(24 * 32, np.uint16)
    ref.ref_pack_trellis(st.reshape(-1), 24, a)
    assert np.array_equal(a, oracle.pack_trellis(st).reshape(-1))
    sw = np.zeros_like(a)
    ref.ref_swizzle(a, 64, 96, sw)
    assert np.array_equal(sw, oracle.swizzle(a, 64, 96))
    un = np.zeros((24, 128), np.uint16)
    ref.ref_unpack_trellis(a, 24, un.reshape(-1))
    assert np.array_equal(un, oracle.unpack_trellis(a))
    for n in (272, 1024, 1296):
        G = rng.normal(size=(n, n + 128))
        if n == 1296:        # correlated channels and a few of large scale: the fp32 rounding of L hides less here
            G[:, 1:] += 0.8 * G[:, :-1]
            G[rng.choice(n, 16, replace=False)] *= 20
        H = G @ G.T / (n + 128) + 0.02 * np.eye(n)
        C1, C2 = np.tril(H), np.tril(H)
        assert ref.ref_cholesky(C1.reshape(-1), n, 4) == 1 and L.qo_cholesky(C2.reshape(-1), n) == 1
        assert np.array_equal(np.tril(C1).view(np.uint64), np.tril(C2).view(np.uint64)), "fp64 Cholesky factors differ"
        A = H.copy()
        Lr = np.zeros((n, n), np.float32)
        assert ref.ref_block_ldl(A.reshape(-1), n, Lr.reshape(-1), 4) == 1
        Lo = oracle.block_ldl(H)
        assert np.array_equal(Lr.view(np.uint32), Lo.view(np.uint32))
