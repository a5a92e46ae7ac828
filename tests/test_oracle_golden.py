"""Pins oracle/ (the CPU restatement) against the golden vectors the reference's own CPU test holds
(tests/test_cpu.cpp:35-166, vectors under tests/refvec, copied as data into tests/golden/refvec) and,
where those leave something open, against what the mathematics fixes.  No GPU."""
import json
import os

import numpy as np
import pytest

from conftest import GOLDEN, REFVEC


def load(name, dt):
    return np.fromfile(os.path.join(REFVEC, name), dtype=dt)


def test_manifest():
    man = json.load(open(os.path.join(REFVEC, "manifest.json")))
    assert man == {"nvit": 24, "pack_m": 64, "pack_n": 96, "ldl_n": 96}


# ------------------------------------------------------------------ number formats
def test_fp16_bf16_against_numpy(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.normal(size=4000).astype(np.float32),
        (rng.normal(size=2000) * 1e-6).astype(np.float32),      # fp16 subnormal range
        (rng.normal(size=500) * 1e5).astype(np.float32),        # overflow range
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 6e-8, 2.98e-8, 2.99e-8, np.inf, -np.inf], np.float32),
        np.arange(1, 2049, dtype=np.float32) * np.float32(2.0 ** -25),   # halfway cases of subnormals
        (1.0 + (np.arange(0, 4096) + 0.5) * 2.0 ** -11).astype(np.float32),  # ties in [1, 2)
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.qo_f32_to_fp16(float(v)) for v in vals], np.uint16)
    assert np.array_equal(got, want)
    allh = np.arange(65536, dtype=np.uint16)
    back = np.array([L.qo_fp16_to_f32(int(h)) for h in allh], np.float32)
    wantb = allh.view(np.float16).astype(np.float32)
    assert np.array_equal(back.view(np.uint32)[~np.isnan(wantb)], wantb.view(np.uint32)[~np.isnan(wantb)])
    # bf16 round-to-nearest-even: compare with integer arithmetic on the bit pattern
    u = vals[np.isfinite(vals)].view(np.uint32).astype(np.uint64)
    wantbf = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    gotbf = np.array([L.qo_f32_to_bf16(float(v)) for v in vals[np.isfinite(vals)]], np.uint16)
    assert np.array_equal(gotbf, wantbf)


# ------------------------------------------------------------------ codebook / permutation
def test_lut_golden(oracle, hyb):
    lut = load("lut.bin", np.float32)
    assert np.array_equal(lut[:65536], hyb.lut0) and np.array_equal(lut[65536:], hyb.lut1)
    assert abs(hyb.lut_rms - 0.968247639) < 5e-10
    # packed half2: low = component 0, high = component 1
    assert np.array_equal((hyb.lut_h2 & 0xffff).astype(np.uint16).view(np.float16).astype(np.float32), hyb.lut0)
    assert np.array_equal((hyb.lut_h2 >> 16).astype(np.uint16).view(np.float16).astype(np.float32), hyb.lut1)


def test_lut_closed_form(oracle, syn):
    # quantlut_sym written independently: entry e = flip << 9 | idx, sign fold on component 0
    s = np.arange(65536, dtype=np.uint64)
    p = s * (s + 1)
    idx = ((p >> 6) & 511).astype(np.int64)
    flip = ((p >> 15) & 1).astype(bool)
    th = syn.tlut.astype(np.float16).astype(np.float32)
    c0 = np.where(flip, -th[idx, 0], th[idx, 0])
    assert np.array_equal(c0, syn.lut0) and np.array_equal(th[idx, 1], syn.lut1)
    # only 1024 distinct entries, identified by bits 6..15 of s(s+1)
    code = ((p >> 6) & 1023).astype(np.int64)
    for arr in (syn.lut0, syn.lut1):
        first = np.full(1024, np.nan, np.float32)
        first[code[::-1]] = arr[::-1]
        assert np.array_equal(first[code], arr)


def test_perm_golden(oracle):
    perm, inv = oracle.perm256()
    assert np.array_equal(load("perm.bin", np.int64), perm)
    closed = np.arange(256).reshape(2, 8, 2, 4, 2).transpose(1, 3, 2, 0, 4).reshape(-1)
    assert np.array_equal(closed, perm)
    assert np.array_equal(perm[inv], np.arange(256))
    # second derivation (the runtime's tile decoder, runtime/src/qtip.cpp:93-98): step t = A*16+B*4+C*2+D
    # lands on row D*8+A, columns C*8+B*2+{0,1}
    for t in range(128):
        A, B, Cc, D = t >> 4, (t >> 2) & 3, (t >> 1) & 1, t & 1
        for e in range(2):
            assert perm[2 * t + e] == (D * 8 + A) * 16 + Cc * 8 + B * 2 + e


# ------------------------------------------------------------------ Hadamard
@pytest.mark.parametrize("n", [96, 1024, 12288, 28672])
def test_hadamard_golden(oracle, n):
    x = load("had_%d_x.bin" % n, np.float64)
    for t, tag in ((0, "u"), (1, "ut")):
        ref = load("had_%d_%s.bin" % (n, tag), np.float64)
        y = x.copy()
        assert oracle.lib().qo_hadamard_rows(y, 4, n, n, t) == 0
        assert np.max(np.abs(y - ref)) < 1e-6          # the upstream vectors divide by an fp32 sqrt(n)
        y32 = x.astype(np.float32)
        assert oracle.lib().qo_hadamard_rows_f32(y32, 4, n, n, t) == 0
        assert np.max(np.abs(y32 - ref)) < 2e-5        # tolerance of tests/test_gpu.cpp:61 for the fp32 dataflow


def test_hadamard_f32_equals_the_reference_device_kernels(oracle):
    """The fp32 dataflow against rows the reference's own device kernels transformed on a gfx950 GPU
    (k_hadamard_rows, src/kernels.hip:293-313; tests/golden/make_ref_hadamard_gpu_vectors.py): bit for bit."""
    cases = json.load(open(os.path.join(GOLDEN, "ref_hadamard_gpu.json")))["cases"]
    blob = np.fromfile(os.path.join(GOLDEN, "ref_hadamard_gpu.bin"), np.uint32)
    at = 0
    for n, rows, tr, seed in cases:
        want = blob[at:at + rows * n]
        at += rows * n
        x = oracle.rng_normal(seed, rows * n).astype(np.float32)
        assert oracle.lib().qo_hadamard_rows_f32(x, rows, n, n, tr) == 0
        assert np.array_equal(x.view(np.uint32), want), (n, tr)
    assert at == blob.size


def _had_tables():
    import re
    src = open(os.path.join(os.path.dirname(REFVEC), "..", "..", "behemoth-qtip_amd", "csrc", "data",
                            "qtip_tables.h")).read()
    order = [int(v) for v in re.search(r"qtip_had_order\[QTIP_NUM_HAD\] = \{([^}]*)\}", src).group(1).split(",")]
    out = {}
    for K in order:
        words = re.search(r"qtip_had%d_bits\[\d+\] = \{([^}]*)\}" % K, src).group(1)
        w = np.array([int(v.strip().rstrip("u"), 16) for v in words.split(",") if v.strip()], np.uint64)
        wpr = (K + 31) // 32
        Hm = np.zeros((K, K))
        for r in range(K):
            for k in range(K):
                Hm[r, k] = 1.0 if (int(w[r * wpr + (k >> 5)]) >> (k & 31)) & 1 else -1.0
        out[K] = Hm
    return order, out


def test_hadamard_tables_orthogonal():
    order, tabs = _had_tables()
    assert order == [172, 156, 140, 124, 116, 108, 60, 52, 36, 28, 20, 12]
    for K, Hm in tabs.items():
        assert np.array_equal(Hm @ Hm.T, K * np.eye(K)), K


@pytest.mark.parametrize("n", [64, 96, 80, 448, 3072])
def test_hadamard_explicit_definition(oracle, n):
    # (hadK^(T) (x) H_p) x / sqrt(n), H_p[i][j] = (-1)^popcount(i & j); involution U(U^t x) = x
    _, tabs = _had_tables()
    K = oracle.lib().qo_had_K(n)
    assert K > 0
    P = n // K
    i = np.arange(P)
    Hp = np.where(np.array([[bin(a & b).count("1") & 1 for b in i] for a in i]) == 1, -1.0, 1.0)
    hk = tabs[K] if K > 1 else np.ones((1, 1))
    rng = np.random.default_rng(n)
    x = rng.normal(size=(3, n))
    for t in (0, 1):
        full = np.kron(hk.T if t else hk, Hp) / np.sqrt(n)
        y = x.copy()
        assert oracle.lib().qo_hadamard_rows(y.reshape(-1), 3, n, n, t) == 0
        assert np.max(np.abs(y - x @ full.T)) < 1e-12
        z = y.copy()
        oracle.lib().qo_hadamard_rows(z.reshape(-1), 3, n, n, 1 - t)
        assert np.max(np.abs(z - x)) < 1e-12
        y32 = x.astype(np.float32)
        assert oracle.lib().qo_hadamard_rows_f32(y32.reshape(-1), 3, n, n, t) == 0
        assert np.max(np.abs(y32 - x @ full.T)) < 2e-5
    # strided rows leave the padding alone
    ld = n + 8
    buf = rng.normal(size=(3, ld))
    keep = buf[:, n:].copy()
    want = buf[:, :n] @ (np.kron(hk, Hp) / np.sqrt(n)).T
    flat = buf.reshape(-1).copy()
    oracle.lib().qo_hadamard_rows(flat, 3, n, ld, 0)
    assert np.max(np.abs(flat.reshape(3, ld)[:, :n] - want)) < 1e-12
    assert np.array_equal(flat.reshape(3, ld)[:, n:], keep)


def test_had_K_rule(oracle):
    hk = oracle.lib().qo_had_K
    assert hk(1024) == 1 and hk(12288) == 12 and hk(28672) == 28 and hk(96) == 12 and hk(8192) == 1
    assert hk(57344) == 28 and hk(256) == 1
    assert hk(3000) == 0          # 3000 = 60 * 50: the first dividing K decides, 50 is no power of two
    assert hk(36 * 64) == 36      # 2304 is also 12 * 192, but 36 comes first in the order
    assert hk(100) == 0 and hk(7) == 0


# ------------------------------------------------------------------ Viterbi
def test_viterbi_golden(oracle, hyb):
    X = load("vit_x.bin", np.float32).reshape(24, 256)
    st = load("vit_states.bin", np.int32).reshape(24, 128).astype(np.uint16)
    hat = load("vit_hat.bin", np.float32).reshape(24, 256)
    L = oracle.lib()
    for fast in (False, True):
        got, ghat = oracle.quantize_tiles(hyb, X, fast=fast, want_hat=True)
        assert np.array_equal(got, st)
        assert np.array_equal(ghat, hat)
    for b in range(24):
        s = st[b]
        assert (int(s[127]) & 0xfff) == (int(s[0]) >> 4)                    # tail-biting
        assert np.all(((s[:-1].astype(np.uint32) << 4) & 0xffff) == (s[1:] & 0xfff0))  # trellis links
        h = np.zeros(256, np.float32)
        L.qo_decode_states(hyb.lut0, hyb.lut1, np.ascontiguousarray(s), h)
        assert np.array_equal(h, hat[b])


def _numpy_viterbi(cb, X, overlap):
    """Independent formulation: whole-vector recursion in numpy (fp64), first-minimum tie-breaks."""
    l0 = cb.lut0.astype(np.float64)
    l1 = cb.lut1.astype(np.float64)
    s = np.arange(65536)
    X = X.astype(np.float64)
    cost = (l0 - X[0]) ** 2 + (l1 - X[1]) ** 2
    if overlap >= 0:
        cost = np.where((s >> 4) == overlap, cost, np.inf)
    back = np.zeros((128, 4096), np.int64)
    for i in range(1, 128):
        c = cost.reshape(16, 4096)          # c[d, j] = cost[j | d << 12]
        back[i] = np.argmin(c, axis=0)      # first minimum
        M = c.min(axis=0)
        cost = (l0 - X[2 * i]) ** 2 + (l1 - X[2 * i + 1]) ** 2 + M[s >> 4]
    if overlap >= 0:
        cost = np.where((s & 0xfff) == overlap, cost, np.inf)
    st = np.zeros(128, np.int64)
    st[127] = int(np.argmin(cost))
    for i in range(127, 0, -1):
        j = st[i] >> 4
        st[i - 1] = j | (back[i][j] << 12)
    return st.astype(np.uint16), float(cost.min())


def test_viterbi_independent_formulation(oracle, syn, hyb):
    # numpy rounds (a*a + b*b) without fusing, so compare paths (identical unless a 1e-16 near-tie) and
    # costs to 1e-12; inputs are raw fp32 normals, not fp16-representable
    X = oracle.rng_normal(5, 4 * 256).astype(np.float32).reshape(4, 256)
    L = oracle.lib()
    for cb in (syn, hyb):
        for b in range(4):
            for ov in (-1, 1234, 0, 4095):
                st = np.zeros(128, np.uint16)
                c = L.qo_viterbi(cb.lut0, cb.lut1, X[b], ov, st)
                st2 = np.zeros(128, np.uint16)
                c2 = L.qo_viterbi_fast(cb.lut0, cb.lut1, X[b], ov, st2)
                assert c == c2 and np.array_equal(st, st2)
                ns, nc = _numpy_viterbi(cb, X[b], ov)
                assert np.array_equal(ns, st)
                assert abs(nc - c) < 1e-12 * max(1.0, c)
                assert abs(L.qo_path_cost(cb.lut0, cb.lut1, X[b], st) - c) < 1e-10
                if ov >= 0:
                    assert (int(st[0]) >> 4) == ov and (int(st[127]) & 0xfff) == ov


def test_viterbi_optimality_against_perturbed_paths(oracle, syn):
    # the returned path costs no more than any valid path obtained by re-deciding a window of new bits
    X = oracle.rng_normal(9, 256).astype(np.float32)
    L = oracle.lib()
    st = np.zeros(128, np.uint16)
    c = L.qo_viterbi(syn.lut0, syn.lut1, X, -1, st)
    bits = [int(st[0])] + [int(v) & 15 for v in st[1:]]
    rng = np.random.default_rng(1)
    for _ in range(300):
        nb = list(bits)
        t = int(rng.integers(0, 128))
        if t == 0:
            nb[0] = int(rng.integers(0, 65536))
        else:
            nb[t] = int(rng.integers(0, 16))
        s = nb[0]
        path = [s]
        for t2 in range(1, 128):
            s = ((s << 4) & 0xffff) | nb[t2]
            path.append(s)
        pc = L.qo_path_cost(syn.lut0, syn.lut1, X, np.array(path, np.uint16))
        assert pc >= c - 1e-12


def test_viterbi_exact_recovery(oracle, syn):
    # a sequence that IS a codeword path (cost 0) is recovered; the tail-biting two-pass keeps it when the
    # path itself is tail-biting
    rng = np.random.default_rng(3)
    nibb = rng.integers(0, 16, 128)
    # tail-biting stream of 128 nibbles: state_t = nibbles t-3..t (wrapping)
    st = np.array([(nibb[(t - 3) % 128] << 12) | (nibb[(t - 2) % 128] << 8) | (nibb[(t - 1) % 128] << 4) | nibb[t]
                   for t in range(128)], np.uint16)
    X = np.zeros(256, np.float32)
    oracle.lib().qo_decode_states(syn.lut0, syn.lut1, st, X)
    got = np.zeros(128, np.uint16)
    hat = np.zeros(256, np.float32)
    c = oracle.lib().qo_quantize_seq(syn.lut0, syn.lut1, X, got, hat)
    assert c == 0.0 and np.array_equal(hat, X)


# ------------------------------------------------------------------ packing
def test_pack_golden(oracle):
    st = load("pack_states.bin", np.int32).astype(np.uint16).reshape(-1, 128)
    plain = load("pack_plain.bin", np.uint16)
    kern = load("pack_kernel.bin", np.uint16)
    pk = oracle.pack_trellis(st)
    assert np.array_equal(pk.reshape(-1), plain)
    sw = oracle.swizzle(pk, 64, 96)
    assert np.array_equal(sw, kern)
    assert np.array_equal(oracle.unpack_trellis(oracle.unswizzle(sw, 64, 96)), st)


def test_pack_independent_decoder(oracle, syn):
    # decoder of the kernel layout written from the runtime's description (runtime/src/qtip.cpp:83-100,
    # runtime/include/behemoth/qtip.hpp:63-67): windows of 16 bits at bit 4t of a wrapping 512-bit stream
    m, n = 64, 96
    rng = np.random.default_rng(7)
    B = (m // 16) * (n // 16)
    nib = rng.integers(0, 16, (B, 128))
    st = np.zeros((B, 128), np.uint16)
    for t in range(128):
        st[:, t] = (nib[:, (t - 3) % 128] << 12) | (nib[:, (t - 2) % 128] << 8) | (nib[:, (t - 1) % 128] << 4) | nib[:, t]
    tr = oracle.swizzle(oracle.pack_trellis(st), m, n)
    n2 = n // 32
    for trow in range(m // 16):
        for tcol in range(n // 16):
            i0, i1, j0, j1 = trow // 2, trow % 2, tcol // 2, tcol % 2
            w = [int(tr[(((i0 * n2 + j0) * 32 + c) * 2 + j1) * 2 + i1]) for c in range(32)]
            for t in range(128):
                # the window starting at stream bit 4t is the state of step t (wrapping at 512 bits)
                i, sft = t >> 2, 4 * (t & 3)
                u = (w[i] << 16) | w[(i + 1) & 31]
                state = (u >> (16 - sft)) & 0xffff
                assert state == int(st[trow * (n // 16) + tcol, t])
    # m or n not a multiple of 32 is refused (src/qtip_core.cpp:234)
    assert oracle.lib().qo_swizzle_for_kernel(np.zeros(16 * 6 * 32, np.uint16), 16, 96, np.zeros(16 * 6 * 32, np.uint16)) != 0


# ------------------------------------------------------------------ LDL
def test_ldl_golden(oracle):
    H = load("ldl_H.bin", np.float64).reshape(96, 96)
    Lr = load("ldl_L.bin", np.float64).reshape(96, 96)
    L = oracle.block_ldl(H)
    assert L is not None
    assert np.max(np.abs(L.astype(np.float64) - Lr)) < 1e-5   # tolerance of tests/test_cpu.cpp:136


def test_ldl_textbook(oracle):
    rng = np.random.default_rng(2)
    n = 208
    G = rng.normal(size=(n, 300))
    H = G @ G.T / 300 + 0.05 * np.eye(n)
    A = H.copy()
    assert oracle.lib().qo_cholesky(A.reshape(-1), n) == 1
    Cn = np.linalg.cholesky(H)
    assert np.max(np.abs(np.tril(A) - Cn)) < 1e-12
    L = oracle.block_ldl(H).astype(np.float64)
    # L (with identity diagonal blocks restored) * D * L^T = H, D = blockdiag(C_bb C_bb^T)
    Lf = L.copy()
    D = np.zeros((n, n))
    for b in range(n // 16):
        sl = slice(16 * b, 16 * b + 16)
        assert np.all(Lf[sl, sl] == 0)
        Lf[sl, sl] = np.eye(16)
        D[sl, sl] = Cn[sl, sl] @ Cn[sl, sl].T
    assert np.all(np.triu(L, 1) == 0)
    assert np.max(np.abs(Lf @ D @ Lf.T - H)) < 1e-5
    # not positive definite -> refused (src/qtip_core.cpp:333)
    bad = H.copy()
    bad[5, 5] = -1.0
    assert oracle.block_ldl(bad) is None


# ------------------------------------------------------------------ LDLQ
def _spd(n, seed):
    rng = np.random.default_rng(seed)
    G = rng.normal(size=(n, 2 * n)) * (1.0 + (np.arange(2 * n) % 7))
    return G @ G.T / (2 * n) + 0.05 * np.eye(n)


def test_ldlq_buffered_equals_naive(oracle, hyb):
    m, n = 32, 256
    rng = np.random.default_rng(4)
    Wr = rng.normal(size=(m, n)).astype(np.float32)
    L = oracle.block_ldl(_spd(n, 5))
    hat, Q = oracle.ldlq(hyb, Wr, L)
    hat2, Q2 = oracle.ldlq(hyb, Wr, L, naive=True)
    same = np.all(Q == Q2, axis=1).mean()
    assert same == 1.0, same
    assert np.array_equal(hat, hat2)
    # decode(Q) == hatW per tile, through the tile permutation
    perm, _ = oracle.perm256()
    for b in range(m // 16):
        for blk in range(n // 16):
            h = np.zeros(256, np.float32)
            oracle.lib().qo_decode_states(hyb.lut0, hyb.lut1, np.ascontiguousarray(Q[b * (n // 16) + blk]), h)
            tile = hat[16 * b:16 * b + 16, 16 * blk:16 * blk + 16].reshape(-1)
            assert np.array_equal(tile[perm], h)


def test_ldlq_equals_the_reference_ldlq(oracle, hyb):
    """ldlq_ref of the reference's GPU test program (CPU code, tests/test_gpu.cpp:180-225): every state and every
    reconstructed value of a two-buffer case, from the committed vectors and, where oracle/_ref is built, live."""
    meta = json.load(open(os.path.join(GOLDEN, "ref_ldlq.json")))
    m, n = meta["m"], meta["n"]
    Wr = oracle.rng_normal(meta["w_seed"], m * n).astype(np.float32).reshape(m, n)
    L = np.fromfile(os.path.join(GOLDEN, "ref_ldlq_L.bin"), np.float32).reshape(n, n)
    want = np.fromfile(os.path.join(GOLDEN, "ref_ldlq_Q.bin"), np.uint16).reshape(-1, 128)
    hat, Q = oracle.ldlq(hyb, Wr, L)
    assert np.array_equal(Q, want)
    h = 0xcbf29ce484222325
    for b in hat.tobytes():
        h = ((h ^ b) * 0x100000001b3) & 0xffffffffffffffff
    assert "%016x" % h == meta["fnv1a64_hat"]
    if oracle.ref_gpu_lib() is not None:
        rng = np.random.default_rng(12)
        m2, n2 = 32, 384                                  # three buffers
        W2 = (rng.standard_normal((m2, n2)) * 1.3).astype(np.float32)
        L2 = oracle.block_ldl(_spd(n2, 13))
        hat_o, Q_o = oracle.ldlq(hyb, W2, L2)
        hat_r, Q_r = oracle.ref_ldlq(W2, L2)
        assert np.array_equal(Q_o, Q_r) and np.array_equal(hat_o, hat_r)


def test_ldlq_zero_L_is_tilewise_viterbi(oracle, hyb):
    m, n = 16, 128
    rng = np.random.default_rng(6)
    Wr = rng.normal(size=(m, n)).astype(np.float32)
    hat, Q = oracle.ldlq(hyb, Wr, np.zeros((n, n), np.float32))
    perm, _ = oracle.perm256()
    for blk in range(n // 16):
        x = Wr[:, 16 * blk:16 * blk + 16].reshape(-1)[perm].astype(np.float16).astype(np.float32)
        st = oracle.quantize_tiles(hyb, x)[0]
        assert np.array_equal(st, Q[blk])


def test_ldlq_feedback_lowers_proxy(oracle, hyb):
    # the point of the feedback: with the true L the proxy loss beats plain round-to-nearest-path
    m, n = 32, 256
    rng = np.random.default_rng(8)
    Wr = rng.normal(size=(m, n)).astype(np.float32)
    H = _spd(n, 9)
    L = oracle.block_ldl(H)
    hat, _ = oracle.ldlq(hyb, Wr, L)
    hat0, _ = oracle.ldlq(hyb, Wr, np.zeros_like(L))
    H32 = H.astype(np.float32)
    p = oracle.lib().qo_proxy(Wr.reshape(-1), hat.reshape(-1), H32.reshape(-1), m, n, 0)
    p0 = oracle.lib().qo_proxy(Wr.reshape(-1), hat0.reshape(-1), H32.reshape(-1), m, n, 0)
    D = (Wr - hat).astype(np.float64)
    want = np.trace(D @ H32.astype(np.float64) @ D.T) / np.trace(Wr.astype(np.float64) @ H32.astype(np.float64) @ Wr.T.astype(np.float64))
    assert abs(p - want) < 1e-8 * want
    assert p < p0


# ------------------------------------------------------------------ whole group against the reference's device path
def _group_fixture(name):
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_ref_group_gpu_vectors",
                                                  os.path.join(GOLDEN, "make_ref_group_gpu_vectors.py"))
    gen = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(gen)
    meta = json.load(open(os.path.join(GOLDEN, "ref_group_gpu.json")))[name]
    Ws, H, seed = gen.group_case(name)
    blob = open(os.path.join(GOLDEN, "ref_group_gpu_%s.bin" % name), "rb").read()
    n, want, at = meta["n"], [], 0
    for m in meta["ms"]:
        words = (m // 16) * (n // 16) * 32
        tr = np.frombuffer(blob, np.uint16, words, at)
        su = np.frombuffer(blob, np.uint16, n, at + 2 * words)
        sv = np.frombuffer(blob, np.int8, m, at + 2 * words + 2 * n).astype(np.float32)
        at += 2 * words + 2 * n + m
        want.append((tr, su, sv))
    assert at == len(blob)
    return meta, Ws, H, seed, want


@pytest.mark.parametrize("name", ["a", "b"])
def test_group_composition_matches_reference_device_path(oracle, hyb, name):
    """qo_rotate_hessian + qo_quantize_group against what the reference's own quantize_group returned on a gfx950 GPU
    for the same inputs (committed vectors): the sign vectors from their seeds, Wscale, the two proxy errors and the
    place of every linear's words in the output.  The device path scores and feeds back in fp32, so its codes need not
    equal the fp64 CPU form's word for word once the chains get long: every word must agree at n = 256, 97 % of the
    tiles at n = 1024 (64 sequential column blocks; as committed, all 512 tiles agree)."""
    meta, Ws, H, seed, want = _group_fixture(name)
    n = meta["n"]
    r = oracle.quantize_group(hyb.tlut, Ws, H, seed, threads=8)
    off = 0
    for k, (tr, su, sv) in enumerate(want):
        m = meta["ms"][k]
        words = (m // 16) * (n // 16) * 32
        assert np.array_equal(r["su_bf16"], su), "SU of linear %d" % k
        assert np.array_equal(r["sv"][off:off + m], sv), "SV of linear %d" % k
        ws = float.fromhex(meta["wscale"][k])
        assert abs(r["wscale"][k] - ws) <= 2e-6 * ws          # the device path sums with atomics
        assert abs(r["proxy"][k] - meta["proxy"][k]) <= 2e-3 * meta["proxy"][k]
        assert abs(r["proxy_rot_reg"][k] - meta["proxy_rot_reg"][k]) <= 2e-3 * meta["proxy_rot_reg"][k]
        got = r["trellis"][(off // 16) * (n // 16) * 32:][:words].reshape(-1, 32)
        # both are in kernel layout: compare tile by tile after undoing the swizzle
        same = np.all(oracle.unswizzle(got.reshape(-1), m, n).reshape(-1, 32) ==
                      oracle.unswizzle(tr.copy(), m, n).reshape(-1, 32), axis=1)
        print("case %s linear %d: %d of %d tiles identical to the reference's device path" % (name, k, same.sum(), same.size))
        if n <= 256:
            assert same.all()
        else:
            assert same.mean() >= 0.97
        off += m
