"""GPU parity of the group path through the C ABI: Hadamard rows, Hessian rotation, LDLQ, whole groups.
Mirrors tests/test_gpu.cpp:27-64 (Hadamard), :227-299 (LDLQ vs the CPU form of the algorithm) and :301-372
(quantize_group end to end, proxy recomputed on the CPU from the packed output) of the reference."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)


@pytest.fixture(scope="module")
def synth(pkg):
    import importlib.util
    from conftest import ROOT
    spec = importlib.util.spec_from_file_location("qtip_synth", os.path.join(ROOT, "behemoth-qtip_amd", "synth.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("n", [12, 64, 96, 80, 448, 864, 1024, 2304, 3328, 4096, 8192, 12288, 20480, 28672, 36864, 49152,
                               53248, 57344])
def test_hadamard_rows(qz, oracle, n):
    """Bit-identical to the fp32 dataflow of the reference's kernels (restated on the CPU) and within 2e-5 of the
    fp64 definition (tests/test_gpu.cpp:27-50); strided rows keep their padding."""
    import torch
    say("case: hadamard n=%d" % n)
    rows, ld = 6, n + 32
    x = oracle.rng_normal(n, rows * ld).astype(np.float32).reshape(rows, ld)
    for tr in (0, 1):
        d = torch.from_numpy(x.copy()).cuda()
        qz.hadamard_rows_dev(d, rows, n, ld, tr)
        qz.synchronize()
        y = d.cpu().numpy()
        w32 = x.copy().reshape(-1)
        assert oracle.lib().qo_hadamard_rows_f32(w32, rows, n, ld, tr) == 0
        assert np.array_equal(y.view(np.uint32), w32.reshape(rows, ld).view(np.uint32))
        w64 = x.astype(np.float64).reshape(-1)
        oracle.lib().qo_hadamard_rows(w64, rows, n, ld, tr)
        assert np.max(np.abs(y[:, :n] - w64.reshape(rows, ld)[:, :n])) < 2e-5
        assert np.array_equal(y[:, n:], x[:, n:])


@pytest.mark.parametrize("n", [12288, 20480, 28672, 36864])
def test_hadamard_many_rows(qz, oracle, n):
    """Rows of K x 1024 values, more of them than workgroups are resident: every workgroup walks several rows with the
    next one in flight.  Bit-identical to the fp32 dataflow of the reference's kernels; the last rows, which some
    workgroups no longer have, included."""
    import torch
    say("case: hadamard many rows n=%d" % n)
    rows = 2 * 256 * 2 + 37
    x = oracle.rng_normal(7 + n, rows * n).astype(np.float32).reshape(rows, n)
    for tr in (0, 1):
        d = torch.from_numpy(x).cuda()
        qz.hadamard_rows_dev(d, rows, n, n, tr)
        qz.synchronize()
        y = d.cpu().numpy()
        w32 = x.copy().reshape(-1)
        assert oracle.lib().qo_hadamard_rows_f32(w32, rows, n, n, tr) == 0
        assert np.array_equal(y.view(np.uint32), w32.reshape(rows, n).view(np.uint32)), (n, tr)


def test_hadamard_rejects_unsupported(qz, pkg):
    import torch
    d = torch.zeros((2, 3000), device="cuda")
    with pytest.raises(pkg.QtipError) as e:
        qz.hadamard_rows_dev(d, 2, 3000, 3000, 0)     # 3000 = 60 * 50, 50 is no power of two
    assert e.value.code == pkg.QTIP_E_ARG
    d = torch.zeros((1, 16384), device="cuda")
    with pytest.raises(pkg.QtipError):
        qz.hadamard_rows_dev(d, 1, 16384, 16384, 0)   # power-of-two part above 8192


def _spd(n, seed):
    rng = np.random.default_rng(seed)
    G = rng.normal(size=(n, 2 * n)) * (1.0 + (np.arange(2 * n) % 7))
    return G @ G.T / (2 * n) + 0.05 * np.eye(n)


def _ldlq_gpu(qz, Wr, L):
    import torch
    m, n = Wr.shape
    dWT = torch.from_numpy(np.ascontiguousarray(Wr.T)).cuda()
    dL = torch.from_numpy(L).cuda()
    dH = torch.zeros((n, m), device="cuda")
    dQ = torch.zeros(((m // 16) * (n // 16), 128), dtype=torch.int16, device="cuda")
    torch.cuda.synchronize()
    vs = qz.ldlq_dev(dWT, dL, n, m, dH, dQ, time_viterbi=True)
    return dH.cpu().numpy().T.copy(), dQ.cpu().numpy().view(np.uint16), vs


@pytest.mark.parametrize("m,n", [(64, 256), (32, 128), (16, 384)])
def test_ldlq_matches_cpu_algorithm(qz, oracle, hyb, m, n):
    say("case: ldlq m=%d n=%d" % (m, n))
    qz.set_tlut(None)
    rng = np.random.default_rng(21 + n)
    Wr = rng.normal(size=(m, n)).astype(np.float32)
    H = _spd(n, 5)
    L = oracle.block_ldl(H)
    hat_o, Q_o = oracle.ldlq(hyb, Wr, L)
    hat_g, Q_g, vs = _ldlq_gpu(qz, Wr, L)
    same = np.all(Q_g == Q_o, axis=1).mean()
    H32 = H.astype(np.float32)
    po = oracle.lib().qo_proxy(Wr.reshape(-1), hat_o.reshape(-1), H32.reshape(-1), m, n, 0)
    pg = oracle.lib().qo_proxy(Wr.reshape(-1), np.ascontiguousarray(hat_g).reshape(-1), H32.reshape(-1), m, n, 0)
    say("  identical trellises %.4f, proxy cpu %.6f gpu %.6f, viterbi %.4fs" % (same, po, pg, vs))
    assert same >= 0.99
    assert abs(pg - po) / po < 0.01
    # decode(states) == hatW per tile
    perm, _ = oracle.perm256()
    l0, l1 = qz.lut()
    for b in range(m // 16):
        for blk in range(n // 16):
            st = Q_g[b * (n // 16) + blk]
            h = np.stack([l0[st], l1[st]], axis=-1).reshape(-1)
            tile = hat_g[16 * b:16 * b + 16, 16 * blk:16 * blk + 16].reshape(-1)
            assert np.array_equal(tile[perm], h)


def test_ldlq_split_bf16_feedback(qz, oracle, hyb):
    """feedback = 1 (fp32 sums in the buffer, prod cache by the bf16 hi/lo split MFMA product, the arithmetic of the
    reference's GPU path): not bit-tracking the fp64 CPU form, so the bar is the reference's own for this
    arithmetic (tests/test_gpu.cpp:295-296): proxy within 1 %, decode(states) == hatW."""
    import torch
    say("case: ldlq feedback=1 m=64 n=512")
    qz.set_tlut(None)
    m, n = 64, 512
    rng = np.random.default_rng(77)
    Wr = rng.normal(size=(m, n)).astype(np.float32)
    H = _spd(n, 6)
    L = oracle.block_ldl(H)
    hat_o, Q_o = oracle.ldlq(hyb, Wr, L)
    dWT = torch.from_numpy(np.ascontiguousarray(Wr.T)).cuda()
    dL = torch.from_numpy(L).cuda()
    dH = torch.zeros((n, m), device="cuda")
    dQ = torch.zeros(((m // 16) * (n // 16), 128), dtype=torch.int16, device="cuda")
    torch.cuda.synchronize()
    qz.ldlq_dev(dWT, dL, n, m, dH, dQ, feedback=1)
    hat_g = dH.cpu().numpy().T.copy()
    Q_g = dQ.cpu().numpy().view(np.uint16)
    H32 = H.astype(np.float32)
    po = oracle.lib().qo_proxy(Wr.reshape(-1), hat_o.reshape(-1), H32.reshape(-1), m, n, 0)
    pg = oracle.lib().qo_proxy(Wr.reshape(-1), np.ascontiguousarray(hat_g).reshape(-1), H32.reshape(-1), m, n, 0)
    same = np.all(Q_g == Q_o, axis=1).mean()
    say("  identical trellises %.4f, proxy cpu %.6f gpu %.6f" % (same, po, pg))
    assert abs(pg - po) / po < 0.01
    perm, _ = oracle.perm256()
    l0, l1 = qz.lut()
    for b in range(m // 16):
        for blk in range(n // 16):
            st = Q_g[b * (n // 16) + blk]
            h = np.stack([l0[st], l1[st]], axis=-1).reshape(-1)
            assert np.array_equal(hat_g[16 * b:16 * b + 16, 16 * blk:16 * blk + 16].reshape(-1)[perm], h)
    with pytest.raises(Exception):
        qz.ldlq_dev(dWT, dL, n, m, dH, dQ, feedback=7)


def _bf16_parts(x):
    """hi = bf16(x), lo = bf16(x - hi), both rounded to nearest even, as float32 arrays"""
    def rne(v):
        u = np.ascontiguousarray(v, dtype=np.float32).view(np.uint32).astype(np.uint64)
        u = ((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16
        return u.astype(np.uint32).view(np.float32)
    hi = rne(x)
    return hi, rne(x - hi)


@pytest.mark.parametrize("K,N", [(1408, 192), (8256, 64), (64, 128)])
def test_prod_cache_split_bf16(qz, K, N):
    """The gathered cross-buffer product of feedback = 1 (bf16 hi / lo images, three matrix-core terms, fp32 sums)
    against the same three terms summed in fp64 from operands split on the host (src/quantizer.cpp:66-76 for the
    terms).  The bound, 2e-6 of sum |a| |b|, is some fifty times the rounding of the fp32 sums and a twentieth of
    what a dropped lo term, a wrong row or a wrong k would change; the test checks the latter on its own data.
    Rows padded (ldl, ldw beyond the sizes), N not a multiple of the 128-column tile, K split over workgroups."""
    import torch
    say("case: prod cache split bf16 K=%d N=%d" % (K, N))
    rng = np.random.default_rng(K + N)
    ldl, ldw = 128 + 64, N + 32
    Lr = (rng.normal(size=(K, ldl)) * np.exp(rng.normal(size=(K, 1)))).astype(np.float32)
    WT = rng.normal(size=(K, ldw)).astype(np.float32)
    HT = (WT + 0.1 * rng.normal(size=(K, ldw))).astype(np.float32)
    dP = torch.full((128, N), 7.0, device="cuda")
    qz.prod_cache_bf16x3_dev(N, K, torch.from_numpy(Lr).cuda(), ldl, torch.from_numpy(WT).cuda(),
                             torch.from_numpy(HT).cuda(), ldw, dP)
    got = dP.cpu().numpy().astype(np.float64)
    lh, ll = _bf16_parts(Lr[:, :128])
    dh, dl = _bf16_parts(WT[:, :N] - HT[:, :N])
    lh, ll, dh, dl = (v.astype(np.float64) for v in (lh, ll, dh, dl))
    want = ll.T @ dh + lh.T @ dl + lh.T @ dh
    bound = 2e-6 * (np.abs(lh).T @ np.abs(dh)) + 1e-30
    err = np.abs(got - want)
    say("  largest error over bound %.3f" % (err / bound).max())
    assert np.all(err <= bound)
    if K >= 1024:   # what the bound tells apart: two terms only, and a product shifted by one row of k
        assert np.mean(np.abs(lh.T @ dl + lh.T @ dh - want) > bound) > 0.9
        assert np.mean(np.abs(np.roll(lh + ll, 1, axis=0).T @ (dh + dl) - want) > bound) > 0.9


def test_ldlq_rejects_bad_shapes(qz, pkg):
    import torch
    z = torch.zeros(1, device="cuda")
    for n, m in ((200, 64), (256, 24)):
        with pytest.raises(pkg.QtipError) as e:
            qz.ldlq_dev(z, z, n, m, z, z)
        assert e.value.code == pkg.QTIP_E_ARG


def test_rotate_hessian_matches_cpu(qz, oracle, pkg, synth):
    say("case: rotate_hessian n=256")
    Ws, H = synth.small_group()
    n = H.shape[0]
    hp = qz.rotate_hessian(H, n, 7)
    su = np.zeros(n, np.float32)
    HRr = np.zeros((n, n), np.float32)
    import ctypes
    creg = ctypes.c_double()
    assert oracle.lib().qo_rotate_hessian(H.reshape(-1), n, 7, 1e-2, su, ctypes.byref(creg), HRr.reshape(-1)) == 0
    assert np.array_equal(hp.su, su)
    assert abs(hp.creg - creg.value) <= 1e-12 * abs(creg.value)
    assert np.array_equal(hp.HRr.view(np.uint32), HRr.view(np.uint32))
    # device-resident H takes the same path
    import torch
    hp2 = qz.rotate_hessian(torch.from_numpy(H).cuda(), n, 7)
    assert np.array_equal(hp2.HRr, hp.HRr)


def _decode_proxy(oracle, pkg, cb, lo, W, H):
    """CPU decode of the packed output back to the original domain and the proxy with the unregularised H."""
    m, n = W.shape
    st = pkg.unpack_trellis(pkg.unswizzle_for_kernel(lo.trellis, m, n))
    perm, _ = oracle.perm256()
    hw = np.zeros((m, n))
    for b in range(m // 16):
        for blk in range(n // 16):
            s = st[b * (n // 16) + blk]
            h = np.stack([cb.lut0[s], cb.lut1[s]], axis=-1).reshape(-1).astype(np.float64) * lo.wscale
            tile = np.zeros(256)
            tile[perm] = h
            hw[16 * b:16 * b + 16, 16 * blk:16 * blk + 16] = tile.reshape(16, 16)
    flat = np.ascontiguousarray(hw).reshape(-1)
    oracle.lib().qo_hadamard_rows(flat, m, n, n, 0)
    t = np.ascontiguousarray(flat.reshape(m, n).T).reshape(-1)
    oracle.lib().qo_hadamard_rows(t, n, m, m, 0)
    su = (lo.su_bf16.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    hat = t.reshape(n, m).T * lo.sv[:, None].astype(np.float64) * su[None, :]
    D = W.astype(np.float64) - hat
    H64 = H.astype(np.float64)
    return np.trace(D @ H64 @ D.T) / np.trace(W.astype(np.float64) @ H64 @ W.T.astype(np.float64)), hat


def test_group_small_end_to_end(qz, oracle, pkg, hyb, synth):
    """tests/test_gpu.cpp:301-372: two linears (m = 64 and 32, n = 256) sharing one Hessian."""
    say("case: group n=256, m=64+32")
    qz.set_tlut(None)
    Ws, H = synth.small_group()
    n = H.shape[0]
    lins = [pkg.LinearIn("a", Ws[0].shape[0], w_f32=Ws[0]), pkg.LinearIn("b", Ws[1].shape[0], w_f32=Ws[1])]
    outs, tm = qz.quantize_group_h(lins, n, H, 7, pkg.QuantOpts(want_hatW=True, ldl_threads=4))
    ref = oracle.quantize_group(hyb.tlut, Ws, H, 7)
    off = 0
    for k, lo in enumerate(outs):
        m = lo.m
        words = (m // 16) * (n // 16) * 32
        want = ref["trellis"][off // 16 * (n // 16) * 32: off // 16 * (n // 16) * 32 + words]
        tiles_same = np.all(lo.trellis.reshape(-1, 32) == want.reshape(-1, 32), axis=1).mean()
        say("  %s: proxy %.5f (cpu %.5f) rot_reg %.5f Wscale %.6f (cpu %.6f) tiles identical %.4f" %
            (lo.name, lo.proxy, ref["proxy"][k], lo.proxy_rot_reg, lo.wscale, ref["wscale"][k], tiles_same))
        assert lo.trellis.size == words
        assert np.array_equal(lo.sv, ref["sv"][off:off + m])
        assert np.array_equal(lo.su_bf16, ref["su_bf16"])
        assert lo.wscale == ref["wscale"][k]
        assert np.array_equal(lo.trellis, want)
        assert abs(lo.proxy - ref["proxy"][k]) / ref["proxy"][k] < 1e-3
        assert abs(lo.proxy_rot_reg - ref["proxy_rot_reg"][k]) / ref["proxy_rot_reg"][k] < 1e-3
        assert 0 < lo.proxy < 0.2
        p, hat = _decode_proxy(oracle, pkg, hyb, lo, Ws[k], H)
        say("  %s: CPU decode of the packed output -> proxy %.5f" % (lo.name, p))
        assert abs(p - lo.proxy) / lo.proxy < 1e-3
        assert np.max(np.abs(hat - lo.hatW)) < 1e-5 * max(1.0, np.max(np.abs(hat)) / 1e-2)
        off += m
    assert tm.total > 0 and tm.ldlq > 0 and tm.viterbi > 0


def test_default_chain_count(qz):
    """A context times its side streams when it is made and runs three LDLQ chains by default where three of them
    have hardware queues of their own, else two (unless the environment promises six queues or more)."""
    n = qz.ldlq_default_chains()
    say("default LDLQ chains of this context: %d" % n)
    assert n in (2, 3)


def test_ldlq_chains_give_the_same_codes(qz, oracle, pkg, hyb):
    """The tile rows of a group are dealt to 1, 2 or 3 independent chains of launches (streams of their own, feedback
    slabs of their own, ragged shares of rows with two linears of different height): every packed word, Wscale and
    proxy must come out the same, and two tile rows must equal the CPU form."""
    import torch
    say("case: LDLQ chains 1 / 2 / 3, 12288 + 32 rows x 256 columns")
    n, m1, m2 = 256, 12288, 32
    rng = np.random.default_rng(12)
    W1 = (rng.standard_normal((m1, n)) * 0.02).astype(np.float32)
    W2 = (rng.standard_normal((m2, n)) * 0.05).astype(np.float32)
    G = rng.standard_normal((n, 2 * n)) * (1.0 + (np.arange(2 * n) % 5))
    H = (G @ G.T / (2 * n)).astype(np.float32)
    res = []
    for chains in (1, 2, 3):
        outs, _ = qz.quantize_group_h([pkg.LinearIn("a", m1, w_f32=W1), pkg.LinearIn("b", m2, w_f32=W2)], n, H, 21,
                                      pkg.QuantOpts(ldl_threads=4, ldlq_chains=chains))
        res.append(outs)
    for outs in res[1:]:
        for a, b in zip(res[0], outs):
            assert np.array_equal(a.trellis, b.trellis) and a.wscale == b.wscale and a.proxy == b.proxy
    ref = oracle.quantize_group(hyb.tlut, [W1[:32], W2], H, 21)   # rows are independent given L: but Wscale is not
    # the second linear is complete in both calls: its words must be the oracle's
    t2 = (32 // 16) * (n // 16) * 32
    assert np.array_equal(res[0][1].trellis, ref["trellis"][t2:])
    with pytest.raises(pkg.QtipError):
        qz.quantize_group_h([pkg.LinearIn("b", m2, w_f32=W2)], n, H, 21, pkg.QuantOpts(ldlq_chains=4))


def test_group_input_formats_and_errors(qz, oracle, pkg, synth):
    """bf16 and fp8+scale sources decode to the same fp32 weights the fp32 path sees; precondition failures come
    back as error codes (the reference aborts: src/quantizer.cpp:32-33,209-211, src/qtip_core.cpp:234)."""
    say("case: input formats / errors")
    Ws, H = synth.small_group(ms=(32,))
    n = H.shape[0]
    W = Ws[0]
    wb = ((W.view(np.uint32).astype(np.uint64) + 0x7fff + ((W.view(np.uint32) >> 16) & 1)) >> 16).astype(np.uint16)
    Wb = (wb.astype(np.uint32) << 16).view(np.float32)
    o1, _ = qz.quantize_group_h([pkg.LinearIn("w", 32, w_bf16=wb)], n, H, 3, pkg.QuantOpts(skip_proxy=True))
    o2, _ = qz.quantize_group_h([pkg.LinearIn("w", 32, w_f32=Wb)], n, H, 3, pkg.QuantOpts(skip_proxy=True))
    assert np.array_equal(o1[0].trellis, o2[0].trellis) and o1[0].wscale == o2[0].wscale and o1[0].proxy == 0
    # fp8 e4m3 codes with a per-row bf16 scale
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 256, (32, n)).astype(np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x30        # no NaN codes
    sc = np.full(32, 0x3c00, np.uint16)         # bf16 0x3c00 = 2^-7
    e = ((codes >> 3) & 15).astype(np.int32)
    mnt = (codes & 7).astype(np.float64)
    val = np.where(e == 0, mnt * 2.0 ** -9, (mnt + 8) * 2.0 ** (e - 10.0)) * np.where(codes >> 7, -1.0, 1.0)
    Wf = (val * 2.0 ** -7).astype(np.float32)
    o3, _ = qz.quantize_group_h([pkg.LinearIn("w", 32, w_fp8=codes, scale_bf16=sc)], n, H, 3, pkg.QuantOpts(skip_proxy=True))
    o4, _ = qz.quantize_group_h([pkg.LinearIn("w", 32, w_f32=Wf)], n, H, 3, pkg.QuantOpts(skip_proxy=True))
    assert np.array_equal(o3[0].trellis, o4[0].trellis) and o3[0].wscale == o4[0].wscale
    # errors
    with pytest.raises(pkg.QtipError):
        qz.quantize_group_h([pkg.LinearIn("w", 32, w_f32=W)], n, H, 3, pkg.QuantOpts(share_su=False))
    with pytest.raises(pkg.QtipError) as e:
        qz.quantize_group_h([pkg.LinearIn("w", 16, w_f32=W[:16])], n, H, 3)          # m % 32
    assert e.value.code == pkg.QTIP_E_ARG
    with pytest.raises(pkg.QtipError) as e:
        qz.quantize_group_h([pkg.LinearIn("w", 32, w_f32=W[:, :192])], 192, H[:192, :192].copy(), 3)   # n % 128
    assert e.value.code == pkg.QTIP_E_ARG
    G = rng.standard_normal((n, 8)).astype(np.float32)
    with pytest.raises(pkg.QtipError) as e:                                          # rank 8, no damping: not PD
        qz.quantize_group_h([pkg.LinearIn("w", 32, w_f32=W)], n, G @ G.T, 3, pkg.QuantOpts(sigma_reg=0.0))
    assert e.value.code == pkg.QTIP_E_NOT_PD


def test_group_config2(qz, oracle, pkg, hyb, synth):
    """Benchmark configuration 2 (1024 x 1024, AR(1) Hessian with outlier channels): code agreement >= 99 % and proxy
    within 1 % relative of the CPU restatement (north-star accuracy targets for full LDLQ groups)."""
    say("case: config 2, 1024x1024")
    qz.set_tlut(None)
    Ws, H = synth.config2()
    n = 1024
    outs, tm = qz.quantize_group_h([pkg.LinearIn("w", n, w_f32=Ws[0])], n, H, 11, pkg.QuantOpts(ldl_threads=16))
    ref = oracle.quantize_group(hyb.tlut, Ws, H, 11)
    lo = outs[0]
    got = pkg.unswizzle_for_kernel(lo.trellis, n, n).reshape(-1, 32)
    want = pkg.unswizzle_for_kernel(ref["trellis"], n, n).reshape(-1, 32)
    agree = np.all(got == want, axis=1).mean()
    rel = abs(lo.proxy - ref["proxy"][0]) / ref["proxy"][0]
    say("  code agreement %.4f, proxy gpu %.6f cpu %.6f (rel %.2e), Wscale %.6f/%.6f, ldlq %.2fs viterbi %.2fs" %
        (agree, lo.proxy, ref["proxy"][0], rel, lo.wscale, ref["wscale"][0], tm.ldlq, tm.viterbi))
    assert agree >= 0.99
    assert rel < 0.01
    assert lo.wscale == ref["wscale"][0]
    # the same group with the reference GPU's arithmetic (fp32 feedback, split-bf16 prod cache): reported, and held
    # to the proxy bar only -- one flipped fp16 rounding changes every later tile of its tile row
    outs1, _ = qz.quantize_group_h([pkg.LinearIn("w", n, w_f32=Ws[0])], n, H, 11, pkg.QuantOpts(ldl_threads=16, feedback=1))
    got1 = pkg.unswizzle_for_kernel(outs1[0].trellis, n, n).reshape(-1, 32)
    agree1 = np.all(got1 == want, axis=1).mean()
    rel1 = abs(outs1[0].proxy - ref["proxy"][0]) / ref["proxy"][0]
    say("  feedback=1: code agreement %.4f, proxy %.6f (rel %.2e)" % (agree1, outs1[0].proxy, rel1))
    assert rel1 < 0.01


def test_run_groups_lanes_give_the_same_results(qz, pkg, synth):
    """Small groups run side by side on lanes (qtip_opts.group_lanes): seven groups of four shapes through one lane
    (the reference's schedule, src/pipeline.cpp:229-312), two, three and the automatic number give the same words,
    scales and proxy errors; a lane that gets several groups pipelines them; a new tlut reaches the lanes."""
    say("case: run_groups lanes")
    qz.set_tlut(None)
    cases, shapes = [], []
    for g, (n, ms) in enumerate([(256, (64, 32)), (512, (32,)), (256, (32,)), (1024, (64, 64)), (512, (32, 64)),
                                 (256, (32,)), (1024, (128,))]):
        Ws, H = synth.small_group(seed=70 + g, n=n, ms=ms)
        lins = [pkg.LinearIn("g%d_%d" % (g, k), w.shape[0], w_f32=w) for k, w in enumerate(Ws)]
        if g == 2:   # one group with bf16 weights, one with feedback through the other arithmetic below
            wb = (Ws[0].view(np.uint32) >> 16).astype(np.uint16)
            lins = [pkg.LinearIn("g2_0", Ws[0].shape[0], w_bf16=wb)]
        cases.append((lins, n, H, 200 + g))
        shapes.append((ms, n))
    # an eighth group with fp8 weights and a per-row scale: with one lane the side thread that uploads host inputs
    # takes every format through its four staging slots twice over
    rng8 = np.random.default_rng(8)
    codes = rng8.integers(0, 256, (64, 512)).astype(np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x30        # no NaN codes
    _, H8 = synth.small_group(seed=78, n=512, ms=(64,))
    cases.append(([pkg.LinearIn("g7_0", 64, w_fp8=codes, scale_bf16=np.full(64, 0x3c00, np.uint16))], 512, H8, 207))
    shapes.append(((64,), 512))
    assert qz.group_lanes(shapes) == 8            # 8 tile rows at most: all of them side by side
    assert qz.group_lanes(shapes, pkg.QuantOpts(group_lanes=1)) == 1
    assert qz.group_lanes(shapes, pkg.QuantOpts(group_lanes=3)) == 3
    assert qz.group_lanes([((12288,), 28672)] * 4) == 1

    def same(ra, rb):
        for (oa, ta, _), (ob, _, _) in zip(ra, rb):
            for a, b in zip(oa, ob):
                assert a.name == b.name
                assert np.array_equal(a.trellis, b.trellis) and np.array_equal(a.sv, b.sv)
                assert np.array_equal(a.su_bf16, b.su_bf16)
                assert a.wscale == b.wscale and a.proxy == b.proxy and a.proxy_rot_reg == b.proxy_rot_reg
            assert ta.total > 0 and ta.ldl_cpu > 0

    one = qz.run_groups(cases, pkg.QuantOpts(ldl_threads=8, group_lanes=1))
    for lanes in (2, 3, 0):
        say("  lanes %d" % lanes)
        same(qz.run_groups(cases, pkg.QuantOpts(ldl_threads=8, group_lanes=lanes)), one)
    same(qz.run_groups(cases, pkg.QuantOpts(ldl_threads=8, group_lanes=3, ldl_device_updates=False)), one)
    same(qz.run_groups(cases, pkg.QuantOpts(ldl_threads=8, group_lanes=4, feedback=1)),
         qz.run_groups(cases, pkg.QuantOpts(ldl_threads=8, group_lanes=1, feedback=1)))
    # the lanes keep their device buffers between calls: a second call of the same shape allocates nothing
    import torch
    torch.cuda.synchronize()
    free1 = torch.cuda.mem_get_info()[0]
    same(qz.run_groups(cases, pkg.QuantOpts(ldl_threads=8, group_lanes=3, ldl_device_updates=False)), one)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] >= free1 - (1 << 20)
    # a codebook set after the lanes exist
    rng = np.random.default_rng(9)
    tl = (rng.standard_normal((512, 2)) * 0.9).astype(np.float32)
    qz.set_tlut(tl)
    try:
        a = qz.run_groups(cases[:4], pkg.QuantOpts(ldl_threads=8, group_lanes=4))
        b = qz.run_groups(cases[:4], pkg.QuantOpts(ldl_threads=8, group_lanes=1))
        same(a, b)
        assert not np.array_equal(a[0][0][0].trellis, one[0][0][0].trellis)
    finally:
        qz.set_tlut(None)
    with pytest.raises(pkg.QtipError):
        qz.run_groups(cases, pkg.QuantOpts(group_lanes=13))
    # mixed sizes: a group that fills the chip runs through the overlapped schedule, the small ones on lanes
    say("  lanes, mixed sizes")
    Ws, H = synth.small_group(seed=99, n=256, ms=(8192, 4096))
    wide = ([pkg.LinearIn("wide%d" % k, w.shape[0], w_f32=w) for k, w in enumerate(Ws)], 256, H, 400)
    mixed = [cases[0], wide, cases[2], cases[5]]
    same(qz.run_groups(mixed, pkg.QuantOpts(ldl_threads=8)), qz.run_groups(mixed, pkg.QuantOpts(ldl_threads=8, group_lanes=1)))
    # groups of 384 tile rows: two lanes of one LDLQ chain each against one lane that deals the rows to two chains
    say("  lanes, 6144 x 512 groups")
    big = []
    for g in range(3):
        Ws, H = synth.small_group(seed=90 + g, n=512, ms=(4096, 2048))
        big.append(([pkg.LinearIn("b%d_%d" % (g, k), w.shape[0], w_f32=w) for k, w in enumerate(Ws)], 512, H, 300 + g))
    assert qz.group_lanes([((4096, 2048), 512)] * 3) == 2
    same(qz.run_groups(big, pkg.QuantOpts(ldl_threads=8)), qz.run_groups(big, pkg.QuantOpts(ldl_threads=8, group_lanes=1)))


def test_run_groups_equals_group_by_group(qz, oracle, pkg, synth):
    """The overlapped scheduler (run_qtip_groups, src/pipeline.cpp:229-312) returns, for five groups of three
    different widths through its ring of three staging buffers, exactly what quantize_group returns one at a time;
    a Hessian that is not positive definite stops it with the LDL's error code after the groups before it."""
    say("case: run_groups, 5 groups")
    qz.set_tlut(None)
    cases = []
    for g, (n, ms) in enumerate([(256, (64, 32)), (512, (32,)), (256, (32,)), (1024, (64,)), (512, (32, 64))]):
        Ws, H = synth.small_group(seed=50 + g, n=n, ms=ms)
        lins = [pkg.LinearIn("g%d_%d" % (g, k), w.shape[0], w_f32=w) for k, w in enumerate(Ws)]
        cases.append((lins, n, H, 100 + g))
    opt = pkg.QuantOpts(ldl_threads=8)
    res = qz.run_groups(cases, opt)
    assert len(res) == len(cases)
    for (lins, n, H, seed), (outs, tm, wait) in zip(cases, res):
        one, _ = qz.quantize_group_h(lins, n, H, seed, opt)
        for a, b in zip(outs, one):
            assert a.name == b.name and a.m == b.m and a.n == n
            assert np.array_equal(a.trellis, b.trellis) and np.array_equal(a.sv, b.sv)
            assert np.array_equal(a.su_bf16, b.su_bf16)
            assert a.wscale == b.wscale and a.proxy == b.proxy and a.proxy_rot_reg == b.proxy_rot_reg
        assert tm.total > 0 and tm.ldl_cpu > 0 and tm.rht > 0 and wait >= 0
    assert qz.run_groups([], opt) == []
    # the same with the factorization on the host alone (the reference's form): identical outputs
    host = qz.run_groups(cases, pkg.QuantOpts(ldl_threads=8, ldl_device_updates=False))
    for (outs, _, _), (houts, htm, _) in zip(res, host):
        for a, b in zip(outs, houts):
            assert np.array_equal(a.trellis, b.trellis) and a.wscale == b.wscale
            assert a.proxy == b.proxy and a.proxy_rot_reg == b.proxy_rot_reg
        assert htm.ldl_cpu > 0
    # failure in the third of four groups
    rng = np.random.default_rng(1)
    G = rng.standard_normal((256, 8)).astype(np.float32)
    bad = list(cases[:2]) + [(cases[2][0], 256, G @ G.T, 5), cases[3]]
    for dev in (True, False):
        with pytest.raises(pkg.QtipError) as e:
            qz.run_groups(bad, pkg.QuantOpts(ldl_threads=8, sigma_reg=0.0, ldl_device_updates=dev))
        assert e.value.code == pkg.QTIP_E_NOT_PD
    # the context is still usable
    again = qz.run_groups(cases[:1], opt)
    assert np.array_equal(again[0][0][0].trellis, res[0][0][0].trellis)
