"""Full-size checks (benchmark configurations 3, 4 and 5) of the GPU group path: agreement with the CPU form on a row
subset of the rotated weights (LDLQ is row-independent given L), and size-independent properties of the packed
output (every trellis tail-biting and link-consistent, decode(states) == hatW on sampled tiles)."""
import os

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


def check_trellis_paths(st):
    st = st.astype(np.uint32)
    assert np.all((st[:, 127] & 0xfff) == (st[:, 0] >> 4)), "tail-biting"
    assert np.all(((st[:, :-1] << 4) & 0xffff) == (st[:, 1:] & 0xfff0)), "trellis links"


def reference_factor(oracle, HRr, threads=16):
    """L of the rotated Hessian from the REFERENCE's own block_ldl_to_L (its CPU core compiled into oracle/_ref),
    after the symmetrization of its ldl_hessian (src/quantizer.cpp:154-165).  A missing library is a failure here,
    not a skip: these tests are what ties the full-depth chains to the reference's factor."""
    R = oracle.ref_lib()
    assert R is not None, "oracle/_ref/libqtip_ref.so is missing: build it with make -C oracle ref"
    n = HRr.shape[0]
    A = np.empty((n, n), np.float64)
    blk = 2048
    for i in range(0, n, blk):                                   # 0.5 * (H + H^T), a row block at a time
        A[i:i + blk] = 0.5 * (HRr[i:i + blk].astype(np.float64) + HRr[:, i:i + blk].T.astype(np.float64))
    L = np.zeros((n, n), np.float32)
    assert R.ref_block_ldl(A.reshape(-1), n, L.reshape(-1), threads) == 1
    return L


def agreement_by_depth(same, nblk, label):
    """same: (tile rows, n / 16) booleans, column block 0 first.  LDLQ walks from the last column block to the first,
    so depth octile 0 is the right-most eighth of the columns.  Prints the share of identical trellises per octile."""
    by_depth = same[:, ::-1]
    parts = np.array_split(np.arange(nblk), 8)
    shares = [float(by_depth[:, p].mean()) for p in parts]
    say("  %s: identical trellises per depth octile (first quantized -> last): %s"
        % (label, " ".join("%.4f" % v for v in shares)))
    return shares


def test_config3_group_rows_against_reference_chain(qz, pkg, oracle, hyb, synth):
    """Configuration 3 on its own inputs (12288 x 12288, 1 % of the weights x 10, 32 outlier channels) through the group
    call, whose factor comes from the library's default LDL (host panels, trailing updates on the GPU).  The reference
    chain beside it: block_ldl_to_L of the compiled reference on the same rotated Hessian, then the CPU LDLQ on three
    tile rows.  The two factors must be the same 32-bit words and the codes of those rows identical (>= 99 % is the
    bar) over all 768 column blocks.  Three LDLQ chains are asked for and one tile row of each chain's share is compared."""
    import torch
    say("case: config 3 through the group call (three chains), 48 rows against reference LDL + CPU LDLQ")
    qz.set_tlut(None)
    Ws, H = synth.large_config(3)
    n, m = H.shape[0], Ws[0].shape[0]
    seed = 11
    hp = qz.rotate_hessian(H, n, seed)
    del H
    L_ref = reference_factor(oracle, hp.HRr)
    qz.ldl_hessian_device_updates(hp, threads=16)
    diff = int(np.count_nonzero(hp.L.view(np.uint32) != L_ref.view(np.uint32)))
    say("  words of L differing from the reference's factor: %d of %d" % (diff, L_ref.size))
    assert diff == 0
    outs, tm = qz.quantize_group([pkg.LinearIn("q", m, w_f32=Ws[0])], hp, pkg.QuantOpts(ldl_threads=16, ldlq_chains=3))
    lo = outs[0]
    say("  ldlq %.1fs viterbi %.1fs (%.1f Mweights/s) proxy %.5f wscale %.6f"
        % (tm.ldlq, tm.viterbi, m * n / tm.viterbi / 1e6, lo.proxy, lo.wscale))
    assert 0 < lo.proxy < 0.2 and 0 < lo.proxy_rot_reg < 0.2
    st = pkg.unpack_trellis(pkg.unswizzle_for_kernel(lo.trellis, m, n))
    check_trellis_paths(st)
    su, sv = pkg.sign_vector(seed, n), pkg.sign_vector(seed * 1000003 + 1, m)
    assert np.array_equal(hp.su, su) and np.array_equal(lo.sv, sv)
    # Wr^T = U^T_m (U^T_n (diag(SV) W diag(SU)))^T with the library's transform (pinned bit for bit elsewhere), then
    # the fp32 multiplication by 1 / Wscale
    A = Ws[0] * torch.from_numpy(sv).cuda()[:, None] * torch.from_numpy(su).cuda()[None, :]
    torch.cuda.synchronize()
    qz.hadamard_rows_dev(A, m, n, n, True)
    qz.synchronize()
    AT = A.T.contiguous()
    del A
    torch.cuda.synchronize()
    qz.hadamard_rows_dev(AT, n, m, m, True)
    qz.synchronize()
    rows = np.r_[0:16, 6400:6416, 11200:11216]                   # tile rows 0, 400, 700: one from each of the three chains
    sub = (AT[:, torch.from_numpy(rows).cuda()] * float(np.float32(1.0) / np.float32(lo.wscale))).T.contiguous().cpu().numpy()
    del AT
    hat_o, Q_o = oracle.ldlq(hyb, sub, L_ref, threads=16)
    Q_g = st.reshape(m // 16, n // 16, 128)[[0, 400, 700]].reshape(-1, 128)
    same = np.all(Q_g == Q_o, axis=1).reshape(3, n // 16)
    agreement_by_depth(same, n // 16, "config 3")
    say("  identical trellises: %d of %d" % (int(same.sum()), same.size))
    assert same.mean() >= 0.99


def test_config5_group_properties(qz, pkg, oracle, synth):
    """The headline shape end to end (12288 x 28672, rank-deficient damped Hessian): every one of the 1 376 256
    trellises is a valid tail-biting path, the reconstruction error is sane, SU/SV reproduce from the seed, and a
    sample of tiles decodes consistently through the kernel layout."""
    import torch
    say("case: config 5 group, properties at full size")
    qz.set_tlut(None)
    Ws, H = synth.large_config(5)
    n, m = H.shape[0], Ws[0].shape[0]
    outs, tm = qz.quantize_group_h([pkg.LinearIn("down", m, w_f32=Ws[0])], n, H, 3, pkg.QuantOpts(ldl_threads=16))
    lo = outs[0]
    say("  proxy %.5f rot_reg %.5f wscale %.6f; ldl %.1fs ldlq %.1fs viterbi %.1fs proxy %.1fs" %
        (lo.proxy, lo.proxy_rot_reg, lo.wscale, tm.ldl_cpu, tm.ldlq, tm.viterbi, tm.proxy))
    assert lo.trellis.size == (m // 16) * (n // 16) * 32
    assert 0 < lo.proxy < 0.2 and 0 < lo.proxy_rot_reg < 0.2 and lo.wscale > 0
    assert np.array_equal(lo.sv, pkg.sign_vector(3 * 1000003 + 1, m))
    su = (lo.su_bf16.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(su, pkg.sign_vector(3, n))
    st = pkg.unpack_trellis(pkg.unswizzle_for_kernel(lo.trellis, m, n))
    check_trellis_paths(st)
    # states are not degenerate: all 16 new-bit values occur about equally often
    hist = np.bincount((st[::97].reshape(-1) & 15).astype(np.int64), minlength=16) / st[::97].size
    assert hist.min() > 0.04 and hist.max() < 0.09


def rotated_scaled_rows(qz, W, sv, su, wscale, rows):
    """Rows `rows` of Wr / Wscale: Wr^T = U^T_m (U^T_n (diag(SV) W diag(SU)))^T with the library's transform (pinned bit for
    bit elsewhere), then the fp32 multiplication by 1 / Wscale.  W: m x n device tensor.  Returns a host array."""
    import torch
    m, n = W.shape
    A = W * torch.from_numpy(sv).cuda()[:, None] * torch.from_numpy(su).cuda()[None, :]
    torch.cuda.synchronize()                                     # the library works on a stream of its own
    qz.hadamard_rows_dev(A, m, n, n, True)
    qz.synchronize()
    AT = A.T.contiguous()
    del A
    torch.cuda.synchronize()
    qz.hadamard_rows_dev(AT, n, m, m, True)
    qz.synchronize()
    sub = (AT[:, torch.from_numpy(rows).cuda()] * float(np.float32(1.0) / np.float32(wscale))).T.contiguous()
    return sub.cpu().numpy(), AT


def test_config5_timed_path_rows_against_reference_chain(qz, pkg, oracle, hyb, synth):
    """The path the benchmark times, at its own size: two 12288 x 28672 groups through qtip_run_groups with W and H
    handed over as host pointers (loader thread, staging slots), the LDL's trailing updates on the GPU and the factor
    resident on the device (ring), three LDLQ chains (each with its own split-K gather sums and share of the
    kept-metrics slots).  n = 28672 is the headline depth: a tile row is a chain of 1792 tiles, each depending on every
    later column.  Of the second group, one tile row from each chain's share is compared with the reference chain -
    block_ldl_to_L of the compiled reference on the same rotated Hessian, then the CPU LDLQ on those rows - per depth
    octile (>= 99 % is the bar); the library's own factor must equal the reference's in every 32-bit word, and the
    reported proxy errors must agree with an fp64 recomputation over the whole group."""
    import torch
    say("case: config 5 through run_groups (host inputs, device-updated LDL, three chains), rows against the reference chain")
    qz.set_tlut(None)
    Ws, H = synth.large_config(5)
    n, m = H.shape[0], Ws[0].shape[0]
    Wh, Hh = Ws[0].cpu().numpy(), H.cpu().numpy()
    opt = pkg.QuantOpts(ldl_threads=16, ldl_device_updates=True, ldlq_chains=3, group_lanes=1)
    seeds = (21, 22)
    res = qz.run_groups([([pkg.LinearIn("down", m, w_f32=Wh)], n, Hh, sd) for sd in seeds], opt)
    (outs, tm, wait) = res[1]
    lo, seed = outs[0], seeds[1]
    say("  second group: ldlq %.2fs viterbi %.2fs (%.1f Mweights/s) ldl wait %.3fs proxy %.6f rot_reg %.6f wscale %.6f; "
        "passes repeated on fp64 metrics: %s" % (tm.ldlq, tm.viterbi, m * n / tm.viterbi / 1e6, wait, lo.proxy,
                                                  lo.proxy_rot_reg, lo.wscale, qz.viterbi_stats()))
    st = pkg.unpack_trellis(pkg.unswizzle_for_kernel(lo.trellis, m, n))
    check_trellis_paths(st)
    su, sv = pkg.sign_vector(seed, n), pkg.sign_vector(seed * 1000003 + 1, m)
    assert np.array_equal((lo.su_bf16.astype(np.uint32) << 16).view(np.float32), su) and np.array_equal(lo.sv, sv)
    # the reference chain's factor, and the library's own (as run_groups forms it) word for word
    hp = qz.rotate_hessian(H, n, seed)
    del H, Hh
    qz.ldl_hessian_device_updates(hp, threads=16)
    say("  own factor done; reference block_ldl_to_L on 16 threads ...")
    L_ref = reference_factor(oracle, hp.HRr)
    diff = int(np.count_nonzero(hp.L.view(np.uint32) != L_ref.view(np.uint32)))
    say("  words of L differing from the reference's factor: %d of %d" % (diff, L_ref.size))
    assert diff == 0
    hp.L = None
    # one tile row from each chain's share (768 tile rows dealt to three chains: 0..255, 256..511, 512..767)
    tile_rows = [5, 300, 700]
    rows = np.concatenate([np.arange(16 * t, 16 * t + 16) for t in tile_rows])
    sub, AT = rotated_scaled_rows(qz, Ws[0], sv, su, lo.wscale, rows)
    say("  CPU LDLQ on %d rows x %d columns, 16 threads ..." % (len(rows), n))
    hat_o, Q_o = oracle.ldlq(hyb, sub, L_ref, threads=16)
    Q_g = st.reshape(m // 16, n // 16, 128)[tile_rows].reshape(-1, 128)
    same = np.all(Q_g == Q_o, axis=1).reshape(len(tile_rows), n // 16)
    for k, t in enumerate(tile_rows):
        agreement_by_depth(same[k:k + 1], n // 16, "config 5, chain %d (tile row %d)" % (k, t))
    say("  identical trellises: %d of %d" % (int(same.sum()), same.size))
    assert same.mean() >= 0.99
    # proxy errors over the whole group in fp64: D = Wr / Wscale - decode(trellis), num = tr(D HRr D^T), den likewise
    del L_ref
    dT = torch.from_numpy(lo.trellis.view(np.int16)).cuda()
    hatWr = torch.empty((m, n), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    qz.decode_trellis_dev(dT, m, n, hatWr)
    qz.synchronize()
    assert np.array_equal(hatWr[torch.from_numpy(rows).cuda()].cpu().numpy()[same.all(axis=1).repeat(16)],
                          hat_o[same.all(axis=1).repeat(16)])
    Wr = (AT * float(np.float32(1.0) / np.float32(lo.wscale))).T      # m x n view of the scaled rotated weights
    HR = torch.from_numpy(hp.HRr).cuda().double()
    num = den = nd = nw = 0.0
    for r0 in range(0, m, 2048):
        w = Wr[r0:r0 + 2048].double()
        dlt = w - hatWr[r0:r0 + 2048].double()
        num += float(((dlt @ HR) * dlt).sum())
        den += float(((w @ HR) * w).sum())
        nd += float((dlt * dlt).sum())
        nw += float((w * w).sum())
    rot_reg = num / den
    plain = (num - hp.creg * nd) / (den - hp.creg * nw)
    say("  proxy_rot_reg %.8f (fp64 %.8f), proxy %.8f (fp64 %.8f)" % (lo.proxy_rot_reg, rot_reg, lo.proxy, plain))
    assert abs(lo.proxy_rot_reg - rot_reg) <= 1e-3 * rot_reg
    assert abs(lo.proxy - plain) <= 1e-3 * plain


def test_config4_two_linears_shared_hessian_rows_against_cpu(qz, pkg, oracle, hyb, synth):
    """gate + up, two stacked 28672 x 12288 linears sharing one Hessian (one SU, one L, two SV / Wscale): the group
    call at full size, then two tile rows of each linear recomputed by the CPU form from the same rotated, scaled
    rows and the reference's own factor of the same rotated Hessian (which the library's host LDL must equal word for
    word) must give the codes found in that linear's slice of the packed output (>= 99 % is the bar).
    The rotated rows are formed with the library's own transform, which other tests pin bit for bit."""
    import torch
    say("case: config 4 (two linears, shared Hessian) at full size, 64 rows against the CPU form")
    qz.set_tlut(None)
    Ws, H = synth.large_config(4)
    n, m = H.shape[0], Ws[0].shape[0]
    seed = 4
    hp = qz.rotate_hessian(H, n, seed)
    del H
    pkg.Quantizer.ldl_hessian(hp, threads=16)
    L = reference_factor(oracle, hp.HRr)                         # the reference's own factor of the same matrix
    assert np.array_equal(hp.L.view(np.uint32), L.view(np.uint32)), "host LDL differs from the reference's factor"
    lins = [pkg.LinearIn("gate", m, w_f32=Ws[0]), pkg.LinearIn("up", m, w_f32=Ws[1])]
    outs, tm = qz.quantize_group(lins, hp, pkg.QuantOpts(ldl_threads=16))
    say("  ldlq %.1fs viterbi %.1fs (%.1f Mweights/s) proxy %.5f / %.5f wscale %.6f / %.6f" %
        (tm.ldlq, tm.viterbi, 2 * m * n / tm.viterbi / 1e6, outs[0].proxy, outs[1].proxy, outs[0].wscale,
         outs[1].wscale))
    su = pkg.sign_vector(seed, n)
    assert np.array_equal(hp.su, su)
    d_su = torch.from_numpy(su).cuda()
    rows = np.r_[0:16, 17008:17024]                              # tile rows 0 and 1063 of each linear
    d_rows = torch.from_numpy(rows).cuda()
    lut_rms = np.float32(qz.lut_rms)
    for li, lo in enumerate(outs):
        assert np.array_equal((lo.su_bf16.astype(np.uint32) << 16).view(np.float32), su)
        sv = pkg.sign_vector(seed * 1000003 + li + 1, m)
        assert np.array_equal(lo.sv, sv)
        assert 0 < lo.proxy < 0.2 and 0 < lo.proxy_rot_reg < 0.2
        st = pkg.unpack_trellis(pkg.unswizzle_for_kernel(lo.trellis, m, n))
        check_trellis_paths(st)
        # Wr^T = U^T_m (U^T_n (diag(SV) W diag(SU)))^T, then the fp32 multiplication by 1 / Wscale
        A = Ws[li] * torch.from_numpy(sv).cuda()[:, None] * d_su[None, :]
        torch.cuda.synchronize()                                 # the library works on a stream of its own
        qz.hadamard_rows_dev(A, m, n, n, True)
        qz.synchronize()
        AT = A.T.contiguous()
        del A
        torch.cuda.synchronize()
        qz.hadamard_rows_dev(AT, n, m, m, True)
        qz.synchronize()
        rms = float(AT.double().pow(2).mean().sqrt())
        wscale = rms / (float(lut_rms) * 0.9)
        assert abs(wscale - lo.wscale) <= 2e-6 * wscale
        sub = (AT[:, d_rows] * float(np.float32(1.0) / np.float32(lo.wscale))).T.contiguous().cpu().numpy()
        del AT
        hat_o, Q_o = oracle.ldlq(hyb, sub, L, threads=16)
        Q_g = st.reshape(m // 16, n // 16, 128)[[0, 1063]].reshape(-1, 128)
        same = np.all(Q_g == Q_o, axis=1)
        agreement_by_depth(same.reshape(2, n // 16), n // 16, "config 4 linear %d" % li)
        say("  linear %d: identical trellises %d of %d" % (li, int(same.sum()), same.size))
        assert same.mean() >= 0.99
