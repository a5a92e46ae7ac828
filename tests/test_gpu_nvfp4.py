"""GPU parity of the NVFP4 fallback quantizer through the C ABI: the device block loop (scale search, calibrated
rounding) against the oracle's CPU restatement of the same formulas, byte for byte, and the criteria of the
reference's own test (tests/test_nvfp4.cpp:59-105)."""
import numpy as np
import pytest

from test_oracle_nvfp4 import _hessian, _weights, device_path_vectors

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)


@pytest.mark.parametrize("name", ["gauss", "heavy"])
def test_block_loop_bytes_equal_the_cpu_restatement(qz, pkg, oracle, name):
    say("case: nvfp4 block loop %s" % name)
    w, _ = _weights(oracle, name)
    m, n = w.shape
    H = _hessian(oracle, n, 21)
    L, D = oracle.nvfp4_prepare(H, 1e-2, True)
    _, dH = oracle.nvfp4_prepare(H, 1e-2, False)
    g = oracle.nvfp4_quantize(w)[2]
    for (Lx, dx, search) in ((None, None, False), (None, None, True), (None, dH, True), (L, D, False), (L, D, True)):
        t = qz.nvfp4_quantize_prepared([w], n, Lx, dx, search)[0]
        want = oracle.nvfp4_blocks(w, Lx, dx, g, Lx is not None, search)
        assert t.global_scale == g
        assert np.array_equal(t.packed, want[0]) and np.array_equal(t.scales, want[1]), (Lx is not None, dx is not None, search)
    # upgrades off: the plain host quantizer, byte for byte (tests/test_nvfp4.cpp:64-67)
    plain = pkg.nvfp4_quantize(w)
    off = qz.nvfp4_quantize_group([w], n, None, scale_search=False, calibrate=False)[0][0]
    assert np.array_equal(off.packed, plain.packed) and np.array_equal(off.scales, plain.scales)
    assert off.global_scale == plain.global_scale


@pytest.mark.parametrize("name", ["gauss", "heavy"])
def test_group_meets_the_reference_test_criteria(qz, pkg, oracle, name):
    say("case: nvfp4 group %s" % name)
    w, _ = _weights(oracle, name)
    m, n = w.shape
    H = _hessian(oracle, n, 21)
    naive = pkg.nvfp4_quantize(w)
    dq = pkg.nvfp4_dequantize
    (cal,), used = qz.nvfp4_quantize_group([w], n, H)
    assert used
    (search_h,), used2 = qz.nvfp4_quantize_group([w], n, H, calibrate=False)
    assert not used2
    (search_plain,), _ = qz.nvfp4_quantize_group([w], n, None, calibrate=False)
    (cal_only,), _ = qz.nvfp4_quantize_group([w], n, H, scale_search=False)
    pe = oracle.nvfp4_proxy_error
    p_naive, p_search, p_cal, p_cal_only = pe(w, dq(naive), H), pe(w, dq(search_h), H), pe(w, dq(cal), H), pe(w, dq(cal_only), H)
    say("  proxy: naive %.4g  search %.4g  calibrated+search %.4g (%.1f%% of naive)  calibrated only %.4g" %
        (p_naive, p_search, p_cal, 100 * p_cal / p_naive, p_cal_only))
    assert pe(w, dq(search_plain)) <= pe(w, dq(naive)) * (1 + 1e-9)
    assert p_search <= p_naive * 1.02 and p_cal < 0.9 * p_naive and p_cal_only <= p_naive
    for t in (cal, search_h, search_plain, cal_only):
        assert t.packed.shape == naive.packed.shape and t.global_scale == naive.global_scale
        assert np.all((t.scales & 0x7f) <= 126) and np.all(np.isfinite(dq(t)))
    # the library's own factor differs from the oracle's in the last bits at most: nearly all bytes agree
    L, D = oracle.nvfp4_prepare(H, 1e-2, True)
    want = oracle.nvfp4_blocks(w, L, D, naive.global_scale, True, True)
    assert np.mean(cal.packed == want[0]) > 0.98
    # a group of two matrices equals two single calls
    grp, _ = qz.nvfp4_quantize_group([w, w[:32]], n, H)
    (single2,), _ = qz.nvfp4_quantize_group([w[:32]], n, H)
    assert np.array_equal(grp[0].packed, cal.packed) and np.array_equal(grp[0].scales, cal.scales)
    assert np.array_equal(grp[1].packed, single2.packed) and np.array_equal(grp[1].scales, single2.scales)


@pytest.mark.parametrize("name", ["gauss", "heavy"])
def test_group_bytes_equal_the_golden_device_path_vectors(qz, oracle, name):
    """The committed bytes of the reference's device path (tests/golden/ref_nvfp4_gpu_*), all option combinations."""
    say("case: nvfp4 group vs golden device-path vectors, %s" % name)
    w, _ = _weights(oracle, name)
    H, cases, g = device_path_vectors(name)
    for (h, s, c, pk, sc) in cases:
        (t,), used = qz.nvfp4_quantize_group([w], 256, H if h else None, scale_search=s, calibrate=c)
        assert used == (h and c) and t.global_scale == g
        assert np.array_equal(t.packed, pk) and np.array_equal(t.scales, sc), (h, s, c)


@pytest.mark.parametrize("name", ["gauss", "heavy"])
def test_group_bytes_equal_the_reference_device_path(qz, oracle, name):
    """The reference's own nvfp4_quantize_group, compiled for this GPU from its sources (oracle/_ref), on the same
    inputs: every packed byte, scale code and global scale of every option combination."""
    assert oracle.ref_gpu_lib() is not None, "oracle/_ref/libqtip_ref_gpu.so is missing: build it with make -C oracle ref"
    say("case: nvfp4 group vs the compiled reference, %s" % name)
    w, _ = _weights(oracle, name)
    m, n = w.shape
    H = _hessian(oracle, n, 21)
    for (Hx, search, cal) in ((None, False, False), (None, True, True), (H, True, False), (H, False, True), (H, True, True)):
        got, used = qz.nvfp4_quantize_group([w, w[:32]], n, Hx, scale_search=search, calibrate=cal)
        want, used_ref = oracle.ref_gpu_nvfp4_quantize_group([w, w[:32]], n, Hx, scale_search=search, calibrate=cal)
        assert used == used_ref
        for t, (pk, sc, g) in zip(got, want):
            agree = float(np.mean(t.packed == pk))
            say("  H %s search %d calibrate %d: packed bytes equal %.4f%%, scales equal %.4f%%" %
                (Hx is not None, search, cal, 100 * agree, 100 * float(np.mean(t.scales == sc))))
            assert t.global_scale == g
            assert np.array_equal(t.scales, sc) and np.array_equal(t.packed, pk)


@pytest.mark.parametrize("n", [272, 1040, 2560])
def test_prepare_with_device_updates_equals_host_prepare(qz, pkg, n):
    """The calibration's factor with the trailing updates of its Cholesky factorization on the GPU (one panel, a ragged
    last panel, ten panels): L and dw equal the host preparation's bit for bit; a Hessian that is not positive definite
    is refused with the same code; the group call gives the same bytes either way."""
    say("case: nvfp4 prepare, device updates, n = %d" % n)
    rng = np.random.default_rng(n)
    X = rng.standard_normal((2 * n, n)).astype(np.float32) * np.exp(0.8 * rng.standard_normal(n)).astype(np.float32)
    H = np.ascontiguousarray(X.T @ X / (2 * n), np.float32)
    H[3, 7] += 1e-3      # not exactly symmetric: the preparation takes the mean of the two triangles
    L0, dw0 = pkg.nvfp4_prepare(H, 1e-2, True, 5)
    L1, dw1 = qz.nvfp4_prepare_device_updates(H, 1e-2, 7)
    assert np.array_equal(L0.view(np.uint32), L1.view(np.uint32))
    assert np.array_equal(dw0.view(np.uint32), dw1.view(np.uint32))
    assert np.all(np.triu(L1) == 0)
    bad = H.copy()
    bad[n // 2, n // 2] = -10.0
    with pytest.raises(pkg.QtipError) as e:
        qz.nvfp4_prepare_device_updates(bad, 1e-2, 7)
    assert e.value.code == pkg.QTIP_E_NOT_PD
    if n == 272:
        w = (rng.standard_normal((64, n)) * 0.02).astype(np.float32)
        (a,), ua = qz.nvfp4_quantize_group([w], n, H)
        (b,), ub = qz.nvfp4_quantize_group([w], n, H, factor_on_host=True)
        assert ua and ub and np.array_equal(a.packed, b.packed) and np.array_equal(a.scales, b.scales)


def test_nvfp4_layer_shape(qz, pkg, oracle):
    """A 4096 x 4096 matrix with a dense Hessian: calibrated result beats the plain quantizer in the proxy (fp64 on the
    device), format valid; prints the time."""
    import time
    import torch
    say("case: nvfp4 4096x4096")
    m = n = 4096
    g = torch.Generator(device="cuda").manual_seed(3)
    w = (torch.randn((m, n), generator=g, device="cuda") * 0.02).cpu().numpy()
    X = torch.randn((8192, n), generator=g, device="cuda") * torch.exp(0.8 * torch.randn((n,), generator=g, device="cuda"))
    Hd = (X.T @ X / 8192).double()
    H = Hd.float().cpu().numpy()
    t0 = time.time()
    (cal,), used = qz.nvfp4_quantize_group([w], n, H)
    dt = time.time() - t0
    plain = pkg.nvfp4_quantize(w)

    def proxy(t):
        E = torch.from_numpy(w - pkg.nvfp4_dequantize(t)).cuda().double()
        return float(((E @ Hd) * E).sum() / m)

    p_cal, p_plain = proxy(cal), proxy(plain)
    say("  %.2f s; proxy calibrated %.4g, plain %.4g (%.1f%%)" % (dt, p_cal, p_plain, 100 * p_cal / p_plain))
    assert used and p_cal < 0.9 * p_plain and np.all((cal.scales & 0x7f) <= 126)
    if oracle.ref_gpu_lib() is not None and oracle.ref_lib() is not None:
        # 16.8 M weights x 11 candidates: a multiply-add rounded differently anywhere in the block loop shows here.
        # Byte equality is asked with the factor from the reference's own Cholesky; the library's factor differs from
        # it in the last bit of a few entries, so the group call is held to 99.999 %.
        t0 = time.time()
        ((pk, sc, gl),), _ = oracle.ref_gpu_nvfp4_quantize_group([w], n, H)
        t1 = time.time()
        L, dw = oracle.ref_nvfp4_prepare(H)
        same_l = qz.nvfp4_quantize_prepared([w], n, L, dw, True)[0]
        say("  compiled reference: %.2f s; group call: packed bytes equal %.5f%%, scales %.5f%%; with its factor: %d differ" %
            (t1 - t0, 100 * float(np.mean(cal.packed == pk)), 100 * float(np.mean(cal.scales == sc)),
             int((same_l.packed != pk).sum() + (same_l.scales != sc).sum())))
        assert gl == cal.global_scale and np.array_equal(same_l.scales, sc) and np.array_equal(same_l.packed, pk)
        assert np.mean(cal.packed == pk) > 0.99999 and np.mean(cal.scales == sc) > 0.99999


def test_nvfp4_config5_shape(qz, pkg):
    """12288 x 28672 with a dense 28672^2 Hessian (the down-proj shape of the headline configuration): host
    preparation and device block loop timed apart; format valid, Hessian-weighted error below the plain quantizer's."""
    import time
    import torch
    say("case: nvfp4 12288x28672")
    m, n = 12288, 28672
    g = torch.Generator(device="cuda").manual_seed(4)
    wd = torch.randn((m, n), generator=g, device="cuda") * 0.02
    X = torch.randn((8192, n), generator=g, device="cuda") * torch.exp(0.8 * torch.randn((n,), generator=g, device="cuda"))
    Hd = X.T @ X / 8192
    del X
    w, H = wd.cpu().numpy(), Hd.cpu().numpy()
    t0 = time.time()
    L, dw = pkg.nvfp4_prepare(H, 1e-2, True, 16)
    t1 = time.time()
    cal = qz.nvfp4_quantize_prepared([w], n, L, dw, True)[0]
    t2 = time.time()
    Ld, dwd = qz.nvfp4_prepare_device_updates(H, 1e-2, 16)
    t3 = time.time()
    say("  preparation %.2f s on the host, %.2f s with the updates on the GPU; block loop %.2f s (%.0f Mweights/s)" %
        (t1 - t0, t3 - t2, t2 - t1, m * n / (t2 - t1) / 1e6))
    assert np.array_equal(Ld.view(np.uint32), L.view(np.uint32)) and np.array_equal(dwd.view(np.uint32), dw.view(np.uint32))
    del L, Ld
    plain = pkg.nvfp4_quantize(w)
    assert cal.global_scale == plain.global_scale and np.all((cal.scales & 0x7f) <= 126)

    def proxy(t):
        E = wd - torch.from_numpy(pkg.nvfp4_dequantize(t)).cuda()
        tot = 0.0
        for r0 in range(0, m, 2048):          # fp32 GEMM slabs, fp64 sums: a comparison of two numbers 2.5x apart
            e = E[r0:r0 + 2048]
            tot += float(((e @ Hd) * e).double().sum())
        return tot / m

    p_cal, p_plain = proxy(cal), proxy(plain)
    say("  proxy calibrated %.4g, plain %.4g (%.1f%%)" % (p_cal, p_plain, 100 * p_cal / p_plain))
    assert p_cal < 0.9 * p_plain
