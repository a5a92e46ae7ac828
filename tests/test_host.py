"""CPU-side checks of the product library: the C ABI exports everything include/qtip_mi355.h declares, and the
host-only entry points (packers, sign streams, Hadamard factor rule, fp64 block LDL) agree with the oracle and
with the golden vectors.  No GPU, no compute call that needs one."""
import ctypes as C
import json
import os
import re

import numpy as np
import pytest

from conftest import GOLDEN, REFVEC, ROOT


def test_abi_exports_every_declared_symbol(pkg):
    hdr = open(os.path.join(ROOT, "include", "qtip_mi355.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    names = sorted(set(re.findall(r"\b(qtip_[a-z0-9_]+)\s*\(", hdr)))
    assert len(names) >= 20
    L = C.CDLL(pkg.LIB_PATH)
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing


def test_failed_device_allocation_is_retried(pkg):
    """A context buffer whose hipMalloc failed must stay empty (n = 0), so that the next ensure() allocates again;
    the failure is simulated on the host, no GPU involved."""
    L = C.CDLL(pkg.LIB_PATH)
    L.qtip_last_error.restype = C.c_char_p
    assert L.qtip_selftest_failed_alloc_is_retried() == 0, L.qtip_last_error()


def test_missing_library_fails_loudly(pkg, monkeypatch):
    monkeypatch.setattr(pkg, "LIB_PATH", os.path.join(ROOT, "nowhere", "libqtip_mi355.so"))
    monkeypatch.setattr(pkg, "_lib", None)
    with pytest.raises(pkg.QtipError):
        pkg.lib()


def test_packers_match_golden_and_oracle(pkg, oracle):
    st = np.fromfile(os.path.join(REFVEC, "pack_states.bin"), np.int32).astype(np.uint16).reshape(-1, 128)
    plain = np.fromfile(os.path.join(REFVEC, "pack_plain.bin"), np.uint16)
    kern = np.fromfile(os.path.join(REFVEC, "pack_kernel.bin"), np.uint16)
    pk = pkg.pack_trellis(st)
    assert np.array_equal(pk.reshape(-1), plain)
    sw = pkg.swizzle_for_kernel(pk, 64, 96)
    assert np.array_equal(sw, kern)
    assert np.array_equal(pkg.unswizzle_for_kernel(sw, 64, 96), plain)
    # unpack needs tail-biting states to round-trip; random words still unpack like the oracle
    rng = np.random.default_rng(0)
    words = rng.integers(0, 65536, (40, 32)).astype(np.uint16)
    assert np.array_equal(pkg.unpack_trellis(words), oracle.unpack_trellis(words))
    assert np.array_equal(pkg.pack_trellis(pkg.unpack_trellis(words)), words)
    big = rng.integers(0, 65536, ((96 // 16) * (160 // 16), 32)).astype(np.uint16)
    assert np.array_equal(pkg.swizzle_for_kernel(big, 96, 160), oracle.swizzle(big, 96, 160))
    with pytest.raises(pkg.QtipError):
        pkg.swizzle_for_kernel(np.zeros(16 * 6 * 32, np.uint16), 16, 96)   # m % 32 != 0


def test_sign_stream_and_had_rule(pkg, oracle):
    want = json.load(open(os.path.join(GOLDEN, "ref_rng.json")))
    for seed in (0, 7):
        assert [int(v) for v in pkg.sign_vector(seed, 64)] == want[str(seed)]["sign"]
    assert np.array_equal(pkg.sign_vector(7 * 1000003 + 2, 500), oracle.rng_sign(7 * 1000003 + 2, 500))
    for n in (1024, 12288, 28672, 96, 3000, 2304, 57344, 100, 7, 8192, 640):
        assert pkg.had_K(n) == oracle.lib().qo_had_K(n)


def _spd(n, seed, rank=None):
    rng = np.random.default_rng(seed)
    G = rng.normal(size=(n, rank or 2 * n))
    return (G @ G.T / G.shape[1]).astype(np.float32)


def test_host_ldl_matches_golden(pkg, oracle):
    H = np.fromfile(os.path.join(REFVEC, "ldl_H.bin"), np.float64).reshape(96, 96)
    Lr = np.fromfile(os.path.join(REFVEC, "ldl_L.bin"), np.float64).reshape(96, 96)
    hp = pkg.HessPrep(n=96, HRr=H.astype(np.float32))
    pkg.Quantizer.ldl_hessian(hp, threads=2)
    # the input is rounded to fp32 here, so compare with the oracle on the same fp32 input and loosely with the vector
    Lo = np.zeros((96, 96), np.float32)
    assert oracle.lib().qo_ldl_hessian(hp.HRr.reshape(-1), 96, Lo.reshape(-1)) == 0
    assert np.max(np.abs(hp.L - Lo)) <= 1e-6 * np.max(np.abs(Lo))
    assert np.max(np.abs(hp.L - Lr)) < 1e-3


@pytest.mark.parametrize("n,threads", [(16, 1), (272, 3), (1024, 8), (1200 // 16 * 16, 5), (2560, 8)])
def test_host_ldl_matches_oracle(pkg, oracle, n, threads):
    """The factor is the reference's bit for bit (the oracle restates its order of operations and is itself pinned to
    the compiled reference and to committed rows); sizes on both sides of the panel width (256) and of the update
    tile (384), not multiples of either."""
    H = _spd(n, n) + 0.05 * np.eye(n, dtype=np.float32)
    H[3, 7] += 1e-3            # asymmetric input: the factorisation works on (H + H^T) / 2
    hp = pkg.HessPrep(n=n, HRr=np.ascontiguousarray(H))
    pkg.Quantizer.ldl_hessian(hp, threads=threads)
    Lo = np.zeros((n, n), np.float32)
    assert oracle.lib().qo_ldl_hessian(hp.HRr.reshape(-1), n, Lo.reshape(-1)) == 0
    assert np.array_equal(hp.L.view(np.uint32), Lo.view(np.uint32)), \
        "%d words of L differ" % np.count_nonzero(hp.L.view(np.uint32) != Lo.view(np.uint32))
    for b in range(n // 16):   # strictly block-lower
        assert np.all(hp.L[16 * b:16 * b + 16, 16 * b:] == 0)


@pytest.mark.parametrize("n,threads", [(16, 1), (272, 3), (528, 8), (800, 5)])
def test_ldl_panel_handover_on_host(pkg, n, threads):
    """The panel hand-over of the device-updated LDL (columns fetched, factored and solved on the host, rows handed
    back, L assembled from the rows as they pass) with a plain host stand-in for the device's trailing matrix: L equals
    the host-only factorization's bit for bit, also with a ragged last panel and a single panel."""
    H = _spd(n, n) + 0.05 * np.eye(n, dtype=np.float32)
    H[2, 5] += 1e-3
    H = np.ascontiguousarray(H)
    hp = pkg.HessPrep(n=n, HRr=H)
    pkg.Quantizer.ldl_hessian(hp, threads=threads)
    L2 = np.full((n, n), -1.0, np.float32)
    assert pkg.lib().qtip_selftest_ldl_panel_handover(H.ctypes.data, n, threads, L2.ctypes.data) == 0
    assert np.array_equal(L2.view(np.uint32), hp.L.view(np.uint32))
    bad = H.copy()
    bad[n // 2, n // 2] = -1.0
    assert pkg.lib().qtip_selftest_ldl_panel_handover(bad.ctypes.data, n, threads, L2.ctypes.data) != 0


def test_group_lane_rule(pkg):
    """qtip_run_groups' lane rule on a chip with 768 Viterbi workgroup slots: groups that fill the chip run one at a
    time, small groups share it, bounded by the slots, the lanes' staging memory, the number of groups and the
    library's maximum; an explicit request is honoured up to the number of groups and refused beyond the maximum."""
    import ctypes as C
    L = pkg.lib()

    def lanes(ng, m, n, req=0, slots=768):
        out = C.c_int(-1)
        rc = L.qtip_selftest_group_lanes(slots, ng, m, n, req, C.byref(out))
        return rc, out.value

    assert lanes(16, 12288, 28672) == (0, 1)        # 768 tile rows: the chip is full
    assert lanes(16, 12288, 12288) == (0, 1)
    assert lanes(16, 57344, 12288) == (0, 1)
    assert lanes(16, 8192, 4096) == (0, 2)          # 512 tile rows: a second lane fills the slots the first leaves
    assert lanes(16, 6144, 4096) == (0, 2)
    assert lanes(16, 4096, 4096) == (0, 3)
    assert lanes(16, 1024, 1024) == (0, 12)         # 64 tile rows: 12 fill the chip, which is also the maximum
    assert lanes(16, 256, 1024) == (0, 12)
    assert lanes(5, 1024, 1024) == (0, 5)           # no more lanes than groups
    assert lanes(1, 1024, 1024) == (0, 1)
    assert lanes(0, 1024, 1024) == (0, 1)
    assert lanes(16, 1024, 16384) == (0, 8)         # 4 n^2 floats of staging and work matrices per lane, 32 GiB in all
    assert lanes(16, 8192, 28672) == (0, 2)
    assert lanes(16, 1024, 28672) == (0, 2)
    assert lanes(16, 1024, 40960) == (0, 1)
    assert lanes(16, 1024, 1024, req=1) == (0, 1)   # the reference's schedule on request
    assert lanes(16, 12288, 28672, req=3) == (0, 3)
    assert lanes(2, 1024, 1024, req=8) == (0, 2)
    assert lanes(16, 1024, 1024, slots=304) == (0, 5)
    rc, _ = lanes(16, 1024, 1024, req=13)
    assert rc != 0 and b"lanes" in L.qtip_last_error()
    rc, _ = lanes(16, 1024, 1024, req=-1)
    assert rc != 0


def test_cholesky_inplace_fp64_bits(pkg, oracle):
    """qtip_cholesky_inplace: every bit of the fp64 factor equals the compiled reference's committed rows (n = 528) and
    the oracle's factor of a matrix with correlated, badly scaled channels (n = 784)."""
    L = pkg.lib()
    L.qtip_cholesky_inplace.argtypes = [C.c_void_p, C.c_int, C.c_int]
    n = 528
    gm = oracle.rng_normal(6, n * 64).reshape(n, 64)
    A = np.tril(gm @ gm.T / 64 + 0.05 * np.eye(n))
    assert L.qtip_cholesky_inplace(A.ctypes.data, n, 3) == 0
    rows = [255, 256, 300, 511, 512, 527]
    want = np.fromfile(os.path.join(GOLDEN, "ref_chol_528_rows.bin"), np.uint64).reshape(len(rows), n)
    assert np.array_equal(np.tril(A)[rows].view(np.uint64), want)
    n = 784
    rng = np.random.default_rng(4)
    G = rng.normal(size=(n, n + 100))
    G[:, 1:] += 0.8 * G[:, :-1]
    G[rng.choice(n, 16, replace=False)] *= 20
    H = np.tril(G @ G.T / (n + 100) + 0.02 * np.eye(n))
    A, B = H.copy(), H.copy()
    assert L.qtip_cholesky_inplace(A.ctypes.data, n, 8) == 0
    assert oracle.lib().qo_cholesky(B.reshape(-1), n) == 1
    assert np.array_equal(np.tril(A).view(np.uint64), np.tril(B).view(np.uint64))
    bad = -np.eye(16)
    assert L.qtip_cholesky_inplace(bad.ctypes.data, 16, 1) == pkg.QTIP_E_NOT_PD


def test_host_ldl_golden_1024(pkg, oracle):
    n = 1024
    gm = oracle.rng_normal(3, n * 64).reshape(n, 64)
    H = gm @ gm.T / 64 + 0.05 * np.eye(n)
    hp = pkg.HessPrep(n=n, HRr=H.astype(np.float32))
    pkg.Quantizer.ldl_hessian(hp, threads=8)
    want = np.fromfile(os.path.join(GOLDEN, "ref_ldl_1024.bin"), np.float32).reshape(8, n)
    # the fixture was computed from the fp64 matrix, this call from its fp32 rounding
    assert np.max(np.abs(hp.L[1000:1008] - want)) <= 2e-5 * np.max(np.abs(want))


def test_host_ldl_golden_2560_bits(pkg, oracle):
    """Rows of L written by the compiled reference's block_ldl_to_L for an fp32 input, ten panels deep: identical
    32-bit words, with one thread and with many (the schedule must not change a bit)."""
    n = 2560
    gm = oracle.rng_normal(5, n * 64).reshape(n, 64)
    H32 = (gm @ gm.T / 64 + 0.05 * np.eye(n)).astype(np.float32)
    rows = [255, 256, 257, 1279, 1280, 2558, 2559]
    want = np.fromfile(os.path.join(GOLDEN, "ref_ldl_2560_f32.bin"), np.uint32).reshape(len(rows), n)
    for threads in (1, 7):
        hp = pkg.HessPrep(n=n, HRr=H32.copy())
        pkg.Quantizer.ldl_hessian(hp, threads=threads)
        assert np.array_equal(hp.L[rows].view(np.uint32), want)


def test_host_ldl_rejects_singular_and_bad_shapes(pkg):
    n = 64
    H = _spd(n, 1, rank=8)     # rank 8 < n and no damping: not positive definite
    hp = pkg.HessPrep(n=n, HRr=H)
    with pytest.raises(pkg.QtipError) as e:
        pkg.Quantizer.ldl_hessian(hp, threads=2)
    assert e.value.code == pkg.QTIP_E_NOT_PD and hp.L is None
    bad = np.eye(n, dtype=np.float32)
    bad[5, 5] = np.nan
    with pytest.raises(pkg.QtipError):
        pkg.Quantizer.ldl_hessian(pkg.HessPrep(n=n, HRr=bad), threads=2)
    with pytest.raises(pkg.QtipError) as e:
        pkg.Quantizer.ldl_hessian(pkg.HessPrep(n=24, HRr=np.eye(24, dtype=np.float32)), threads=1)
    assert e.value.code == pkg.QTIP_E_ARG
