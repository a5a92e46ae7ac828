"""Block LDL with the trailing updates on the GPU (qtip_ldl_hessian_device_updates): the factor must equal the host
factorization's bit for bit (same panel code on the host; the rank-256 updates on the fp64 matrix cores in the host
micro-kernel's order of operations), including ragged last panels, and must fail the same way on a matrix that is not
positive definite."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)


def spd(n, seed, rows=None):
    rng = np.random.default_rng(seed)
    rows = rows or 2 * n
    X = rng.standard_normal((rows, n)).astype(np.float32) * np.linspace(0.2, 3.0, n, dtype=np.float32)
    X[:, 1:] += 0.8 * X[:, :-1]
    H = (X.T @ X / rows).astype(np.float32)
    H += 0.01 * np.float32(np.mean(np.diag(H))) * np.eye(n, dtype=np.float32)
    return H


@pytest.mark.parametrize("n", [16, 496, 512, 1024, 1040, 1152, 2560])
def test_factor_equals_host_factor(qz, pkg, n):
    say("case: LDL with device updates, n = %d" % n)
    H = spd(n, 100 + n)
    a = pkg.HessPrep(n=n, HRr=H.copy())
    b = pkg.HessPrep(n=n, HRr=H.copy())
    pkg.Quantizer.ldl_hessian(a, threads=16)
    qz.ldl_hessian_device_updates(b, threads=16)
    assert np.array_equal(a.L.view(np.uint32), b.L.view(np.uint32))
    # and once more through the same context (buffers reused, a smaller matrix after a larger one)
    if n == 2560:
        H2 = spd(1024, 7)
        a2 = pkg.HessPrep(n=1024, HRr=H2.copy())
        b2 = pkg.HessPrep(n=1024, HRr=H2.copy())
        pkg.Quantizer.ldl_hessian(a2, threads=16)
        qz.ldl_hessian_device_updates(b2, threads=16)
        assert np.array_equal(a2.L.view(np.uint32), b2.L.view(np.uint32))


@pytest.mark.parametrize("n", [272, 1040, 2560])
def test_device_resident_form_equals_host_factor(qz, pkg, n):
    """qtip_ldl_hessian_device_updates_dev: the rotated Hessian stays on the device and is not written, L arrives in the
    host buffer and, column block by column block, in the device buffer; both equal the host factorization's words."""
    import torch
    say("case: LDL with device updates, Hessian resident on the device, n = %d" % n)
    H = spd(n, 300 + n)
    a = pkg.HessPrep(n=n, HRr=H.copy())
    pkg.Quantizer.ldl_hessian(a, threads=16)
    dH = torch.from_numpy(H).cuda()
    L_pin = torch.full((n, n), -1.0, dtype=torch.float32).pin_memory()
    dL = torch.full((n, n), -1.0, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    for _ in range(2):   # twice through the same context: the panel buffers alternate and are reused
        qz.ldl_hessian_device_resident(dH, n, L_pin, dL, threads=16)
        assert np.array_equal(L_pin.numpy().view(np.uint32), a.L.view(np.uint32))
        assert torch.equal(dL.cpu(), L_pin)
        assert torch.equal(dH.cpu(), torch.from_numpy(H))
    # without the device copy of L
    L2 = np.full((n, n), -1.0, np.float32)
    qz.ldl_hessian_device_resident(dH, n, L2, None, threads=16)
    assert np.array_equal(L2.view(np.uint32), a.L.view(np.uint32))


def test_rank_deficient_matrix_is_refused(qz, pkg):
    say("case: LDL with device updates, matrix not positive definite")
    n = 1024
    rng = np.random.default_rng(5)
    X = rng.standard_normal((300, n)).astype(np.float32)      # rank 300 < n, no damping
    H = (X.T @ X / 300).astype(np.float32)
    H[700, 700] = -1.0
    hp = pkg.HessPrep(n=n, HRr=H)
    with pytest.raises(pkg.QtipError):
        qz.ldl_hessian_device_updates(hp, threads=16)
    assert hp.L is None
    # the context is usable afterwards
    ok = pkg.HessPrep(n=512, HRr=spd(512, 3))
    qz.ldl_hessian_device_updates(ok, threads=16)
    assert np.isfinite(ok.L).all()
