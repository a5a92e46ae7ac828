"""GPU parity of the Hessian accumulation through the C ABI (the step before the path: hess() in
LayerRunner::forward_batch, src/model.cpp:352-363; symmetrize_hess, src/model.cpp:260-264; the 1 / token count of
src/pipeline.cpp:160-166).  The reference computes it with a vendor bf16 GEMM (fp32 accumulate); the check here is
X^T X in fp64 on the same bf16 values, to the tolerance fp32 accumulation of `rows` exact products allows."""
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)


def _bf16_bits(x):
    u = x.astype(np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _bf16_vals(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


@pytest.mark.parametrize("rows,n", [(64, 256), (300, 1024), (1, 96), (257, 2304), (130, 3000), (4096, 512)])
def test_hessian_accumulate_matches_fp64(qz, rows, n):
    """Ragged row counts (not multiples of the 64-row stage), widths that are not multiples of the 256 tile, two
    batches accumulated into one H, then mirrored and scaled by 1 / count."""
    import torch
    say("case: hessian rows=%d n=%d" % (rows, n))
    rng = np.random.default_rng(rows * 7 + n)
    X1 = _bf16_bits(rng.standard_normal((rows, n)) * (1 + 3 * (rng.random(n) < 0.02)))
    X2 = _bf16_bits(rng.standard_normal((rows + 3, n)))
    dH = torch.zeros((n, n), dtype=torch.float32, device="cuda")
    for X in (X1, X2):
        dX = torch.from_numpy(X.view(np.int16)).cuda()
        qz.hessian_accumulate_dev(dX, X.shape[0], n, dH)
    count = 2 * rows + 3
    qz.hessian_finish_dev(dH, n, 1.0 / count)
    qz.synchronize()
    H = dH.cpu().numpy()
    A1, A2 = _bf16_vals(X1).astype(np.float64), _bf16_vals(X2).astype(np.float64)
    want = (A1.T @ A1 + A2.T @ A2) / count
    bound = (np.abs(A1).T @ np.abs(A1) + np.abs(A2).T @ np.abs(A2)) / count   # sum of |products|
    err = np.abs(H - want)
    # products of bf16 values are exact in fp32; the sum of k terms carries at most ~k * 2^-24 relative to sum |terms|
    tol = bound * (count * 2.0 ** -24 + 2.0 ** -22) + 1e-30
    say("  max err %.3e (max |H| %.3e), worst err/tol %.3f" % (err.max(), np.abs(want).max(), (err / tol).max()))
    assert np.all(err <= tol)
    assert np.array_equal(H, H.T)                      # the mirrored triangle is a copy


def test_hessian_rejects_bad_shapes(qz, pkg):
    import torch
    d = torch.zeros(100, dtype=torch.int16, device="cuda")
    h = torch.zeros((10, 10), dtype=torch.float32, device="cuda")
    with pytest.raises(pkg.QtipError):
        qz.hessian_accumulate_dev(d, 10, 10, h)        # n % 8
    qz.hessian_accumulate_dev(d, 0, 8, h)              # no rows: nothing to do


def test_hessian_config5_shape(qz):
    """Benchmark configuration 5 width (n = 28672) with 8192 token rows: sampled entries against fp64, exact symmetry,
    and the achieved matrix-core rate."""
    import torch
    say("case: hessian 8192 x 28672")
    rows, n = 8192, 28672
    g = torch.Generator(device="cuda").manual_seed(11)
    X = (torch.randn((rows, n), generator=g, device="cuda") * 0.5).to(torch.bfloat16)
    dH = torch.zeros((n, n), dtype=torch.float32, device="cuda")
    # timed: the last of five calls in a row (batch image and update; the chip's clock settles over the first calls)
    for it in range(5):
        if it == 4:
            dH.zero_()
        torch.cuda.synchronize()
        t0 = time.time()
        qz.hessian_accumulate_dev(X.view(torch.int16), rows, n, dH)
        qz.synchronize()
        dt = time.time() - t0
        say("  call %d: %.2f ms" % (it, dt * 1e3))
    tiles = n // 256
    flop = 2.0 * rows * 256 * 256 * (tiles * (tiles + 1) // 2)
    say("  accumulate %.2f ms: %.1f TFLOP/s executed (lower-triangular tiles), %.1f%% of the 2.5 PFLOP/s bf16 peak; "
        "%.1f TFLOP/s counted on the full square" % (dt * 1e3, flop / dt / 1e12, flop / dt / 2.5e15 * 100, 2.0 * rows * n * n / dt / 1e12))
    qz.hessian_finish_dev(dH, n, 1.0 / rows)
    qz.synchronize()
    rng = np.random.default_rng(3)
    idx = np.unique(np.concatenate([rng.integers(0, n, 40), [0, 255, 256, n - 1]]))
    Xs = X[:, torch.from_numpy(idx).cuda()].to(torch.float64)
    want = (Xs.T @ Xs / rows).cpu().numpy()
    got = dH[torch.from_numpy(idx).cuda()][:, torch.from_numpy(idx).cuda()].cpu().numpy()
    assert np.max(np.abs(got - want)) < 5e-4 * np.max(np.abs(want))
    # symmetry on a band of rows
    band = dH[:512].cpu().numpy()
    assert np.array_equal(band[:, :512], band[:, :512].T)
    assert np.array_equal(band[:, 20000:20512], dH[20000:20512, :512].cpu().numpy().T)
