"""Seeded synthetic layers for the benchmark configurations (the five benchmark configurations: tiles only, 1024 x 1024, q-proj, gate+up, down-proj).

Small configurations are generated with numpy on the host (bit-stable across machines); the large ones with
torch on the GPU so that set-up takes seconds, not minutes.  Input synthesis is never timed.
"""
import numpy as np


def _bf16_round(x):
    """fp32 -> bf16 (round to nearest even) -> fp32, numpy."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7fff + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32)


def ar1_activations(rng, rows, n, rho, n_outliers, outlier_scale):
    """rows x n activations: an AR(1) process across channels plus a few channels scaled up; bf16-rounded."""
    e = rng.standard_normal((rows, n)).astype(np.float32)
    x = np.empty_like(e)
    x[:, 0] = e[:, 0]
    s = np.float32(np.sqrt(1.0 - rho * rho))
    for j in range(1, n):
        x[:, j] = np.float32(rho) * x[:, j - 1] + s * e[:, j]
    ch = rng.choice(n, size=n_outliers, replace=False)
    x[:, ch] *= np.float32(outlier_scale)
    return _bf16_round(x)


def config2(seed=2):
    """Full group, small layer: W 1024x1024 ~ 0.02 * Student-t(5); H = X^T X / N, X 8192x1024 bf16 AR(1) rho 0.9
    with 8 outlier channels x20."""
    rng = np.random.default_rng(seed)
    n = 1024
    W = (0.02 * rng.standard_t(5, size=(n, n))).astype(np.float32)
    X = ar1_activations(rng, 8192, n, 0.9, 8, 20.0)
    H = (X.T.astype(np.float32) @ X.astype(np.float32) / np.float32(8192)).astype(np.float32)
    H = ((H + H.T) * np.float32(0.5)).astype(np.float32)
    return [W], H


def small_group(seed=33, n=256, ms=(64, 32)):
    """The reference's end-to-end test case (tests/test_gpu.cpp:301-318): two linears sharing one Hessian."""
    rng = np.random.default_rng(seed)
    Ws = [(rng.standard_normal((m, n)) * s).astype(np.float32) for m, s in zip(ms, (0.02, 0.05, 0.03, 0.01))]
    G = rng.standard_normal((n, 3 * n))
    H = (G @ G.T / (3 * n)).astype(np.float32)
    return Ws, H


# ---------------------------------------------------------------- large configurations (torch, on the GPU)
def _ar1_torch(gen, rows, n, rho, n_outliers, outlier_scale, device):
    import torch
    # stationary AR(1) across channels, built blockwise with the closed form x_j = sum_k rho^(j-k) s e_k via a
    # scan in chunks (exact recurrence inside a chunk, carried state between chunks)
    e = torch.randn((rows, n), generator=gen, device=device, dtype=torch.float32)
    s = float(np.sqrt(1.0 - rho * rho))
    x = torch.empty_like(e)
    # recurrence as a causal filter: cumulative sum in a scaled domain, 256 channels at a time for range safety
    carry = torch.zeros((rows,), device=device)
    step = 256
    for j0 in range(0, n, step):
        j1 = min(n, j0 + step)
        w = j1 - j0
        k = torch.arange(w, device=device, dtype=torch.float32)
        scale = rho ** k                     # rho^k
        blk = e[:, j0:j1] * s
        if j0 == 0:
            blk[:, 0] = e[:, 0]
        y = torch.cumsum(blk / scale, dim=1) * scale
        y = y + carry[:, None] * (rho ** (k + 1))
        x[:, j0:j1] = y
        carry = y[:, -1]
    ch = torch.randperm(n, generator=gen, device=device)[:n_outliers]
    x[:, ch] *= outlier_scale
    return x.to(torch.bfloat16)


def _hessian_from(xb):
    import torch
    x = xb.to(torch.float32)
    H = (x.T @ x) / float(x.shape[0])
    return ((H + H.T) * 0.5).contiguous()


def large_config(cfg, device="cuda", seed=None):
    """Configurations 3, 4 and 5 as device tensors: (list of W, H).  fp32 GEMM accumulation for H."""
    import torch
    torch.backends.cuda.matmul.allow_tf32 = False
    gen = torch.Generator(device=device)
    gen.manual_seed(1000 + cfg if seed is None else seed)
    if cfg == 3:     # q-proj: W 12288x12288 Gaussian*0.015 with 1% entries x10
        n, ms = 12288, [12288]
        Ws = []
        for m in ms:
            w = torch.randn((m, n), generator=gen, device=device) * 0.015
            mask = torch.rand((m, n), generator=gen, device=device) < 0.01
            Ws.append(torch.where(mask, w * 10.0, w).contiguous())
        H = _hessian_from(_ar1_torch(gen, 16384, n, 0.8, 32, 20.0, device))
    elif cfg == 4:   # gate+up: two stacked 28672x12288, Gaussian*0.012 with 0.5% x8, shared Hessian
        n, ms = 12288, [28672, 28672]
        Ws = []
        for m in ms:
            w = torch.randn((m, n), generator=gen, device=device) * 0.012
            mask = torch.rand((m, n), generator=gen, device=device) < 0.005
            Ws.append(torch.where(mask, w * 8.0, w).contiguous())
        H = _hessian_from(_ar1_torch(gen, 16384, n, 0.8, 32, 20.0, device))
    elif cfg == 5:   # down-proj: W 12288x28672 Student-t(4)*0.01; X = g1 * silu(g2), 8192 rows: rank-deficient H
        n, m = 28672, 12288
        z = torch.randn((m, n), generator=gen, device=device)
        chi = torch.zeros((m, n), device=device)
        for _ in range(4):
            g = torch.randn((m, n), generator=gen, device=device)
            chi += g * g
            del g
        Ws = [(0.01 * z / torch.sqrt(chi / 4.0)).contiguous()]
        del z, chi
        g1 = torch.randn((8192, n), generator=gen, device=device)
        g2 = torch.randn((8192, n), generator=gen, device=device)
        xb = (g1 * torch.nn.functional.silu(g2)).to(torch.bfloat16)
        del g1, g2
        H = _hessian_from(xb)
    else:
        raise ValueError("large_config: cfg must be 3, 4 or 5")
    torch.cuda.synchronize()
    return Ws, H
