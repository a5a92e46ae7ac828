"""Seeded synthetic layers for the benchmark configurations (the five benchmark configurations: tiles only, 1024 x 1024, q-proj, gate+up, down-proj).

Small configurations are generated with numpy on the host (bit-stable across machines); the large ones on the GPU so
that set-up takes seconds, not minutes, from the reference's own splitmix64 stream (Rng, src/common.hpp:91-107): the
k-th output of a stream is a function of (seed, k) alone, so a tensor is filled in parallel and depends on no
library's generator, only on fp64 log / cos / sqrt of the device.  Input synthesis is never timed.
"""
import numpy as np

_M64 = (1 << 64) - 1
_GAMMA = 0x9E3779B97F4A7C15


def splitmix_u64(seed, count, start=0):
    """Outputs start .. start + count - 1 of Rng(seed).next() (src/common.hpp:91-100) as a uint64 array."""
    s0 = (int(seed) * _GAMMA + 0x1234567) & _M64
    k = np.arange(start + 1, start + count + 1, dtype=np.uint64)
    with np.errstate(over="ignore"):
        z = np.uint64(s0) + k * np.uint64(_GAMMA)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def splitmix_uniform(seed, count, start=0):
    """Rng::uniform: the top 53 bits of next() as a double in [0, 1)."""
    return (splitmix_u64(seed, count, start) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def splitmix_normal(seed, count):
    """Rng::normal (Box-Muller on two consecutive uniforms, src/common.hpp:101-105), numpy on the host."""
    u = splitmix_uniform(seed, 2 * count).reshape(count, 2)
    u1 = np.maximum(u[:, 0], 1e-300)
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(6.283185307179586 * u[:, 1])


def synthetic_tlut(seed=1):
    """Benchmark configuration 1's codebook: 512 x 2 fp32 drawn N(0, 1) from the splitmix stream, rescaled to unit rms."""
    v = splitmix_normal(seed, 1024).astype(np.float32).reshape(512, 2)
    return (v / np.float32(np.sqrt(np.mean(v.astype(np.float64) ** 2)))).astype(np.float32)


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


# ---------------------------------------------------------------- large configurations (on the GPU)
class DeviceStream:
    """The splitmix stream of one seed on a torch device; every draw continues where the last one ended."""

    def __init__(self, seed, device="cuda"):
        self.s0 = (int(seed) * _GAMMA + 0x1234567) & _M64
        self.pos = 0
        self.device = device

    @staticmethod
    def _i64(v):      # a 64-bit pattern as the int64 torch computes with (wrapping arithmetic)
        v &= _M64
        return v - (1 << 64) if v >= (1 << 63) else v

    @staticmethod
    def _srl(z, k):   # logical shift right of an int64 tensor
        return (z >> k) & ((1 << (64 - k)) - 1)

    def _uniform_flat(self, count):
        import torch
        k = torch.arange(self.pos + 1, self.pos + count + 1, dtype=torch.int64, device=self.device)
        self.pos += count
        z = k * self._i64(_GAMMA) + self._i64(self.s0)
        z = (z ^ self._srl(z, 30)) * self._i64(0xBF58476D1CE4E5B9)
        z = (z ^ self._srl(z, 27)) * self._i64(0x94D049BB133111EB)
        z = z ^ self._srl(z, 31)
        return self._srl(z, 11).to(torch.float64) * (1.0 / 9007199254740992.0)

    def uniform(self, shape, chunk=1 << 25):
        import torch
        count = int(np.prod(shape))
        out = torch.empty(count, dtype=torch.float32, device=self.device)
        for a in range(0, count, chunk):
            b = min(count, a + chunk)
            out[a:b] = self._uniform_flat(b - a).to(torch.float32)
        return out.reshape(shape)

    def normal(self, shape, chunk=1 << 24):
        """fp32 N(0, 1): Box-Muller on two consecutive uniforms per value, in fp64, as Rng::normal."""
        import torch
        count = int(np.prod(shape))
        out = torch.empty(count, dtype=torch.float32, device=self.device)
        for a in range(0, count, chunk):
            b = min(count, a + chunk)
            u = self._uniform_flat(2 * (b - a)).reshape(b - a, 2)
            u1 = torch.clamp(u[:, 0], min=1e-300)
            out[a:b] = (torch.sqrt(-2.0 * torch.log(u1)) * torch.cos(6.283185307179586 * u[:, 1])).to(torch.float32)
        return out.reshape(shape)


def _ar1_device(st, rows, n, rho, n_outliers, outlier_scale):
    import torch
    device = st.device
    # stationary AR(1) across channels, x_j = rho x_(j-1) + s e_j, as a scan in chunks of 256 channels (a cumulative
    # sum in a domain scaled by rho^k, which stays in range over 256 channels), the state carried between chunks
    e = st.normal((rows, n))
    s = float(np.sqrt(1.0 - rho * rho))
    x = torch.empty_like(e)
    carry = torch.zeros((rows,), device=device)
    step = 256
    for j0 in range(0, n, step):
        j1 = min(n, j0 + step)
        w = j1 - j0
        k = torch.arange(w, device=device, dtype=torch.float32)
        scale = rho ** k
        blk = e[:, j0:j1] * s
        if j0 == 0:
            blk[:, 0] = e[:, 0]
        y = torch.cumsum(blk / scale, dim=1) * scale
        y = y + carry[:, None] * (rho ** (k + 1))
        x[:, j0:j1] = y
        carry = y[:, -1]
    ch = torch.argsort(st.uniform((n,)))[:n_outliers]      # the channels scaled up: the n_outliers smallest draws
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
    st = DeviceStream(1000 + cfg if seed is None else seed, device)
    if cfg == 3:     # q-proj: W 12288x12288 Gaussian*0.015 with 1% entries x10
        n, ms = 12288, [12288]
        Ws = []
        for m in ms:
            w = st.normal((m, n)) * 0.015
            mask = st.uniform((m, n)) < 0.01
            Ws.append(torch.where(mask, w * 10.0, w).contiguous())
        H = _hessian_from(_ar1_device(st, 16384, n, 0.8, 32, 20.0))
    elif cfg == 4:   # gate+up: two stacked 28672x12288, Gaussian*0.012 with 0.5% x8, shared Hessian
        n, ms = 12288, [28672, 28672]
        Ws = []
        for m in ms:
            w = st.normal((m, n)) * 0.012
            mask = st.uniform((m, n)) < 0.005
            Ws.append(torch.where(mask, w * 8.0, w).contiguous())
        H = _hessian_from(_ar1_device(st, 16384, n, 0.8, 32, 20.0))
    elif cfg == 5:   # down-proj: W 12288x28672 Student-t(4)*0.01; X = g1 * silu(g2), 8192 rows: rank-deficient H
        n, m = 28672, 12288
        z = st.normal((m, n))
        chi = torch.zeros((m, n), device=device)
        for _ in range(4):
            g = st.normal((m, n))
            chi += g * g
            del g
        Ws = [(0.01 * z / torch.sqrt(chi / 4.0)).contiguous()]
        del z, chi
        g1 = st.normal((8192, n))
        g2 = st.normal((8192, n))
        xb = (g1 * torch.nn.functional.silu(g2)).to(torch.bfloat16)
        del g1, g2
        H = _hessian_from(xb)
    else:
        raise ValueError("large_config: cfg must be 3, 4 or 5")
    torch.cuda.synchronize()
    return Ws, H
