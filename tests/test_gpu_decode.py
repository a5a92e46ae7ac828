"""GPU parity of the decoder of the packed output through the C ABI: kernel-layout trellis words back to the rotated
weight (decode_rows, runtime/src/qtip.cpp:83-118) and on to the original domain (src/quantizer.cpp:321-338).
The expected values come from the reference's golden pack vectors, from a decoder written from the runtime's
description of the layout, and from the reconstruction quantize_group itself returns."""
import os
import time

import numpy as np
import pytest

from conftest import REFVEC

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)


def _window_states(tr, m, n):
    """States of every tile from kernel-layout words: 16-bit windows at bit 4t of the wrapping 512-bit stream
    (runtime/src/qtip.cpp:90-95), words addressed as HostLinear::word (runtime/include/behemoth/qtip.hpp:63-67)."""
    n2 = n // 32
    w = tr.reshape(m // 32, n2, 32, 2, 2).astype(np.uint32)          # [i0][j0][c][j1][i1]
    w = w.transpose(0, 4, 1, 3, 2).reshape(m // 16, n // 16, 32)      # [tile_row][tile_col][c]
    two = (w << 16) | np.roll(w, -1, axis=2)
    st = np.empty((m // 16, n // 16, 128), np.uint32)
    for k in range(4):
        st[:, :, k::4] = (two >> (16 - 4 * k)) & 0xffff
    return st


def _decode_expected(tr, m, n, lut0, lut1):
    st = _window_states(tr, m, n)
    t = np.arange(128)
    A, B, Cc, D = t >> 4, (t >> 2) & 3, (t >> 1) & 1, t & 1
    r, col = D * 8 + A, Cc * 8 + B * 2
    out = np.zeros((m // 16, n // 16, 16, 16), np.float32)
    out[:, :, r, col] = lut0[st]
    out[:, :, r, col + 1] = lut1[st]
    return out.transpose(0, 2, 1, 3).reshape(m, n)


def _gpu_decode(qz, tr, m, n):
    import torch
    d_tr = torch.from_numpy(tr.view(np.int16)).cuda()
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
    qz.decode_trellis_dev(d_tr, m, n, out)
    qz.synchronize()
    return out.cpu().numpy()


def test_decode_golden_pack_vectors(qz, oracle, hyb):
    """tests/refvec/pack_{states,kernel}.bin (m=64, n=96): decode(kernel words) == codebook[states] placed by _PERMUTE."""
    say("case: decode golden pack vectors 64x96")
    qz.set_tlut(None)
    m, n = 64, 96
    st = np.fromfile(os.path.join(REFVEC, "pack_states.bin"), dtype=np.int32).astype(np.uint16).reshape(-1, 128)
    kern = np.fromfile(os.path.join(REFVEC, "pack_kernel.bin"), dtype=np.uint16)
    perm, _ = oracle.perm256()
    want = np.zeros((m, n), np.float32)
    for b in range(m // 16):
        for blk in range(n // 16):
            s = st[b * (n // 16) + blk]
            tile = np.zeros(256, np.float32)
            tile[perm] = np.stack([hyb.lut0[s], hyb.lut1[s]], axis=-1).reshape(-1)
            want[16 * b:16 * b + 16, 16 * blk:16 * blk + 16] = tile.reshape(16, 16)
    got = _gpu_decode(qz, kern, m, n)
    assert np.array_equal(got, want)
    assert np.array_equal(_decode_expected(kern, m, n, hyb.lut0, hyb.lut1), want)   # the test's own decoder agrees


@pytest.mark.parametrize("m,n", [(32, 32), (64, 160), (96, 4096), (1024, 1056)])
def test_decode_random_words(qz, oracle, syn, m, n):
    """Any 512 bits are a valid tail-biting stream: random words, ragged column counts (n/32 not a multiple of 4)."""
    say("case: decode random words %dx%d" % (m, n))
    qz.set_tlut(oracle.synthetic_tlut(1))
    try:
        rng = np.random.default_rng(m * 131 + n)
        tr = rng.integers(0, 65536, (m // 16) * (n // 16) * 32, dtype=np.uint16)
        got = _gpu_decode(qz, tr, m, n)
        assert np.array_equal(got, _decode_expected(tr, m, n, syn.lut0, syn.lut1))
    finally:
        qz.set_tlut(None)


def test_decode_rejects_bad_shapes(qz, pkg):
    import torch
    d = torch.zeros(16 * 96 * 2, dtype=torch.int16, device="cuda")
    o = torch.zeros((16, 96), dtype=torch.float32, device="cuda")
    with pytest.raises(pkg.QtipError):
        qz.decode_trellis_dev(d, 16, 96, o)      # m not a multiple of 32
    with pytest.raises(pkg.QtipError):
        qz.decode_trellis_dev(d, 32, 48, o)      # n not a multiple of 32


def test_dequantize_equals_group_reconstruction(qz, oracle, pkg, hyb):
    """dequantize_linear(packed output) is bit-identical to the hatW quantize_group reconstructs from its LDLQ
    buffer, and decode(trellis) * Wscale is the rotated weight the CPU decode of the same words gives."""
    import importlib.util
    from conftest import ROOT
    spec = importlib.util.spec_from_file_location("qtip_synth", os.path.join(ROOT, "behemoth-qtip_amd", "synth.py"))
    synth = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(synth)
    say("case: dequantize group n=256, m=64+32")
    qz.set_tlut(None)
    Ws, H = synth.small_group()
    n = H.shape[0]
    lins = [pkg.LinearIn("a", Ws[0].shape[0], w_f32=Ws[0]), pkg.LinearIn("b", Ws[1].shape[0], w_f32=Ws[1])]
    outs, _ = qz.quantize_group_h(lins, n, H, 7, pkg.QuantOpts(want_hatW=True, ldl_threads=4))
    for lo in outs:
        hat = qz.dequantize_linear(lo)
        assert hat.shape == (lo.m, n)
        assert np.array_equal(hat, lo.hatW)
        hr = _gpu_decode(qz, lo.trellis, lo.m, n)
        st = pkg.unpack_trellis(pkg.unswizzle_for_kernel(lo.trellis, lo.m, n))
        assert np.array_equal(_window_states(lo.trellis, lo.m, n).reshape(-1, 128), st)
        assert np.array_equal(hr, _decode_expected(lo.trellis, lo.m, n, hyb.lut0, hyb.lut1))


def test_decode_full_size_sample(qz, hyb):
    """Benchmark configuration 5 shape (12288 x 28672): random words decoded on the device, a sample of 32-row blocks
    compared with the CPU decoder, every value a codebook entry; prints the achieved HBM rate."""
    import torch
    say("case: decode 12288x28672 random words")
    qz.set_tlut(None)
    m, n = 12288, 28672
    g = torch.Generator(device="cuda").manual_seed(5)
    tr = torch.randint(-32768, 32768, ((m // 16) * (n // 16) * 32,), dtype=torch.int16, device="cuda", generator=g)
    out = torch.empty((m, n), dtype=torch.float32, device="cuda")
    qz.decode_trellis_dev(tr, m, n, out)
    qz.synchronize()
    t0 = time.time()
    reps = 5
    for _ in range(reps):
        qz.decode_trellis_dev(tr, m, n, out)
    qz.synchronize()
    dt = (time.time() - t0) / reps
    say("  decode %.3f ms: %.1f Gweights/s, %.2f TB/s of HBM traffic (0.25 B read + 4 B written per weight)" %
        (dt * 1e3, m * n / dt / 1e9, m * n * 4.25 / dt / 1e12))
    per_block = (n // 32) * 128
    for i0 in (0, 1, 191, 383):
        words = tr[i0 * per_block:(i0 + 1) * per_block].cpu().numpy().view(np.uint16)
        want = _decode_expected(words, 32, n, hyb.lut0, hyb.lut1)
        assert np.array_equal(out[32 * i0:32 * i0 + 32].cpu().numpy(), want)
    # every output is one of the 2 x 1024 codebook values: squares summed per row stay finite and positive
    assert bool(torch.isfinite(out).all())
    vals = torch.unique(out)
    cb = np.unique(np.concatenate([hyb.lut0, hyb.lut1]))
    assert np.isin(vals.cpu().numpy(), cb).all()
