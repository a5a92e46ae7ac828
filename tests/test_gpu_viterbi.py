"""GPU parity of the two-pass tail-biting Viterbi (C ABI qtip_viterbi_tiles*) against the CPU oracle and the
golden vectors: bit-exact state paths.  Mirrors tests/test_cpu.cpp:65-96 and tests/test_gpu.cpp:90-129 of the
reference, with the stricter bar of identical codes on inputs that are not fp16-representable."""
import json
import os
import sys

import numpy as np
import pytest

from conftest import GOLDEN, REFVEC

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def g(name, dt):
    return np.fromfile(os.path.join(GOLDEN, name), dtype=dt)


def check_invariants(st):
    st = st.astype(np.uint32)
    assert np.all((st[:, 127] & 0xfff) == (st[:, 0] >> 4)), "tail-biting"
    assert np.all(((st[:, :-1] << 4) & 0xffff) == (st[:, 1:] & 0xfff0)), "trellis links"


def test_refvec_sequences(qz, pkg):
    say("case: 24 upstream sequences, HYB tlut")
    qz.set_tlut(None)
    X = np.fromfile(os.path.join(REFVEC, "vit_x.bin"), np.float32).reshape(24, 256)
    want = np.fromfile(os.path.join(REFVEC, "vit_states.bin"), np.int32).reshape(24, 128).astype(np.uint16)
    hat = np.fromfile(os.path.join(REFVEC, "vit_hat.bin"), np.float32).reshape(24, 256)
    st, pk = qz.viterbi_tiles(X)
    assert np.array_equal(st, want)
    check_invariants(st)
    l0, l1 = qz.lut()
    dec = np.stack([l0[st], l1[st]], axis=-1).reshape(24, 256)
    assert np.array_equal(dec, hat)
    assert np.array_equal(pk, pkg.pack_trellis(st))
    assert np.array_equal(pkg.unpack_trellis(pk), st)


def test_raw_inputs_golden(qz):
    X = g("ref_vit_raw_x.bin", np.float32).reshape(64, 256)
    for tl, name in ((None, "ref_vit_raw_hyb.bin"), ("syn", "ref_vit_raw_syn.bin")):
        say("case: 64 raw fp32 tiles, tlut=%s" % tl)
        if tl is None:
            qz.set_tlut(None)
        else:
            from oracle import binding as ob
            qz.set_tlut(ob.synthetic_tlut(1))
        st, _ = qz.viterbi_tiles(X)
        want = g(name, np.uint16).reshape(64, 128)
        same = np.all(st == want, axis=1)
        assert same.all(), "tiles differing: %s" % np.nonzero(~same)[0][:10]
    qz.set_tlut(None)


def test_config1_full(qz, oracle):
    """Benchmark configuration 1: 4096 tiles of raw fp32 N(0,1), synthetic unit-rms tlut; packed words bit-exact against
    the output of the compiled reference (committed fixture)."""
    say("case: config 1, 4096 tiles")
    meta = json.load(open(os.path.join(GOLDEN, "ref_config1.json")))
    X = oracle.rng_normal(meta["x_seed"], 4096 * 256).astype(np.float32).reshape(4096, 256)
    qz.set_tlut(oracle.synthetic_tlut(meta["tlut_seed"]))
    st, pk = qz.viterbi_tiles(X)
    want = g("ref_config1_packed.bin", np.uint16).reshape(4096, 32)
    same = np.all(pk == want, axis=1)
    assert same.all(), "%d of 4096 tiles differ, first %s" % ((~same).sum(), np.nonzero(~same)[0][:10])
    check_invariants(st)
    qz.set_tlut(None)


def test_edge_inputs_against_oracle(qz, oracle, hyb):
    """Exact ties and extremes: zero tiles, constant tiles, exact codewords, huge and tiny magnitudes; the
    first-minimum tie-break rules decide these paths."""
    say("case: edge inputs")
    qz.set_tlut(None)
    rng = np.random.default_rng(5)
    X = np.zeros((12, 256), np.float32)
    X[1] = 1.0
    X[2] = -0.75
    X[3] = rng.normal(size=256).astype(np.float32) * 1e-4
    X[4] = rng.normal(size=256).astype(np.float32) * 50.0
    X[5, ::2] = 3.0
    nib = rng.integers(0, 16, 128)
    stc = np.array([(nib[(t - 3) % 128] << 12) | (nib[(t - 2) % 128] << 8) | (nib[(t - 1) % 128] << 4) | nib[t]
                    for t in range(128)], np.uint16)
    X[6, 0::2] = hyb.lut0[stc]
    X[6, 1::2] = hyb.lut1[stc]
    X[7] = np.round(rng.normal(size=256) * 2) / 2          # coarse grid: many equal errors
    X[8] = rng.normal(size=256).astype(np.float16).astype(np.float32)
    X[9, :128] = rng.normal(size=128).astype(np.float32)   # half zero
    X[10] = np.float32(1e-30)
    X[11] = rng.standard_t(3, size=256).astype(np.float32) * 3
    want = oracle.quantize_tiles(hyb, X, fast=False)
    st, pk = qz.viterbi_tiles(X)
    same = np.all(st == want, axis=1)
    assert same.all(), "edge tiles differing: %s" % np.nonzero(~same)[0]
    # the exact-codeword tile is recovered at zero error (its path is not unique: states s and 65535-s share
    # one codebook entry, so the tie-break picks between two zero-cost paths)
    l0, l1 = qz.lut()
    assert np.array_equal(l0[st[6]], X[6, 0::2]) and np.array_equal(l1[st[6]], X[6, 1::2])


def test_ragged_batches_and_device_entry(qz, oracle, hyb):
    """B = 0, 1, and a batch larger than the number of resident workgroups (tiles are walked with a stride);
    device-pointer entry point; states-only and packed-only outputs."""
    import torch
    say("case: ragged batches")
    qz.set_tlut(None)
    st, pk = qz.viterbi_tiles(np.zeros((0, 256), np.float32))
    assert st.shape == (0, 128) and pk.shape == (0, 32)
    X = oracle.rng_normal(99, 1000 * 256).astype(np.float32).reshape(1000, 256)
    idx = [0, 1, 500, 767, 768, 769, 999]
    want = oracle.quantize_tiles(hyb, X[idx], fast=True)
    st1, _ = qz.viterbi_tiles(X[:1], want_packed=False)
    assert np.array_equal(st1[0], want[0])
    dX = torch.from_numpy(X).cuda()
    dS = torch.zeros((1000, 128), dtype=torch.int16, device="cuda")
    dP = torch.zeros((1000, 32), dtype=torch.int16, device="cuda")
    torch.cuda.synchronize()
    qz.viterbi_tiles_dev(dX, 1000, dS, dP)
    qz.synchronize()
    st = dS.cpu().numpy().view(np.uint16)
    pk = dP.cpu().numpy().view(np.uint16)
    assert np.array_equal(st[idx], want)
    check_invariants(st)
    assert np.array_equal(pk, oracle.pack_trellis(st))
    # size-independent property at full batch: decode(encode) reproduces hat, cost never above the oracle's on a sample
    dH = torch.zeros((1000, 256), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()                     # the library works on a stream of its own
    qz.decode_states_dev(dS, 1000, dH)
    qz.synchronize()
    l0, l1 = qz.lut()
    assert np.array_equal(dH.cpu().numpy(), np.stack([l0[st], l1[st]], axis=-1).reshape(1000, 256))
    # determinism: a second run gives the same bits
    dS2 = torch.zeros_like(dS)
    torch.cuda.synchronize()
    qz.viterbi_tiles_dev(dX, 1000, dS2, None)
    qz.synchronize()
    assert torch.equal(dS, dS2)


def test_non_finite_inputs_leave_other_tiles_alone(qz, oracle, hyb):
    """Tiles holding NaN or infinite inputs have no meaningful codes, but the launch must complete, write 16-bit
    states for them and leave every other tile of the same launch exactly as the CPU algorithm has it."""
    say("case: non-finite inputs")
    qz.set_tlut(None)
    X = oracle.rng_normal(123, 64 * 256).astype(np.float32).reshape(64, 256)
    bad = {3: np.nan, 17: np.inf, 40: -np.inf}
    for t, v in bad.items():
        X[t, :] = v
    X[29, 100] = np.nan                                      # one NaN in the middle of a sequence
    good = [t for t in range(64) if t not in bad and t != 29]
    want = oracle.quantize_tiles(hyb, X[good], fast=True)
    st, pk = qz.viterbi_tiles(X)
    assert np.array_equal(st[good], want)
    assert np.array_equal(pk[good], oracle.pack_trellis(want))


def _mixed_inputs(oracle, B=320):
    """raw, fp16-rounded, tie-laden and extreme tiles"""
    rng = np.random.default_rng(11)
    X = oracle.rng_normal(4242, B * 256).astype(np.float32).reshape(B, 256)
    X[64:128] = X[64:128].astype(np.float16).astype(np.float32)           # fp16-representable, as LDLQ feeds them
    X[128:160] = (X[128:160] * np.float32(0.87)).astype(np.float16).astype(np.float32)
    X[160:176] = np.round(X[160:176] * 2) / 2                              # coarse grid: many equal errors
    X[176] = 0.0
    X[177] = 1.0
    X[178] = 40.0                                                          # squared errors beyond the 32-bit range
    X[179, ::2] = -3.0
    X[180] = X[180] * np.float32(1e-3)
    X[181:192] = rng.standard_t(3, size=(11, 256)).astype(np.float32) * 2
    return X


def test_metric_modes_give_the_same_states(qz, oracle, hyb):
    """The default runs each pass on 32-bit metrics and repeats it on fp64 metrics when a decision on the surviving
    path is too close to call; fp64-only, and the default with a margin no decision can reach (every pass repeated),
    must give the same states, the CPU algorithm's, on raw inputs, fp16-rounded inputs (the LDLQ case) and inputs full
    of exact ties.  The counters say how many passes were repeated."""
    say("case: 32-bit-first, fp64-only and all-repeated passes agree")
    qz.set_tlut(None)
    B = 320
    X = _mixed_inputs(oracle, B)
    want = oracle.quantize_tiles(hyb, X, fast=True)
    try:
        qz.viterbi_stats(reset=True)
        qz.set_viterbi_mode(0)
        st0, pk0 = qz.viterbi_tiles(X)
        r0 = qz.viterbi_stats(reset=True)
        say("  default: %d first and %d second passes of %d tiles repeated on fp64 metrics" % (r0[0], r0[1], B))
        qz.set_viterbi_mode(1)
        st1, pk1 = qz.viterbi_tiles(X)
        assert qz.viterbi_stats(reset=True) == (0, 0)
        qz.set_viterbi_mode(0, 0xffffffff)
        st2, pk2 = qz.viterbi_tiles(X)
        r2 = qz.viterbi_stats(reset=True)
    finally:
        qz.set_viterbi_mode(0)
    for name, st in (("default", st0), ("fp64 only", st1), ("all repeated", st2)):
        same = np.all(st == want, axis=1)
        assert same.all(), "%s: tiles differing from the CPU algorithm: %s" % (name, np.nonzero(~same)[0][:10])
    assert np.array_equal(pk0, pk1) and np.array_equal(pk0, pk2)
    assert r2 == (B, B)
    # near-ties of 2e-6 relative are rare: the bulk of the passes stands on 32-bit metrics (the tie-laden tiles
    # 160..179 may all be repeated)
    assert r0[0] <= 40 and r0[1] <= 40


def test_metric_unit_follows_the_scale_of_the_inputs(qz, oracle, hyb):
    """The unit of a 32-bit pass is chosen from the winner expected (the free pass's, for the tail-biting pass of the
    same tile): inputs an eighth or twice the size of normalized weights still give the CPU algorithm's states, and at
    twice or six times the size - where a free pass in the default unit cannot hold its winner and is repeated on
    fp64 metrics, which gives the true winner - the tail-biting passes run in a coarser unit instead of being repeated
    as well."""
    say("case: inputs of other scales")
    qz.set_tlut(None)
    B = 96
    base = oracle.rng_normal(77, B * 256).astype(np.float32).reshape(B, 256)
    try:
        qz.set_viterbi_mode(0)
        for scale in (0.125, 2.0, 6.0):
            X = (base * np.float32(scale)).astype(np.float32)
            want = oracle.quantize_tiles(hyb, X, fast=True)
            qz.viterbi_stats(reset=True)
            st, pk = qz.viterbi_tiles(X)
            r = qz.viterbi_stats(reset=True)
            say("  x %g: %d first and %d second passes of %d repeated" % (scale, r[0], r[1], B))
            same = np.all(st == want, axis=1)
            assert same.all(), "x %g: tiles differing from the CPU algorithm: %s" % (scale, np.nonzero(~same)[0][:10])
            if scale == 0.125:
                assert r[0] <= 4 and r[1] <= 4
            if scale >= 2.0:
                assert r[1] <= B // 4
    finally:
        qz.set_viterbi_mode(0)


def test_wide_workgroups_give_the_same_states(qz, oracle, hyb):
    """A launch that cannot fill the chip gives every tile 512 threads instead of 256 (the 32-bit forward passes
    share the groups out over all of them; everything else, the fp64 repeat of a pass included, is done by both
    halves alike).  Forced on and off on the same inputs, with and without every pass repeated: the CPU algorithm's
    states each time; and benchmark configuration 1 in full through the wide form against the compiled reference's
    packed words."""
    say("case: 512-thread workgroups")
    qz.set_tlut(None)
    B = 320
    X = _mixed_inputs(oracle, B)
    want = oracle.quantize_tiles(hyb, X, fast=True)
    try:
        for mode, margin, name in ((2, 0, "256 threads"), (3, 0, "512 threads"), (3, 0xffffffff, "512 threads, all repeated")):
            qz.viterbi_stats(reset=True)
            qz.set_viterbi_mode(mode, margin)
            st, pk = qz.viterbi_tiles(X)
            r = qz.viterbi_stats(reset=True)
            say("  %s: %d first and %d second passes repeated" % (name, r[0], r[1]))
            same = np.all(st == want, axis=1)
            assert same.all(), "%s: tiles differing from the CPU algorithm: %s" % (name, np.nonzero(~same)[0][:10])
            assert r == (B, B) if margin else (r[0] <= 40 and r[1] <= 40)
        meta = json.load(open(os.path.join(GOLDEN, "ref_config1.json")))
        X1 = oracle.rng_normal(meta["x_seed"], 4096 * 256).astype(np.float32).reshape(4096, 256)
        qz.set_tlut(oracle.synthetic_tlut(meta["tlut_seed"]))
        qz.set_viterbi_mode(3)
        st, pk = qz.viterbi_tiles(X1)
        want1 = g("ref_config1_packed.bin", np.uint16).reshape(4096, 32)
        same = np.all(pk == want1, axis=1)
        assert same.all(), "%d of 4096 tiles differ, first %s" % ((~same).sum(), np.nonzero(~same)[0][:10])
    finally:
        qz.set_viterbi_mode(0)
        qz.set_tlut(None)
