"""The allocation-free Viterbi entry point (qtip_viterbi_tiles_dev_noalloc) against qtip_viterbi_tiles_dev through the
C ABI: identical state words and packed words, on two calls in a row that share the library's fixed workspace, the
second with a smaller batch; and the size limit is refused with an error instead of a launch."""
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _run(qz, call, dX, B):
    import torch
    dS = torch.full((max(B, 1), 128), -1, dtype=torch.int16, device="cuda")
    dP = torch.full((max(B, 1), 32), -1, dtype=torch.int16, device="cuda")
    torch.cuda.synchronize()  # the library works on a stream of its own
    call(dX, B, dS, dP)
    qz.synchronize()
    return dS.cpu().numpy().view(np.uint16)[:B], dP.cpu().numpy().view(np.uint16)[:B]


def test_noalloc_equals_allocating_entry_point(qz, pkg, oracle, hyb):
    import torch
    qz.set_tlut(None)
    # 200 tiles: more than the 32 fixed slots, so every slot is reused within the call; then 37 (ragged last round)
    for seed, B in ((2024, 200), (2025, 37)):
        say("case: no-alloc Viterbi, seed %d, B = %d" % (seed, B))
        X = oracle.rng_normal(seed, B * 256).astype(np.float32).reshape(B, 256)
        dX = torch.from_numpy(X).cuda()
        st_ref, pk_ref = _run(qz, qz.viterbi_tiles_dev, dX, B)
        st, pk = _run(qz, qz.viterbi_tiles_dev_noalloc, dX, B)
        assert np.array_equal(st, st_ref), "states differ in tiles %s" % np.nonzero((st != st_ref).any(1))[0][:10]
        assert np.array_equal(pk, pk_ref)
        # and both are the CPU algorithm's on a sample
        idx = [0, 31, 32, B - 1]
        assert np.array_equal(st[idx], oracle.quantize_tiles(hyb, X[idx], fast=True))


def test_noalloc_call_allocates_nothing(qz, pkg, oracle):
    """The property the entry point exists for: across the call the library makes no device allocation (its own
    counter of hipMalloc calls) and the device's free memory does not move."""
    import torch
    say("case: no-alloc Viterbi makes no device allocation")
    qz.set_tlut(None)
    B = 96
    X = oracle.rng_normal(77, B * 256).astype(np.float32).reshape(B, 256)
    dX = torch.from_numpy(X).cuda()
    dS = torch.zeros((B, 128), dtype=torch.int16, device="cuda")
    dP = torch.zeros((B, 32), dtype=torch.int16, device="cuda")
    torch.cuda.synchronize()
    calls0, free0 = pkg.device_alloc_calls(), torch.cuda.mem_get_info()[0]
    qz.viterbi_tiles_dev_noalloc(dX, B, dS, dP)
    qz.synchronize()
    calls1, free1 = pkg.device_alloc_calls(), torch.cuda.mem_get_info()[0]
    assert calls1 == calls0, "the call made %d device allocations" % (calls1 - calls0)
    assert free1 == free0, "free device memory moved by %d bytes across the call" % (free0 - free1)
    # (the allocating entry point, by contrast, is allowed to: its workspace comes from hipMalloc on first use)


def test_noalloc_limits(qz, pkg):
    import torch
    say("case: no-alloc Viterbi, B = 0 and B above the limit")
    dX = torch.zeros((1, 256), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    qz.viterbi_tiles_dev_noalloc(dX, 0, None, None)  # nothing to do, no error
    with pytest.raises(pkg.QtipError) as e:
        qz.viterbi_tiles_dev_noalloc(dX, pkg.NOALLOC_MAX_TILES + 1, None, None)  # refused before any launch
    assert e.value.code == pkg.QTIP_E_ARG and "maximum" in str(e.value)
    qz.synchronize()
