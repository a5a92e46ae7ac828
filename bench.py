#!/usr/bin/env python3
"""Benchmark of the QTIP per-Hessian-group quantize path on one MI355X.

A step is one pass of the hot path over one synthetic group: Hessian rotation (GPU), fp64 block LDL (host),
weight RHT + Wscale, LDLQ with the two-pass Viterbi, packing to the kernel-layout trellis.  Default workload:
benchmark configuration 5, the 12288 x 28672 down-proj group.  The K timed steps are K groups handled the way the
reference's scheduler handles consecutive groups (src/pipeline.cpp:254-290): Hessians are rotated ahead of use
(two groups ahead, through a ring of three staging buffers), a side thread factors them in order, and the GPU
quantizes group k as soon as its factor is ready, so the host LDL of group k+1 overlaps the GPU work of group k;
the scheduling is the library's own (qtip_run_groups).
Nothing is precomputed outside the timed region; the first group's LDL is fully exposed.

Prints ONE JSON line (see the keys below).  `value` is weights quantized per second over the whole timed region.
"""
import argparse
import json
import os
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FLOP_PER_WEIGHT = 393216.0      # 2^16 add-compare-selects per weight, counted as 6 flop each
PEAK_FP64_TFLOPS = 78.6         # MI355X vector fp64
PEAK_32BIT_TFLOPS = 157.3       # MI355X vector fp32: the rate of 32-bit lanes, which the u32 path metrics run on
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
HBM_BYTES_PER_WEIGHT = 2040.0   # algorithmic HBM traffic of the Viterbi per weight (4-bit back-pointers of two passes + X)


def load_pkg():
    from __graft_entry__ import _pkg
    return _pkg()


def load_synth():
    import importlib.util
    spec = importlib.util.spec_from_file_location("qtip_synth", os.path.join(ROOT, "behemoth-qtip_amd", "synth.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def cpu_viterbi_sample(seconds_budget, threads):
    """Reference CPU Viterbi (oracle/_ref when present, else the oracle port) on a bounded sample of tiles."""
    import concurrent.futures as cf
    import numpy as np
    from oracle import binding as ob
    R = ob.ref_lib()
    kind = "reference" if R is not None else "port"
    cb = ob.Codebook()
    X = ob.rng_normal(77, 4096 * 256).astype(np.float32).astype(np.float16).astype(np.float32).reshape(4096, 256)
    done = [0]
    lock = threading.Lock()
    deadline = time.time() + seconds_budget

    def work(lo):
        st = np.zeros(128, np.uint16)
        hat = np.zeros(256, np.float32)
        n = 0
        for b in range(lo, 4096, threads):
            if time.time() > deadline:
                break
            if R is not None:
                R.ref_quantize_seq(X[b], st, hat)
            else:
                ob.lib().qo_quantize_seq(cb.lut0, cb.lut1, X[b], st, hat)
            n += 1
        with lock:
            done[0] += n

    t0 = time.time()
    with cf.ThreadPoolExecutor(threads) as ex:
        list(ex.map(work, range(threads)))
    dt = time.time() - t0
    return {"value": done[0] * 256 / dt / 1e6, "unit": "Mweights/s", "cores": threads, "kind": kind,
            "sample": "%d tiles of 256 fp16-rounded N(0,1) weights, two-pass Viterbi only (the dominant stage), "
                      "%.1f s on %d threads" % (done[0], dt, threads)}


def cpu_baseline(threads=16, group=None):
    """The CPU path timed on this host.  Always: the reference's CPU Viterbi on a sample of tiles.  With `group`
    (n, weights, HRr, L of the benchmark's group, host arrays): the group path as the reference's CPU code would run
    it, from two bounded samples: the CPU LDLQ (oracle port of tests/test_gpu.cpp:180-225: fp64 feedback, fp16
    rounding, two-pass Viterbi per tile) on 256 weight rows over the last 4096 columns of the group (its own factor),
    and the reference's compiled block_ldl_to_L on the group's rotated Hessian in full.  `value` extrapolates the
    LDLQ sample's rate to the group's weights and adds the factorization."""
    import numpy as np
    from oracle import binding as ob
    vit = cpu_viterbi_sample(10.0 if group else 15.0, threads)
    if not group:
        return vit
    n, weights, HRr, L = group
    ncol = min(n, 4096)
    rows = 16 * threads
    Lsub = np.ascontiguousarray(L[n - ncol:, n - ncol:])
    Wr = (ob.rng_normal(78, rows * ncol).reshape(rows, ncol) * (0.9 * ob.Codebook().lut_rms)).astype(np.float32)
    t0 = time.time()
    ob.ldlq(ob.Codebook(), Wr, Lsub, threads=threads)
    t_ldlq = time.time() - t0
    ldlq_rate = rows * ncol / t_ldlq
    out = {"unit": "Mweights/s", "cores": threads, "kind": "port", "viterbi_only": vit,
           "ldlq_sample_Mweights_s": ldlq_rate / 1e6,
           "sample": "CPU LDLQ (port) on %d rows x the last %d columns of the group with the group's own factor, rows "
                     "drawn at the rotated weights' scale, %.1f s on %d threads; extrapolated to %d weights"
                     % (rows, ncol, t_ldlq, threads, weights)}
    R = ob.ref_lib()
    t_ldl = None
    if R is not None:
        A = np.empty((n, n), np.float64)
        for i in range(0, n, 2048):       # 0.5 (H + H^T) as the reference's ldl_hessian forms it, not timed
            A[i:i + 2048] = 0.5 * (HRr[i:i + 2048].astype(np.float64) + HRr[:, i:i + 2048].T.astype(np.float64))
        Lr = np.zeros((n, n), np.float32)
        t0 = time.time()
        ok = R.ref_block_ldl(A.reshape(-1), n, Lr.reshape(-1), threads)
        t_ldl = time.time() - t0
        out["block_ldl_reference_s"] = t_ldl
        out["block_ldl_reference_same_factor_bits"] = bool(ok == 1 and np.array_equal(Lr.view(np.uint32), L.view(np.uint32)))
        out["sample"] += "; block_ldl_to_L of the compiled reference on the group's rotated Hessian (n = %d) in full, " \
                         "%.1f s on %d threads" % (n, t_ldl, threads)
        del A, Lr
    out["value"] = weights / (weights / ldlq_rate + (t_ldl or 0.0)) / 1e6
    return out


def run_viterbi_only(args, pkg):
    """Configuration 1: 4096 independent tiles, Viterbi only."""
    import numpy as np
    import torch
    synth = load_synth()
    q = pkg.Quantizer(0, tlut=synth.synthetic_tlut(1))
    q.set_viterbi_mode(1 if args.viterbi_fp64 else 0)
    X = torch.from_numpy(synth.splitmix_normal(1234, 4096 * 256).astype(np.float32).reshape(4096, 256)).cuda()
    S = torch.zeros((4096, 128), dtype=torch.int16, device="cuda")
    P = torch.zeros((4096, 32), dtype=torch.int16, device="cuda")
    for _ in range(args.warmup):
        q.viterbi_tiles_dev(X, 4096, S, P)
    q.synchronize()
    torch.cuda.synchronize()
    t0 = time.time()
    for _ in range(args.steps):
        q.viterbi_tiles_dev(X, 4096, S, P)
    q.synchronize()
    torch.cuda.synchronize()
    dt = time.time() - t0
    weights = 4096 * 256 * args.steps
    per_launch = dt / args.steps
    return dict(weights=weights, wall=dt, vit_launch_s=per_launch, vit_launch_weights=4096 * 256,
                workload="config1: 4096 independent 16x16 tiles, Viterbi only", extra={})


def run_group(args, pkg):
    import numpy as np
    import torch
    synth = load_synth()
    q = pkg.Quantizer(0)
    cfg = args.config
    if cfg == 2:
        Ws_h, H_h = synth.config2()
        Ws = [torch.from_numpy(w).cuda() for w in Ws_h]
        H = torch.from_numpy(H_h).cuda()
    else:
        Ws, H = synth.large_config(cfg)
    n = H.shape[0]
    ms = [int(w.shape[0]) for w in Ws]
    lins = [pkg.LinearIn("w%d" % i, m, w_f32=w) for i, (m, w) in enumerate(zip(ms, Ws))]
    opt = pkg.QuantOpts(ldl_threads=args.ldl_threads, skip_proxy=False, feedback=args.feedback,
                        ldl_device_updates=not args.host_ldl, ldlq_chains=args.chains, group_lanes=args.lanes)
    weights_per_step = sum(ms) * n

    stats = {}

    def run_steps(K, record):
        """K groups through the library's scheduler: the Hessian of group k+2 is rotated and the one of group k+1 is
        factored on a side thread while the GPU quantizes group k.  Every group does all of quantize_group's work,
        the two proxy errors included."""
        res = q.run_groups([(lins, n, H, 3 + k) for k in range(K)], opt)
        if record:
            tms = [r[1] for r in res]
            stats.update(rht_s=sum(t.rht for t in tms) / K,      # Hessian rotation + weight RHT + Wscale
                         ldl_s=sum(t.ldl_cpu for t in tms) / K, ldl_wait_s=sum(r[2] for r in res) / K,
                         ldlq_s=sum(t.ldlq for t in tms) / K, viterbi_s=sum(t.viterbi for t in tms) / K,
                         load_s=sum(t.load for t in tms) / K, pack_s=sum(t.pack for t in tms) / K,
                         proxy_s=sum(t.proxy for t in tms) / K, proxy=float(res[-1][0][0].proxy),
                         wscale=float(res[-1][0][0].wscale), cmp_outs=res[min(K, 6) - 1][0],
                         cmp_outs3=res[min(K, 3) - 1][0])

    q.reserve_groups(n)   # page-locked staging ring (3 x (HRr, L)); a worker keeps it for its lifetime
    q.set_viterbi_mode(1 if args.viterbi_fp64 else 0)
    if args.warmup > 0:
        run_steps(args.warmup, False)
    q.synchronize()
    torch.cuda.synchronize()
    q.viterbi_stats(reset=True)
    t0 = time.time()
    run_steps(args.steps, True)
    q.synchronize()
    torch.cuda.synchronize()
    wall = time.time() - t0
    redone = q.viterbi_stats(reset=True)   # passes of the timed region that were run again on fp64 metrics
    tiles_timed = (sum(ms) // 16) * (n // 16) * args.steps
    vit = dict(viterbi_metrics="fp64" if args.viterbi_fp64 else
               "u32 in units of 2^-k, k even per pass, 26 for normalized weights (errors formed in fp64), a pass repeated on fp64 metrics when a traced decision "
               "is won by less than 160 units",
               viterbi_first_passes_repeated=redone[0], viterbi_second_passes_repeated=redone[1],
               viterbi_repeated_share=(redone[0] + redone[1]) / (2.0 * tiles_timed))
    legs = {}
    if not args.viterbi_fp64 and not args.no_fp64_leg:
        # beside it (outside the timed region): three groups with fp64 path metrics only, the arithmetic of the CPU
        # algorithm; every word of the output must be the same
        kf = min(args.steps, 3)
        q.set_viterbi_mode(1)
        q.synchronize()
        tf = time.time()
        fres = q.run_groups([(lins, n, H, 3 + k) for k in range(kf)], opt)
        q.synchronize()
        tf = time.time() - tf
        q.set_viterbi_mode(0)
        legs.update(fp64_metrics_Mweights_s=weights_per_step * kf / tf / 1e6, fp64_metrics_groups=kf,
                    fp64_metrics_viterbi_s=sum(r[1].viterbi for r in fres) / kf,
                    fp64_metrics_same_codes=bool(all(np.array_equal(a.trellis, b.trellis) and a.proxy == b.proxy
                                                     for a, b in zip(fres[-1][0], stats["cmp_outs3"]))))
        del fres
    if args.chains == 0 and not args.no_chains2_leg:
        # beside it: three groups with two LDLQ chains, what a caller gets whose context found fewer than three side
        # streams with hardware queues of their own when it was made
        kc = min(args.steps, 3)
        copt = pkg.QuantOpts(ldl_threads=args.ldl_threads, skip_proxy=False, feedback=args.feedback,
                             ldl_device_updates=not args.host_ldl, ldlq_chains=2, group_lanes=args.lanes)
        q.synchronize()
        tc = time.time()
        cres = q.run_groups([(lins, n, H, 3 + k) for k in range(kc)], copt)
        q.synchronize()
        tc = time.time() - tc
        legs.update(chains2_Mweights_s=weights_per_step * kc / tc / 1e6, chains2_groups=kc,
                    chains2_same_codes=bool(all(np.array_equal(a.trellis, b.trellis) and a.proxy == b.proxy
                                                for a, b in zip(cres[-1][0], stats["cmp_outs3"]))))
        del cres
    host_only = {}
    if not args.host_ldl and not args.no_host_ldl_leg:
        # beside it (outside the timed region): the same groups with the block LDL on the host alone, as the
        # reference factors; fewer groups, so the one exposed factorization at the start weighs more
        kh = min(args.steps, 6)
        hopt = pkg.QuantOpts(ldl_threads=args.ldl_threads, skip_proxy=False, feedback=args.feedback,
                             ldl_device_updates=False, ldlq_chains=args.chains, group_lanes=args.lanes)
        q.synchronize()
        th = time.time()
        hres = q.run_groups([(lins, n, H, 3 + k) for k in range(kh)], hopt)
        q.synchronize()
        th = time.time() - th
        host_only = dict(host_ldl_Mweights_s=weights_per_step * kh / th / 1e6, host_ldl_groups=kh,
                         host_ldl_s=sum(r[1].ldl_cpu for r in hres) / kh,
                         host_ldl_same_codes=bool(all(np.array_equal(a.trellis, b.trellis) and a.proxy == b.proxy
                                                      for a, b in zip(hres[-1][0], stats["cmp_outs"]))))
    host_inputs = {}
    if not args.no_host_input_leg:
        # beside it (outside the timed region): the same groups with W and H handed over as host pointers, as the
        # reference's entry point takes them (src/quantizer.hpp:21-28,75-77): pageable host memory, PCIe inside.
        # As many groups as the timed region, so that the first group's upload and factorization, which nothing
        # hides, weigh on both figures alike
        kq = min(args.steps, 16)
        lins_h = [pkg.LinearIn("w%d" % i, m, w_f32=w.cpu().numpy()) for i, (m, w) in enumerate(zip(ms, Ws))]
        H_host = H.cpu().numpy()
        q.synchronize()
        th = time.time()
        hres = q.run_groups([(lins_h, n, H_host, 3 + k) for k in range(kq)], opt)
        q.synchronize()
        th = time.time() - th
        host_inputs = dict(host_inputs_Mweights_s=weights_per_step * kq / th / 1e6, host_inputs_groups=kq,
                           host_inputs_load_s=sum(r[1].load for r in hres) / kq,
                           host_inputs_same_codes=bool(all(np.array_equal(a.trellis, b.trellis) and a.proxy == b.proxy
                                                           for a, b in zip(hres[min(kq, 6) - 1][0], stats["cmp_outs"]))))
        del lins_h, H_host, hres
    fb1 = {}
    if args.feedback == 0 and not args.no_feedback1_leg:
        # beside it (outside the timed region): the same groups with the LDLQ feedback in the reference GPU's
        # arithmetic (fp32 sums, prod cache from bf16 hi/lo split operands on the matrix cores)
        kf = min(args.steps, 3)
        fopt = pkg.QuantOpts(ldl_threads=args.ldl_threads, skip_proxy=False, feedback=1,
                             ldl_device_updates=not args.host_ldl, ldlq_chains=args.chains, group_lanes=args.lanes)
        q.synchronize()
        tf = time.time()
        fres = q.run_groups([(lins, n, H, 3 + k) for k in range(kf)], fopt)
        q.synchronize()
        tf = time.time() - tf
        a, b = fres[-1][0][0], stats["cmp_outs3"][0]
        same = np.all(a.trellis.reshape(-1, 32) == b.trellis.reshape(-1, 32), axis=1).mean()
        fb1 = dict(feedback1_Mweights_s=weights_per_step * kf / tf / 1e6, feedback1_groups=kf,
                   feedback1_ldlq_s=sum(r[1].ldlq for r in fres) / kf, feedback1_proxy=float(a.proxy),
                   feedback1_word_blocks_equal_to_default=float(same))
        del fres
    cpu_group = None
    if not args.no_cpu_baseline:
        hp = q.rotate_hessian(H, n, 3)
        q.ldl_hessian_device_updates(hp, threads=args.ldl_threads)
        cpu_group = (n, weights_per_step, hp.HRr, hp.L)
    stats.pop("cmp_outs", None)
    stats.pop("cmp_outs3", None)
    ntr = sum(ms) // 16
    launches = n // 128   # one Viterbi launch per 128-column buffer and chain: a workgroup takes its tile row through 8 column blocks
    # the library's rule: three chains where its side streams have hardware queues of their own (it times them when
    # the context is made) or the environment promises 6 queues, else two; a chain must fill its share of the 768
    # resident workgroups
    nch = args.chains or q.ldlq_default_chains()
    while nch > 1 and ntr < 768:
        nch -= 1
    # groups too small to fill the chip run side by side (qtip_opts.group_lanes): that many times as many launches
    # share the chip
    lanes = q.group_lanes([(ms, n)] * args.steps, opt)
    gpu_s = stats["rht_s"] + stats["load_s"] + stats["ldlq_s"] + stats["proxy_s"] + stats["pack_s"]
    extra = dict(stats)
    extra.update(gpu_only_Mweights_s=weights_per_step / gpu_s / 1e6,
                 serial_Mweights_s=weights_per_step / (gpu_s + stats["ldl_s"]) / 1e6,
                 viterbi_only_Mweights_s=weights_per_step / stats["viterbi_s"] / 1e6,
                 proxy_in_timed_region=True, ldl_threads=args.ldl_threads, feedback=args.feedback,
                 hw_queues=int(os.environ.get("GPU_MAX_HW_QUEUES", "4")), ldlq_chains=nch, group_lanes=lanes,
                 ldl_device_updates=not args.host_ldl)
    extra.update(vit)
    extra.update(legs)
    extra.update(host_only)
    extra.update(host_inputs)
    extra.update(fb1)
    names = {2: "config2: 1024x1024 group", 3: "config3: 12288x12288 q-proj group",
             4: "config4: gate+up 2x(28672x12288) group", 5: "config5: 12288x28672 down-proj group"}
    return dict(weights=weights_per_step * args.steps, wall=wall, vit_launch_s=stats["viterbi_s"] / launches,
                vit_launch_weights=ntr * 256 * 8 * lanes, blocks_per_launch=8, workload=names[cfg] + (" (RHT + host fp64 LDL + LDLQ + 2-pass Viterbi + pack)" if args.host_ldl else
                                       " (RHT + fp64 LDL: host panels, GPU trailing updates + LDLQ + 2-pass Viterbi + pack)"),
                extra=extra, cpu_group=cpu_group, concurrent=nch * lanes,
                ldlq_s=stats["ldlq_s"], weights_per_step=weights_per_step)


def run_ldl_only(args, pkg):
    """The factorization alone (nothing else on the GPU): seconds per call for both forms, and whether the two
    factors are the same bits."""
    import numpy as np
    synth = load_synth()
    q = pkg.Quantizer(0)
    if args.config == 2:
        _, H_h = synth.config2()
        import torch
        H = torch.from_numpy(H_h).cuda()
    else:
        _, H = synth.large_config(args.config if args.config != 1 else 5)
    n = H.shape[0]
    hp = q.rotate_hessian(H, n, 3)
    del H
    import torch
    dev, host, resident = [], [], []
    for _ in range(3):
        q.ldl_hessian_device_updates(hp, threads=args.ldl_threads)
        dev.append(hp.t_ldl)
    L_dev = hp.L
    # the form the group pipeline runs: rotated Hessian resident on the device, L into a page-locked buffer that exists
    # already and, as it is assembled, into a device buffer
    dHRr = torch.from_numpy(hp.HRr).cuda()
    L_pin = torch.empty((n, n), dtype=torch.float32, pin_memory=True)
    dL = torch.empty((n, n), dtype=torch.float32, device="cuda")
    for _ in range(4):
        L_pin.fill_(-1.0)
        dL.fill_(-1.0)
        torch.cuda.synchronize()
        resident.append(q.ldl_hessian_device_resident(dHRr, n, L_pin, dL, threads=args.ldl_threads))
    resident = resident[1:]  # the first call allocates the work buffers
    same_resident = bool(np.array_equal(L_pin.numpy().view(np.uint32), L_dev.view(np.uint32))) and \
        bool(torch.equal(dL.cpu(), L_pin))
    del dHRr, dL
    reps = 1 if args.host_ldl_once else 3
    for _ in range(reps):
        pkg.Quantizer.ldl_hessian(hp, threads=args.ldl_threads)
        host.append(hp.t_ldl)
    same = bool(np.array_equal(L_dev.view(np.uint32), hp.L.view(np.uint32)))
    print(json.dumps({"workload": "block LDL alone, n = %d" % n, "device_resident_s": resident,
                      "device_updates_host_in_out_s": dev, "host_only_s": host,
                      "same_factor_bits": same and same_resident, "ldl_threads": args.ldl_threads}), flush=True)


def run_rht_only(args, pkg):
    """The row transform alone (hadK (x) H_1024 over rows resident in HBM, in place): milliseconds per pass and the
    HBM rate of one read and one write of the matrix, for the shapes the large configurations transform."""
    import torch
    q = pkg.Quantizer(0)
    out = []
    for rows, n in ((28672, 28672), (12288, 28672), (28672, 12288), (12288, 12288)):
        X = torch.randn(rows, n, device="cuda")
        q.hadamard_rows_dev(X, rows, n, n, True)
        q.synchronize()
        torch.cuda.synchronize()
        best = None
        for _ in range(max(args.steps, 3)):
            t0 = time.time()
            q.hadamard_rows_dev(X, rows, n, n, True)
            q.synchronize()
            torch.cuda.synchronize()
            dt = time.time() - t0
            best = dt if best is None else min(best, dt)
        nbytes = 2.0 * rows * n * 4
        out.append({"rows": rows, "n": n, "ms": best * 1e3, "bytes": nbytes,
                    "roofline": {"bound": "hbm", "achieved": nbytes / best / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                 "frac": nbytes / best / 1e9 / PEAK_HBM_GBS}})
        del X
    print(json.dumps({"workload": "RHT rows alone (sign-free pass, transposed factor), best of %d" % max(args.steps, 3),
                      "passes": out}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed groups (default 16; 48 for --config 2, whose groups run twelve at a time)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed groups before them (default 1; 12 for --config 2)")
    ap.add_argument("--config", type=int, default=5, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--ldl-threads", type=int, default=16, help="OpenMP team of the host LDL")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--host-ldl", action="store_true",
                    help="keep the fp64 block LDL on the host alone, as the reference does (default: the host factors and "
                         "solves the panels and hands the trailing updates to the GPU; the factor is the same bit for bit)")
    ap.add_argument("--ldl-only", action="store_true",
                    help="time the block LDL of the configuration's rotated Hessian by itself, three times each: host panels "
                         "with GPU trailing updates, and host alone (not the contract's metric; one line of JSON)")
    ap.add_argument("--rht-only", action="store_true",
                    help="time the row transform by itself on the large configurations' shapes (not the contract's "
                         "metric; one line of JSON with the HBM rate of each pass)")
    ap.add_argument("--host-ldl-once", action="store_true", help="with --ldl-only: one host-only factorization instead of three")
    ap.add_argument("--no-host-input-leg", action="store_true",
                    help="skip the extra groups with W and H passed as host pointers reported beside the default run")
    ap.add_argument("--no-feedback1-leg", action="store_true",
                    help="skip the extra groups with --feedback 1 reported beside the default run")
    ap.add_argument("--no-host-ldl-leg", action="store_true",
                    help="skip the extra host-only-LDL groups reported beside the default run")
    ap.add_argument("--feedback", type=int, default=0, choices=[0, 1],
                    help="0: fp64 LDLQ feedback (default); 1: fp32 feedback + bf16 hi/lo split MFMA prod cache")
    ap.add_argument("--chains", type=int, default=0, choices=[0, 1, 2, 3],
                    help="independent chains of launches LDLQ deals the tile rows to (0: the library's default)")
    ap.add_argument("--lanes", type=int, default=0,
                    help="groups qtip_run_groups runs side by side (0: the library's rule: as many as fit the chip, 1 "
                         "for the large configurations; 1: one after the other)")
    ap.add_argument("--hw-queues", type=int, default=None,
                    help="GPU_MAX_HW_QUEUES for this process (set before the HIP runtime starts; 0: leave the environment "
                         "alone; default: 0, and 16 for --config 2).  The three chains of launches of a large group "
                         "find their hardware queues among HIP's default of 4 (the library times its side streams "
                         "when a context is made); small groups run side by side on as many lanes as there are queues")
    ap.add_argument("--viterbi-fp64", action="store_true",
                    help="fp64 path metrics only (default: 32-bit metrics first, a pass repeated on fp64 metrics when a "
                         "traced decision is too close; same codes)")
    ap.add_argument("--no-fp64-leg", action="store_true",
                    help="skip the extra groups with fp64 path metrics only reported beside the default run")
    ap.add_argument("--no-chains2-leg", action="store_true",
                    help="skip the extra groups with two LDLQ chains reported beside the default run")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="first run one plain 1 GiB device copy kernel (known traffic, scales the rocprof byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (given SU, L and Wscale every 16-row "
              "tile row of a group is independent, so the path would shard by tile rows without any exchange)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    if args.hw_queues is None:
        args.hw_queues = 16 if args.config == 2 else 0
    if args.steps is None:
        args.steps = 48 if args.config == 2 else 16
    if args.warmup is None:
        args.warmup = 12 if args.config == 2 else 1
    if args.hw_queues > 0:
        os.environ["GPU_MAX_HW_QUEUES"] = str(min(args.hw_queues, 32))   # read by the HIP runtime when it starts, below
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    pkg = load_pkg()
    if args.pmc_calibration:
        a = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        b = torch.empty_like(a)
        torch.cuda.synchronize()
        b.copy_(a)          # 1 GiB read + 1 GiB written by one elementwise kernel
        torch.cuda.synchronize()
        del a, b
    if args.ldl_only:
        return run_ldl_only(args, pkg)
    if args.rht_only:
        return run_rht_only(args, pkg)
    res = run_viterbi_only(args, pkg) if args.config == 1 else run_group(args, pkg)
    value = res["weights"] / res["wall"] / 1e6
    achieved = res["vit_launch_weights"] * FLOP_PER_WEIGHT / res["vit_launch_s"] / 1e12
    # counters of the same launch, collected offline with rocprofv3 --pmc (a profiler cannot run inside this process):
    # HBM bytes per launch and the share of cycles the LDS pipe is busy; the files name the commands that made them
    traffic, counters = None, {}
    try:
        traffic = json.load(open(os.path.join(ROOT, "profiles", "viterbi_traffic.json"))).get(
            "config%d_bytes_per_launch%s" % (args.config, "_fp64" if args.viterbi_fp64 else ""))
    except Exception:
        traffic = None
    try:
        counters = json.load(open(os.path.join(ROOT, "profiles", "viterbi_counters.json"))).get(
            "config%d%s" % (args.config, "_fp64" if args.viterbi_fp64 else ""), {})
    except Exception:
        counters = {}
    fp64_only = args.viterbi_fp64
    peak = PEAK_FP64_TFLOPS if fp64_only else PEAK_32BIT_TFLOPS
    alg_traffic = HBM_BYTES_PER_WEIGHT * res["vit_launch_weights"] / res.get("concurrent", 1)
    roof = {"bound": "valu", "kernel": "viterbi_tiles_kernel", "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
            "frac": achieved / peak,
            "peak_is": "MI355X vector fp64" if fp64_only else
                       "MI355X vector rate of 32-bit lanes (the published fp32 figure): the path metrics are u32",
            "frac_of_fp64_vector_peak": achieved / PEAK_FP64_TFLOPS,
            # HBM bytes of one launch: measured (rocprofv3 --pmc, offline) against the algorithmic figure
            "traffic": traffic, "traffic_algorithmic": alg_traffic,
            "traffic_ratio": (traffic / alg_traffic) if traffic else None,
            "traffic_source": "profiles/viterbi_traffic.json (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE; offline)",
            "launch_ms": res["vit_launch_s"] * 1e3, "weights_per_launch": res["vit_launch_weights"],
            "concurrent_launches": res.get("concurrent", 1),
            "tiles_per_launch": res["vit_launch_weights"] // 256 // res.get("concurrent", 1) // res.get("blocks_per_launch", 1),
            "column_blocks_per_launch": res.get("blocks_per_launch", 1),
            "flop_per_weight": FLOP_PER_WEIGHT,
            "lds_frac": counters.get("lds_active_frac"), "valu_frac": counters.get("valu_busy_frac"),
            "counters_source": "profiles/viterbi_counters.json (rocprofv3 --pmc SQ_*; offline)"}
    if res.get("ldlq_s"):
        # the same algorithmic work over the whole LDLQ stage (gathers included) and over a whole step (everything)
        roof["frac_ldlq"] = res["weights_per_step"] * FLOP_PER_WEIGHT / res["ldlq_s"] / 1e12 / peak
        roof["frac_step"] = res["weights_per_step"] * FLOP_PER_WEIGHT / (res["wall"] / args.steps) / 1e12 / peak
    out = {
        "metric": "Mweights/s quantized (RHT+LDLQ+2-pass Viterbi) 12288x28672; % VALU/LDS peak",
        "value": value, "unit": "Mweights/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": res["wall"] / args.steps * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f64" if fp64_only else "u32", "data": "synthetic",
        "config": dict({"workload": res["workload"]}, **res["extra"]),
        # launch_ms: the average duration of one Viterbi launch (a start and a stop event stamped by every launch of
        # the timed region itself); concurrent_launches of them run side by side, each taking tiles_per_launch tile
        # rows through column_blocks_per_launch column blocks, so weights_per_launch weights pass in that time
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(threads=min(16, os.cpu_count() or 1), group=res.get("cpu_group"))
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
