#!/usr/bin/env python3
"""Benchmark of the HEMMer hot path on one MI355X.

Headline metric: ms per 128 x 128 ciphertext-ciphertext matrix product
(HEMMer::singleCCMatMul, N = 2^16, 13 + 4 primes, dnum 3, scale 2^42, inputs fresh at level 12,
target level 4), inputs and keys resident in HBM.  Also reported in the same JSON line: one
key-switched rotation at levels 12 and 6, batched NTT limb-transforms/s, the roofline of the
dominant kernel family (the ModDown chain of the main loop), of the hoisted key-switch sums and of the NTT
launch pair, and the CPU oracle timed on the host cores.

A "step" is one full CCMM.  Everything runs on one GPU; --gpus above 1 is refused.
--roofline-only runs just the roofline legs and --ccmm-only just the headline product loop (used for the committed
rocprofv3 summaries, so that a kernel's average in the profile is the average of exactly the launches timed here).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
LIMB_BYTES = (1 << 16) * 8


def gpu_ccmm(args, out, headline_only=False):
    import numpy as np
    from __graft_entry__ import load_package
    pkg = load_package()
    from efla_amd import hellm
    H = hellm.HEMMer(preset=True, seed=3)
    rng = np.random.default_rng(1)
    A, B = rng.uniform(-1, 1, (128, 128)), rng.uniform(-1, 1, (128, 128))
    ca, cb = H.encrypt(A), H.encrypt(B)
    T = 4
    t0 = time.perf_counter()
    c = H.single_cc_matmul(ca, cb, T)          # first call also builds keys and masks
    H.sync()
    out["setup_s"] = round(time.perf_counter() - t0, 3)
    for _ in range(args.warmup):
        c = H.single_cc_matmul(ca, cb, T)
    H.sync()
    timer = pkg.Timer()
    t0 = time.perf_counter()
    timer.start()
    for _ in range(args.steps):
        c = H.single_cc_matmul(ca, cb, T)
    ev_ms = timer.stop()
    H.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    err = float(np.abs(H.decrypt(c) - A @ B).max())
    out["ms_per_step"] = wall_ms / args.steps
    out["value"] = wall_ms / args.steps
    out["gpu_event_ms_per_step"] = ev_ms / args.steps
    out["max_abs_err"] = err
    out["max_abs_err_ok"] = bool(err <= 2.0 ** -12)
    # algorithmic bytes of one product, counted by the library as it queues the launches: per launch the operands it
    # must read once plus the results it must write once (a two-launch transform = one read and one write per limb)
    H.traffic(reset=True)
    c = H.single_cc_matmul(ca, cb, T)
    H.sync()
    by, ln = H.traffic(reset=True)
    total = sum(by.values())
    out["ccmm_algorithmic_bytes"] = {
        "total": total, "by_kind": by, "launches_by_kind": ln, "launches": sum(ln.values()),
        "achieved_GBps": total / (out["gpu_event_ms_per_step"] * 1e-3) / 1e9,
        "frac_of_hbm_peak": total / (out["gpu_event_ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
    }
    # device memory after the product: evaluation keys by form (the hoisted sums read the compact one) and the buffer
    # pool of the context as a whole (keys, masks, ciphertexts, workspaces)
    out["resident_bytes_after_ccmm"] = H.key_bytes()
    if headline_only:
        return H
    # one rotation (automorphism + hybrid key switch) at the top level
    r = H.left_rotate(ca, 1)
    H.sync()
    timer.start()
    for _ in range(50):
        r = H.left_rotate(ca, 1)
    out["rotation_level12_us"] = timer.stop() / 50 * 1e3
    low = H.level_down(ca, 6)
    r = H.left_rotate(low, 1)
    H.sync()
    timer.start()
    for _ in range(50):
        r = H.left_rotate(low, 1)
    out["rotation_level6_us"] = timer.stop() / 50 * 1e3

    # encode (host message -> device plaintext at level 12: copy, embedding transform, rounding, residues, NTT) and
    # decrypt + decode of the product
    t0 = time.perf_counter()
    for _ in range(20):
        pt = H.encode(B)
    H.sync()
    out["encode_128x128_level12_ms"] = (time.perf_counter() - t0) / 20 * 1e3
    t0 = time.perf_counter()
    for _ in range(20):
        H.decrypt(c)
    out["decrypt_decode_level4_ms"] = (time.perf_counter() - t0) / 20 * 1e3

    # the other product entry points (same context, keys derived on first use; three untimed calls, then 10 timed
    # ones: the first calls of a route also grow the buffer pool)
    def ms(fn, reps=10):
        for _ in range(3):
            fn()
        H.sync()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        H.sync()
        return (time.perf_counter() - t0) / reps * 1e3

    # the same product away from the headline's best case: operands 4 and 3 levels above the target, and operands
    # about whose other slots nothing is known (raw uploads; only B has to be a known single tile for the fast route)
    routes = {}
    for lvl in (12, 8, 7):
        a = H.level_down(ca, lvl) if lvl < 12 else ca
        b = H.level_down(cb, lvl) if lvl < 12 else cb
        ua, ub = H.upload(a.residues(), 128, 128, 128), H.upload(b.residues(), 128, 128, 128)
        routes["level_%d" % lvl] = {"known_single_tiles": ms(lambda: H.single_cc_matmul(a, b, T)),
                                    "A_unknown_B_known": ms(lambda: H.single_cc_matmul(ua, b, T)),
                                    "both_unknown": ms(lambda: H.single_cc_matmul(ua, ub, T))}
    out["ccmm_other_routes_ms"] = routes
    # throughput with two products in flight: a second HEMMer (same seed, its own context, keys and streams) and one
    # recorded product on each, replayed side by side; the headline stays the time of one product on its own
    H2 = hellm.HEMMer(preset=True, seed=3)
    lanes = []
    for Hk in (H, H2):
        xa, xb = Hk.encrypt(A), Hk.encrypt(B)
        Hk.single_cc_matmul(xa, xb, T)
        Hk.sync()
        graph, res = Hk.record(lambda: Hk.single_cc_matmul(xa, xb, T))
        lanes.append((graph, res, xa, xb))

    def replay(graphs, n=20):
        for g in graphs:
            g.launch()
        for g in graphs:
            g.sync()
        t0 = time.perf_counter()
        for _ in range(n):
            for g in graphs:
                g.launch()
        for g in graphs:
            g.sync()
        return (time.perf_counter() - t0) * 1e3 / (n * len(graphs))

    out["ccmm_recorded_replay_ms"] = replay([lanes[0][0]])
    out["ccmm_two_contexts_in_flight_ms_per_product"] = replay([ln[0] for ln in lanes])
    out["ccmm_two_contexts_max_abs_err"] = float(max(np.abs(Hk.decrypt(ln[1]) - A @ B).max()
                                                     for Hk, ln in zip((H, H2), lanes)))
    for ln in lanes:
        ln[0].free()
    del lanes, H2
    A2, B2 = rng.uniform(-1, 1, (128, 128)), rng.uniform(-1, 1, (128, 128))
    pa, pb = H.encrypt2(A, A2), H.encrypt2(B, B2)
    out["ccmm_pair_layout_two_products_ms"] = ms(lambda: H.single_cc_matmul(pa, pb, T))
    ppb = H.encode2(B, B2)
    out["pcmm_pair_layout_two_products_ms"] = ms(lambda: H.single_matmul(pa, ppb, T))
    sb = H.encode(B)
    out["pcmm_single_product_ms"] = ms(lambda: H.single_matmul(ca, sb, T))
    qa, qb = H.encrypt2(A, A2), H.encrypt2(B, B2)
    H.complex_packing_inplace(qa)
    H.complex_packing_row_inplace(qb)
    out["packed_ccmm_two_products_ms"] = ms(lambda: H.packed_matmul(qa, qb, T))
    x = H.complex_packing(H.encrypt2(A, A), H.encrypt2(A2, A2))
    out["hoisted_pcmm_pre_ms"] = ms(lambda: H.matmul_pre(x, T))
    tmp = H.matmul_pre(x, T)
    wp = H.encode_diagonal_to_row4(*[0.02 * rng.normal(size=(128, 128)) for _ in range(4)], level=T + 1)
    out["hoisted_pcmm_reuse_ms"] = ms(lambda: H.matmul_reuse(tmp, wp, T))
    # the other entry points of the path, batched schedule (pair layout where a layout is needed)
    out["transpose_ms"] = ms(lambda: H.transpose_inplace(ca.clone(), T))
    out["diagonal_to_column_level12_ms"] = ms(lambda: H.diagonal_to_column(ca))
    rev = H.matmul_pre_rev(pb, T)
    out["ccmm_pre_rev_ms"] = ms(lambda: H.matmul_pre_rev(pb, T))
    out["ccmm_reuse_ms"] = ms(lambda: H.matmul_cc_reuse(tmp, rev, T))
    return H


def gpu_ntt(args, out):
    import torch
    from __graft_entry__ import load_package
    pkg = load_package()
    limbs = 32 * 24
    res = {}
    for bits in (60, 42):
        qs = pkg.primes_below(bits, 16, 24)
        ctx = pkg.Context(16, qs, [], 1)
        q_t = torch.tensor(qs, dtype=torch.int64, device="cuda").view(1, 24, 1)
        g = torch.Generator(device="cuda").manual_seed(7)
        d = torch.randint(0, 2 ** 62, (32, 24, 1 << 16), dtype=torch.int64, device="cuda", generator=g) % q_t
        ref = d.clone()
        idx = list(range(24))
        for _ in range(3):
            ctx.ntt(d, idx)
            ctx.ntt(d, idx, inverse=True)
        torch.cuda.synchronize()
        assert torch.equal(d, ref), "NTT round trip is not bit-exact"
        timer = pkg.Timer()
        iters = 20
        timer.start()
        for _ in range(iters):
            ctx.ntt(d, idx)
        fwd_ms = timer.stop() / iters
        timer.start()
        for _ in range(iters):
            ctx.ntt(d, idx, inverse=True)
        inv_ms = timer.stop() / iters
        res[bits] = (fwd_ms, inv_ms)
        del ctx, d, ref
    a = torch.empty((32, 24, 1 << 16), dtype=torch.int64, device="cuda").fill_(1)
    b = torch.empty_like(a)
    b.copy_(a)
    timer = pkg.Timer()
    timer.start()
    for _ in range(10):
        b.copy_(a)
        a.copy_(b)
    copy_ms = timer.stop() / 10
    del a, b
    fwd_ms, inv_ms = res[60]
    out["ntt_forward_limbs_per_s"] = limbs / fwd_ms * 1e3
    out["ntt_inverse_limbs_per_s"] = limbs / inv_ms * 1e3
    out["ntt_limbs_per_s"] = 2 * limbs / (fwd_ms + inv_ms) * 1e3
    out["ntt_limbs_per_s_42bit_primes"] = 2 * limbs / (res[42][0] + res[42][1]) * 1e3
    # one forward transform of the batch = one launch of ntt16_cols_kernel + one of ntt16_rows_kernel;
    # algorithmic traffic = read + write of every limb once = 1 MiB per limb-transform (each of the two
    # launches moves that much, so the pair cannot exceed half of the HBM roofline on this figure)
    alg_bytes = limbs * 2 * LIMB_BYTES
    out["roofline_ntt"] = {
        "kernel": "ntt16_cols_kernel<false> + ntt16_rows_kernel<false> (one forward transform of "
                  "32x24 limbs = 2 launches), 60-bit primes / 42-bit primes",
        "bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "achieved": alg_bytes / (fwd_ms * 1e-3) / 1e9, "frac": alg_bytes / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "achieved_42bit": alg_bytes / (res[42][0] * 1e-3) / 1e9,
        "frac_42bit": alg_bytes / (res[42][0] * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "algorithmic_bytes_per_launch_pair": alg_bytes, "avg_ms_per_launch_pair": fwd_ms,
        "avg_ms_per_launch_pair_42bit": res[42][0],
        # the floor of a two-launch transform on this box: two plain device copies of the same 384 MiB
        "two_device_copies_of_the_batch_ms": copy_ms,
        "frac_of_two_copies": copy_ms / fwd_ms, "frac_of_two_copies_42bit": copy_ms / res[42][0],
    }


# HBM bytes per call of the hoisted sum at the shape below (its two launches together), from two rocprofv3 --pmc runs
# of `bench.py --roofline-only` (FETCH_SIZE, WRITE_SIZE), each scaled by what the same counter reads for the
# 1 GiB copy this mode also launches (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0):
# (2 x (159 700.4 + 172 140.0) + 196 608 + 163 840) KiB, see profiles/hoisted_terms_and_ntt_roofline_shapes.txt.
HOISTED_TRAFFIC_BYTES = 1048707891


# HBM bytes of the four launches of one ModDown chain at the shape below, same two counters and scale factors.
MODDOWN_TRAFFIC_BYTES = 1654669312


def gpu_hoisted(args, out):
    """Roofline of the dominant kernels, the hoisted sum of the CCMM's main loop: one call produces 32 column shifts
    of sigma(A) in the extended basis, each the sum of two masked hoisted rotations (of the operand and of its
    copy rotated by -n) under one key (7 chain + 4 special limbs, 2 digits).  The column masks are run tables (their
    NTT form is constant over runs of 256 residues), and a call of this size is two launches over disjoint limbs:
    hoisted_terms_kernel<1, true> (the 6 limbs of primes below 2^44, double precision) and hoisted_terms_kernel<2, true>
    (the 5 limbs of 60-bit primes, integer); the second template argument says that the keys are in the compact layout.  Timed together: the figure is per call."""
    import torch
    from __graft_entry__ import load_package
    pkg = load_package()
    nq, K, dnum, n_out = 7, 4, 3, 32
    big = pkg.primes_below(60, 16, 1 + K)
    qs = [big[0]] + pkg.primes_below(42, 16, 12)
    ps = big[1:]
    ctx = pkg.Context(16, qs, ps, dnum)
    N, E, T, beta, shift = 1 << 16, nq + K, 13 + K, 2, 8
    g = torch.Generator(device="cuda").manual_seed(11)

    def rnd(*shape):
        # residues below 2^41 are valid for every prime of the set; the kernel's work does not depend on values
        return torch.randint(0, 2 ** 41, shape, dtype=torch.int64, device="cuda", generator=g)

    src = [(rnd(beta, E, N), rnd(nq, N)) for _ in range(2)]
    groups = []
    for o in range(n_out):
        # keys in the compact layout, as the product's schedule passes them (6 bytes per residue of a prime below 2^44)
        evk, gal = ctx.compact_key(rnd(dnum, 2, T, N)), pow(5, o + 1, 2 * N)
        groups.append([(src[t][0], src[t][1], evk, rnd(E, N >> shift), gal, shift) for t in range(2)])
    for _ in range(2):
        ctx.hoisted_terms(groups, nq, b_premultiplied=True, compact_keys=True)
    torch.cuda.synchronize()
    timer = pkg.Timer()
    iters = 10
    timer.start()
    for _ in range(iters):
        ctx.hoisted_terms(groups, nq, b_premultiplied=True, compact_keys=True)
    ms = timer.stop() / iters
    # algorithmic bytes: per output beta x 2 x E key limbs read (6 of them 6 bytes per residue, 5 of them 8) + 2 x E
    # limbs written (the mask tables are 2 x E x 4 KiB per output, a value and its Shoup companion per run: counted,
    # negligible); the two rotation sources (beta x E + nq limbs each) read once
    n_small = sum(1 for q in qs[:nq] if q < 2 ** 44)
    key_bytes = beta * 2 * (n_small * 6 + (E - n_small) * 8) * N
    limbs = n_out * 2 * E + 2 * (beta * E + nq)
    alg_bytes = n_out * key_bytes + limbs * LIMB_BYTES + n_out * 2 * E * (N >> shift) * 16
    achieved = alg_bytes / (ms * 1e-3) / 1e9
    out["roofline_hoisted_sum"] = {
        "kernel": "hoisted_terms_kernel<1, true> + hoisted_terms_kernel<2, true> (one hoisted sum of the CCMM main loop: 32 "
                  "outputs x 2 masked sources under one compact key, 7+4 limbs, 2 digits, run-table masks; "
                  "double-precision limbs and integer limbs in one launch each)",
        "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": achieved / HBM_PEAK_GBS, "traffic": HOISTED_TRAFFIC_BYTES,
        "algorithmic_bytes_per_launch": alg_bytes, "avg_ms_per_launch": ms,
    }
    # (b) the hoisted sum of one sigma / tau transform stage, the largest single launch of the product
    # (hoisted_terms_kernel<0, true>): 2 outputs (one per operand) at level T+4, each 7 rotations of two masked sources
    # under one key, full masks over the extended basis (9 + 4 limbs, 2 digits)
    nq2, E2 = 9, 9 + K
    src2 = [[(rnd(beta, E2, N), rnd(nq2, N)) for _ in range(2)] for _ in range(2)]
    groups2 = []
    for o in range(2):
        grp = []
        for r in range(7):
            evk, gal = ctx.compact_key(rnd(dnum, 2, T, N)), pow(5, 8 * o + r + 1, 2 * N)
            grp += [(src2[o][t][0], src2[o][t][1], evk, rnd(E2, N), gal, 0) for t in range(2)]
        groups2.append(grp)
    ctx.traffic(reset=True)
    ctx.hoisted_terms(groups2, nq2, b_premultiplied=True, compact_keys=True)
    stage_bytes = sum(ctx.traffic(reset=True)[0].values())
    torch.cuda.synchronize()
    timer.start()
    for _ in range(iters):
        ctx.hoisted_terms(groups2, nq2, b_premultiplied=True, compact_keys=True)
    ms2 = timer.stop() / iters
    out["roofline_transform_stage"] = {
        "kernel": "hoisted_terms_kernel<0, true> (hoisted sum of one sigma/tau transform stage: 2 outputs x 7 compact keys x 2 "
                  "masked sources, full masks, 9+4 limbs, 2 digits)",
        "bound": "hbm", "achieved": stage_bytes / (ms2 * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": stage_bytes / (ms2 * 1e-3) / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes_per_launch": stage_bytes,
        "avg_ms_per_launch": ms2,
    }
    # (c) the ModDown merged with the rescale of one main-loop batch: 64 polynomials from 7+4 to 6 limbs in four
    # launches (inverse transform of the 5 dropped limbs, forward transform whose first pass computes the basis
    # conversion and whose second ends with the fused (y - conv) / (P q_6) tail)
    y = rnd(64, E, N)
    ctx.traffic(reset=True)
    ctx.moddown_batch(y, nq, True)
    md_by = ctx.traffic(reset=True)[0]
    md_bytes = sum(md_by.values())
    torch.cuda.synchronize()
    timer.start()
    for _ in range(iters):
        ctx.moddown_batch(y, nq, True)
    ms3 = timer.stop() / iters
    # the same arithmetic with the two column passes and the conversion in one kernel per slab (three launches)
    timer.start()
    for _ in range(iters):
        ctx.moddown_batch(y, nq, True, column_slab=True)
    ms3_slab = timer.stop() / iters
    out["roofline"] = {
        "kernel": "ntt16_rows_kernel<true,false> + ntt16_cols_kernel<true> + ntt16_cols_converted_kernel<5> + "
                  "ntt16_rows_kernel<false,true> (ModDown + rescale of one main-loop batch, 64 polynomials, 7+4 -> 6 limbs: "
                  "the largest kernel family of the CCMM; the basis conversion runs inside the first forward pass)",
        "bound": "hbm", "achieved": md_bytes / (ms3 * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": md_bytes / (ms3 * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": MODDOWN_TRAFFIC_BYTES,
        "algorithmic_bytes_per_launch": md_bytes, "avg_ms_per_launch": ms3,
        "algorithmic_bytes_by_kind": {k: v for k, v in md_by.items() if v},
        "column_slab_form_ms": ms3_slab,
    }
    if args.roofline_only:
        # a plain copy of known size in the same process: the scale reference for the --pmc counters
        a = torch.empty(1 << 27, dtype=torch.int64, device="cuda").fill_(1)
        b = torch.empty_like(a)
        for _ in range(4):
            b.copy_(a)
        torch.cuda.synchronize()


def gpu_rotation_60bit(args, out):
    """One key-switched rotation at the reference rotation benchmark's shape: chain of 24 60-bit primes + 4
    special primes, dnum 3, ciphertext at level 20 (random residues and key: timing only)."""
    import torch
    from __graft_entry__ import load_package
    pkg = load_package()
    primes = pkg.primes_below(60, 16, 28)
    ctx = pkg.Context(16, primes[:24], primes[24:], 3)
    g = torch.Generator(device="cuda").manual_seed(5)
    nq, N = 21, 1 << 16
    ct = torch.randint(0, 2 ** 59, (2, nq, N), dtype=torch.int64, device="cuda", generator=g)
    evk = torch.randint(0, 2 ** 59, (3, 2, 28, N), dtype=torch.int64, device="cuda", generator=g)
    for _ in range(3):
        ctx.rotate(ct, evk, 5, nq)
    torch.cuda.synchronize()
    timer = pkg.Timer()
    timer.start()
    for _ in range(30):
        ctx.rotate(ct, evk, 5, nq)
    out["rotation_24x60bit_level20_us"] = timer.stop() / 30 * 1e3


def gpu_pcmm_loop(args, out):
    """A loop of singleMatMul on the pair layout (two 128 x 128 products per call, the weight's tau prepared by the
    warm-up calls), for kernel traces and counters; the figure is an extra key, not the headline."""
    import numpy as np
    from __graft_entry__ import load_package
    load_package()
    from efla_amd import hellm
    H = hellm.HEMMer(preset=True, seed=3)
    rng = np.random.default_rng(1)
    A, A2, B, B2 = (rng.uniform(-1, 1, (128, 128)) for _ in range(4))
    pa, pb = H.encrypt2(A, A2), H.encode2(B, B2)
    for _ in range(max(1, args.warmup)):
        c = H.single_matmul(pa, pb, 4)
    H.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        c = H.single_matmul(pa, pb, 4)
    H.sync()
    out["pcmm_pair_layout_two_products_ms"] = (time.perf_counter() - t0) * 1e3 / args.steps
    d = H.decrypt2(c)
    out["pcmm_max_abs_err"] = float(max(np.abs(d[0] - A @ B).max(), np.abs(d[1] - A2 @ B2).max()))


def gpu_layer_configs(args, out, H):
    """The two layer-level workloads, timed as extra keys (not the headline): the LoRA forward projection and one
    attention block of 12 heads, each with its max abs error against float64 algebra.  Inputs, keys, masks and
    encoded weights are resident before the timed region (a first untimed pass derives them)."""
    import numpy as np
    from efla_amd import hellm
    n, tiles, rank, T = 128, 6, 8, 4
    rng = np.random.default_rng(10)
    X = 0.1 * rng.normal(size=(n, n * tiles))
    W = 0.02 * rng.normal(size=(n * tiles, n * tiles))
    A = 0.02 * rng.normal(size=(n * tiles, rank))
    B = 0.02 * rng.normal(size=(rank, n * tiles))
    xt = [X[:, i * n:(i + 1) * n] for i in range(tiles)]
    # activations: complex-packed pairs of tiles for the frozen weight, single tiles for the encrypted LoRA factors
    xp = [H.complex_packing(H.encrypt2(xt[i], xt[i]), H.encrypt2(xt[i + 1], xt[i + 1])) for i in range(0, tiles, 2)]
    cx = [H.encrypt(t) for t in xt]
    t0 = time.perf_counter()
    wp = {}
    for j in range(0, tiles, 2):
        for i in range(0, tiles, 2):
            w = [W[r * n:(r + 1) * n, c * n:(c + 1) * n] for r in (i, i + 1) for c in (j, j + 1)]
            wp[i, j] = H.encode_diagonal_to_row4(w[0], w[1], w[2], w[3], level=T + 1)
    H.sync()
    out["config4_weight_encoding_ms"] = (time.perf_counter() - t0) * 1e3    # 36 weight tiles as 9 groups of 4
    ca, cb = [], []
    for i in range(tiles):
        Ai, Bi = np.zeros((n, n)), np.zeros((n, n))
        Ai[:, :rank] = A[i * n:(i + 1) * n]
        Bi[:rank] = B[:, i * n:(i + 1) * n]
        ca.append(H.encrypt(Ai))
        cb.append(H.encrypt(Bi))

    def lora_projection():
        pre = [H.matmul_pre(x, T) for x in xp]                         # hoisted shifts of the three activation pairs
        ys = []
        for j in range(0, tiles, 2):                                   # 36 weight tiles = 9 reuse products of 4 tiles
            acc = None
            for p_, i in enumerate(range(0, tiles, 2)):
                y = H.matmul_reuse(pre[p_], wp[i, j], T)
                acc = y if acc is None else H.add(acc, y)
            ys.append(H.repack_cc(acc))
        xa = None
        for i in range(tiles):                                         # X A: 6 products accumulated, level 7
            t = H.single_cc_matmul(cx[i], ca[i], 7)
            xa = t if xa is None else H.add(xa, t)
        zs = [H.single_cc_matmul(xa, cb[j], 4) for j in range(tiles)]  # (X A) B: 6 products, level 4
        return ys, zs

    ys, zs = lora_projection()
    H.sync()
    t0 = time.perf_counter()
    ys, zs = lora_projection()
    H.sync()
    out["config4_lora_projection_ms"] = (time.perf_counter() - t0) * 1e3
    want = X @ W
    err = 0.0
    for k, y in enumerate(ys):
        z = H.decrypt2(y)
        err = max(err, float(np.abs(z[0] - want[:, 2 * k * n:(2 * k + 1) * n]).max()),
                  float(np.abs(z[1] - want[:, (2 * k + 1) * n:(2 * k + 2) * n]).max()))
    want = X @ A @ B
    for j, z in enumerate(zs):
        err = max(err, float(np.abs(H.decrypt(z) - want[:, j * n:(j + 1) * n]).max()))
    out["config4_max_abs_err"] = err
    out["config4_workload"] = ("X 128x768 (6 tiles) x plaintext W 768x768: 3 matMulPre + 9 matMulReUse of 4 weight tiles "
                               "(36 tile products) + repackCC; encrypted rank-8 factors zero-padded to 128-wide tiles: "
                               "6 CCMM (X A, level 7) + 6 CCMM ((X A) B, level 4)")
    del xp, cx, wp, ca, cb, ys, zs

    # attention block of 12 heads with the Gaussian-kernel score; the level checks of the preset ("bootstrap below
    # level 7") are lifted by a second evaluator over the same primes
    H2 = hellm.HEMMer(16, H.q, H.p, dnum=3, min_bootstrap_level=0, seed=3)
    rng = np.random.default_rng(14)
    Q, K, V = (0.1 * rng.normal(size=(n, 12 * 64)) for _ in range(3))
    cts = gk_attention_inputs(H2, Q, K, V, range(3))
    outs = gk_attention(H2, cts)
    H2.sync()
    t0 = time.perf_counter()
    outs = gk_attention(H2, cts)
    H2.sync()
    out["config5_attention_block_ms"] = (time.perf_counter() - t0) * 1e3
    out["config5_max_abs_err"] = gk_attention_error(H2, outs, Q, K, V, range(3))
    out["config5_workload"] = ("12 heads of dim 64 at seq 128, two heads per 128-wide tile, two tiles per ciphertext: per "
                               "ciphertext maskRightLeft of Q, K, V, squares and oneMatRotSumInplace for the row norms, "
                               "transposeInplace of the key norms; per masked half a CCMM Q K^T (two heads per call, level 8), "
                               "-2 QK^T + |q|^2 + |k|^2, the degree-15 Chebyshev table of exp(-x / (2 sqrt 64)) with 4 baby "
                               "steps (level 4), a CCMM scores x V (level 1): 24 products + 6 polynomial evaluations on two "
                               "heads each")


GK_INTERVAL = (0.5, 2.5)      # |q - k|^2 of 64-dimensional 0.1 N(0,1) vectors: 0.02 chi^2_128-like, mean 1.28


def gk_table():
    """Degree-15 Chebyshev interpolant of the Gaussian-kernel score exp(-x / (2 sqrt(64))) on GK_INTERVAL mapped to
    [-1, 1] (an interval of length 2: the map is a subtraction, no level), in the product basis with 4 baby steps."""
    import numpy as np
    from numpy.polynomial import chebyshev as C
    from efla_amd import hellm
    mid = 0.5 * (GK_INTERVAL[0] + GK_INTERVAL[1])
    return hellm.chebyshev_product_basis(C.chebinterpolate(lambda t: np.exp(-(t + mid) / 16.0), 15), 4)


def gk_attention_inputs(H2, Q, K, V, pairs):
    """Pair-layout ciphertexts of the 128-wide tiles 2i and 2i+1 of Q, K, V (two heads of 64 columns per tile) and of
    the transposed key tiles, fresh at the top level."""
    n = 128
    tile = lambda M, t: M[:, t * n:(t + 1) * n]
    return [(H2.encrypt2(tile(Q, 2 * i), tile(Q, 2 * i + 1)), H2.encrypt2(tile(K, 2 * i), tile(K, 2 * i + 1)),
             H2.encrypt2(tile(K, 2 * i).T, tile(K, 2 * i + 1).T), H2.encrypt2(tile(V, 2 * i), tile(V, 2 * i + 1)))
            for i in pairs]


def gk_attention(H2, cts, score_level=8, out_level=1):
    """The attention scores of the reference's layer (src/TransformerBlock.cpp:2415-2501, src/HEMMer.cpp:882-919,
    1245-1249): heads split by maskRightLeft, |q|^2 and |k|^2 by squaring and oneMatRotSumInplace (the key norms
    transposed), -2 Q K^T + |q|^2 + |k|^2, then exp(-x / (2 sqrt 64)) -- as a degree-15 Chebyshev table where the
    reference bootstraps and runs exp_iter_Parallel -- and the product with the masked V.  Returns per ciphertext
    and per half the tensor holding scores x V of two heads (one per tile)."""
    table = gk_table()
    outs = []
    for q, k, kt, v in cts:
        mq, mk, mv = H2.mask_right_left(q), H2.mask_right_left(k), H2.mask_right_left(v)
        sq, sk = [H2.mult(x, x) for x in mq], [H2.mult(x, x) for x in mk]
        H2.one_mat_rot_sum_inplace(sq[0], sq[1])          # row norms of either half, spread over the tile rows
        H2.one_mat_rot_sum_inplace(sk[0], sk[1])
        for j in (0, 1):
            H2.transpose_inplace(sk[j], score_level)      # key norms along the columns
            s = H2.single_cc_matmul(mq[j], kt, score_level)
            x = H2.add(H2.add(H2.mult_const(s, -2.0), H2.level_down(sq[j], score_level)), sk[j])
            p = H2.eval_chebyshev(H2.linear_transform(x, *GK_INTERVAL), table, 4)
            outs.append(H2.single_cc_matmul(p, mv[j], out_level))
    return outs


def gk_attention_error(H2, outs, Q, K, V, pairs):
    import numpy as np
    err, d = 0.0, 64
    for a, i in enumerate(pairs):
        for j in (0, 1):
            z = H2.decrypt2(outs[2 * a + j])
            for t in (0, 1):
                h = 2 * (2 * i + t) + j
                q, k, v = (M[:, h * d:(h + 1) * d] for M in (Q, K, V))
                dist = (q * q).sum(1)[:, None] + (k * k).sum(1)[None, :] - 2.0 * q @ k.T
                want = np.exp(-dist / 16.0) @ v
                err = max(err, float(np.abs(z[t][:, j * d:(j + 1) * d] - want).max()))
    return err


def cpu_baseline(out):
    """The CPU oracle (C++ port of the same arithmetic) on the GPU box's host cores.

    cpu_baseline: ONE whole product of the headline workload -- the oracle's restatement of exactly the launch
    schedule the GPU runs (complex-packed single-tile CCMM, same operation order, same residues) -- on all the cores
    this job may use (the oracle threads over limbs), timed on its second pass so that key derivation stays outside,
    as it does for the GPU.  cpu_baseline_1_thread: a bounded sample of the reference's
    operation order on one thread, scaled by the operation counts of one product (a whole product would take
    about two minutes on one thread)."""
    import numpy as np
    from oracle import hemmer_ref as R
    from oracle import oracle as O
    cores = max(1, min(16, os.cpu_count() or 1))
    qs, ps = O.ckks_chain(16, 13, 4)
    orc = O.Oracle(16, qs, ps, dnum=3, threads=cores)
    orc.gen_secret(3)
    orc.key_seed = 3
    orc.gen_mult_key(3)
    orc.gen_conj_key(3)
    rng = np.random.default_rng(1)
    n = 128
    A, B = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))

    def enc(M, seed):
        z = np.zeros(orc.slots, dtype=np.complex128)
        z[:M.size] = M.reshape(-1)
        return orc.encrypt(orc.encode(z, orc.nQ - 1), seed)

    ca, cb = enc(A, 11), enc(B, 12)
    t0 = time.perf_counter()
    R.mult_mat_mat_cc_packed_single(orc, ca, cb, 4, n, n)       # untimed pass: derives every evaluation key on first use
    first_s = time.perf_counter() - t0
    t0 = time.perf_counter()
    c = R.mult_mat_mat_cc_packed_single(orc, ca, cb, 4, n, n)   # timed pass: the product only, keys resident
    full_s = time.perf_counter() - t0
    err = float(np.abs(orc.decrypt(c)[:n * n].real.reshape(n, n) - A @ B).max())
    out["cpu_baseline"] = {
        "value": full_s * 1e3, "unit": "ms", "cores": cores, "kind": "port",
        "sample": "one whole 128x128 singleCCMatMul on the CPU oracle (restatement of the batched complex-packed "
                  "schedule the GPU runs, N=2^16, 13+4 primes, level 12 -> 4), evaluation keys resident as on the GPU "
                  "(derived by an untimed first pass), %d threads over limbs; max abs error %.2e" % (cores, err),
        "key_derivation_s": max(0.0, first_s - full_s), "resident_keys": len(orc.keys),
    }
    orc1 = O.Oracle(16, qs, ps, dnum=3, threads=1)
    orc1.gen_secret(3)
    orc1.key_seed = 3
    orc1.gen_mult_key(3)
    z = rng.uniform(-1, 1, orc1.slots).astype(np.complex128)
    ct12 = orc1.encrypt(orc1.encode(z, 12), 4)
    ct6 = orc1.level_down(ct12, 6)
    ct5 = orc1.level_down(ct12, 5)
    m12, m6 = orc1.encode(z, 12), orc1.encode(z, 6)
    orc1.left_rotate(ct6, 1)   # derive the key outside the timed region

    def t(fn, reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return (time.perf_counter() - t0) / reps

    t_rot12 = t(lambda: orc1.left_rotate(ct12, 1), 1)
    t_rot6 = t(lambda: orc1.left_rotate(ct6, 1), 2)
    t_mul12 = t(lambda: orc1.mult_plain_no_rescale(ct12, m12), 2)
    t_mul6 = t(lambda: orc1.mult_plain_no_rescale(ct6, m6), 2)
    pre = orc1.mult_plain_no_rescale(ct6, m6)
    t_res6 = t(lambda: orc1.rescale(pre), 2)
    t_tensor5 = t(lambda: orc1.tensor(ct5, ct5), 2)
    t3 = orc1.tensor(ct5, ct5)
    t_relin5 = t(lambda: orc1.relinearize(t3), 1)
    # operation counts of one 128 x 128 CCMM in the reference's order: 2 transforms (32 rotations + 255 mask
    # products each at level 12), 508 rotations + 508 mask products + 254 rescales at level 6, 127 tensor
    # products, 2 relinearisations
    total = (64 * t_rot12 + 510 * t_mul12 + 508 * t_rot6 + 508 * t_mul6 + 254 * t_res6 +
             128 * t_tensor5 + 2 * t_relin5)
    out["cpu_baseline_1_thread"] = {
        "value": total * 1e3, "unit": "ms", "cores": 1, "kind": "port",
        "sample": "CPU oracle, 1 thread, the reference's operation order: timed 1 rotation + 2 mask products at "
                  "level 12, 2 rotations, 2 mask products, 2 rescales at level 6, 2 tensor products + 1 "
                  "relinearisation at level 5; scaled by the operation counts of one CCMM "
                  "(64/510/508/508/254/128/2)",
        "rotation_level12_ms": t_rot12 * 1e3, "rotation_level6_ms": t_rot6 * 1e3,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--roofline-only", action="store_true", help="run only the roofline legs")
    ap.add_argument("--ccmm-only", action="store_true", help="run only the headline product loop (for kernel traces)")
    ap.add_argument("--pcmm-only", action="store_true",
                    help="run only a loop of pair-layout plaintext x ciphertext products (for kernel traces)")
    ap.add_argument("--rotation-only", action="store_true",
                    help="run only the single key-switched rotation at the 24 x 60-bit shape (for kernel traces)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures the one-GPU hot path only: run it with --gpus 1 "
              "(no multi-GPU figure is produced by this build)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU fallback for the product path)", file=sys.stderr)
        sys.exit(3)
    out = {
        "metric": "ms per 128x128 CCMM (N=2^16) on 1 GPU", "value": None, "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": None, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "u64", "data": "synthetic",
        "config": {"workload": "singleCCMatMul 128x128 U(-1,1) seeded, N=2^16, 13 chain (60-bit + 12x42-bit) "
                               "+ 4 special 60-bit primes, dnum=3, scale 2^42, inputs fresh at level 12, "
                               "target level 4, all keys and masks resident in HBM"},
    }
    if args.rotation_only:
        gpu_rotation_60bit(args, out)
        print(json.dumps(out))
        return
    if args.roofline_only:
        gpu_hoisted(args, out)
        gpu_ntt(args, out)
        print(json.dumps(out))
        return
    if args.pcmm_only:
        gpu_pcmm_loop(args, out)
        print(json.dumps(out))
        return
    H = gpu_ccmm(args, out, headline_only=args.ccmm_only)
    if args.ccmm_only:
        print(json.dumps(out))
        return
    gpu_layer_configs(args, out, H)
    del H
    gpu_hoisted(args, out)
    gpu_ntt(args, out)
    gpu_rotation_60bit(args, out)
    if not args.no_cpu:
        cpu_baseline(out)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
