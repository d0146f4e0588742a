"""Bit-exact GPU-vs-oracle checks at the full ring (N = 2^16) and at the shapes the benchmark times:

* the hoisted sum of the CCMM main loop at its benchmark shape (32 outputs, two masked sources under one key,
  7 + 4 limbs, 2 digits, run-table masks), which is large enough to be launched as two kernels (double-precision
  limbs / integer limbs), through the kernel-argument path and the staged-list path, and with every operand at q - 1;
* masked sums at N = 2^16 through both paths and for 1, 2 and 3 polynomials;
* one whole 128 x 128 singleCCMatMul on the preset, residue for residue against the oracle running the same
  schedule (keys derived from the same seed on both sides);
* one key-switched rotation per step of the set {1, 2, 4, ..., 64} and multiples of 128, ciphertext at level 20 of a
  chain of 24 60-bit primes + 4 special primes, dnum 3, with the ModUp / inner product / ModDown stages at that shape."""
import os

import numpy as np
import pytest

from __graft_entry__ import load_package
from oracle import hemmer_ref as R
from oracle import oracle as O
from oracle.oracle import _p

pytestmark = pytest.mark.gpu
THREADS = max(1, min(16, os.cpu_count() or 1))


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int64)).cuda()


def host(t):
    return t.cpu().numpy().view(np.uint64)


def rand_limbs(rng, mods, shape_prefix, N):
    out = np.empty(tuple(shape_prefix) + (len(mods), N), dtype=np.uint64)
    for j, q in enumerate(mods):
        out[..., j, :] = rng.integers(0, q, tuple(shape_prefix) + (N,), dtype=np.uint64)
    return out


class Bench:
    """Preset-sized context (13 + 4 primes, dnum 3) with random sources, keys and column masks at nq = 7."""

    def __init__(self):
        pkg = load_package()
        self.log_n, self.N, self.nq = 16, 1 << 16, 7
        qs, ps = O.ckks_chain(16, 13, 4)
        self.orc = O.Oracle(16, qs, ps, 3, threads=THREADS)
        self.ctx = pkg.Context(16, qs, ps, 3)
        orc, nq, N = self.orc, self.nq, self.N
        self.beta = (nq + orc.alpha - 1) // orc.alpha
        assert self.beta == 2 and orc.nP == 4
        self.ext_mods = [orc.mods[i] for i in orc.ext_primes(nq - 1)]
        rng = np.random.default_rng(2024)
        self.ext = [np.ascontiguousarray(rand_limbs(rng, self.ext_mods, (self.beta,), N)) for _ in range(4)]
        self.b = [rand_limbs(rng, orc.q[:nq], (), N) for _ in range(4)]
        self.evk = [np.ascontiguousarray(rand_limbs(rng, orc.mods, (orc.dnum, 2), N)) for _ in range(4)]
        self.gal = [orc.galois(r) for r in (1, 37, orc.slots - 128, 2048)]
        col = np.arange(orc.slots) % 128
        self.shift = self.log_n - 8
        self.masks = []
        for k in (1, 37, 64, 127):
            main = orc.encode_ext((col < 128 - k).astype(float), nq - 1)
            wrap = orc.encode_ext((col >= 128 - k).astype(float), nq - 1)
            self.masks.append((main, wrap))
        self.d_ext = [dev(x) for x in self.ext]
        self.d_b = [dev(x) for x in self.b]
        self.d_evk = [dev(x) for x in self.evk]
        self.d_evk_compact = [self.ctx.compact_key(k) for k in self.d_evk]   # 6 bytes per residue of a prime below 2^44
        self.d_full = [(dev(m.data), dev(w.data)) for m, w in self.masks]
        self.d_tab = [(self.ctx.compact_mask(m, self.shift), self.ctx.compact_mask(w, self.shift)) for m, w in self.d_full]
        assert all(t is not None for pair in self.d_tab for t in pair)

    def want(self, spec):
        """spec: tuple of (source, key, mask pair, half) -> y[2][E][N] on the oracle."""
        orc = self.orc
        y = np.zeros((2, self.nq + orc.nP, self.N), dtype=np.uint64)
        for i, (s, k, m, half) in enumerate(spec):
            orc.L.orc_hoisted_term(orc.h, _p(self.ext[s]), _p(self.b[s]), _p(self.evk[k]), _p(self.masks[m][half].data),
                                   self.gal[k], self.nq, _p(y), int(i > 0))
        return y

    def term(self, s, k, m, half, table=True, compact=False):
        mask = self.d_tab[m][half] if table else self.d_full[m][half]
        key = self.d_evk_compact[k] if compact else self.d_evk[k]
        return (self.d_ext[s], self.d_b[s], key, mask, self.gal[k], self.shift if table else 0)


@pytest.fixture(scope="module")
def bench():
    return Bench()


def check_outputs(bench, specs, y):
    cache = {}
    for o, spec in enumerate(specs):
        if spec not in cache:
            cache[spec] = bench.want(spec)
        assert np.array_equal(y[o], cache[spec]), (o, spec)


def test_hoisted_sum_at_the_main_loop_shape_two_launches(bench):
    """32 outputs x (main, wrap) halves of one shift under one key: one merged two-source term per output, list and
    outputs within the kernel-argument capacity, 32 * 11 * 128 = 45056 workgroups -> one launch for the
    double-precision limbs and one for the integer limbs."""
    specs = []
    for o in range(32):
        k, m = o % 4, (o // 4) % 4
        s0, s1 = (o // 2) % 4, (o // 2 + 1 + o % 3) % 4
        specs.append(((s0, k, m, 0), (s1, k, m, 1)))
    groups = [[bench.term(*t) for t in spec] for spec in specs]
    y = host(bench.ctx.hoisted_terms(groups, bench.nq))
    check_outputs(bench, specs, y)
    # the same sums on compact keys (the layout the products use): the <1, true> / <2, true> launches
    groups = [[bench.term(*t, compact=True) for t in spec] for spec in specs]
    assert np.array_equal(host(bench.ctx.hoisted_terms(groups, bench.nq, compact_keys=True)), y)


def test_hoisted_sum_staged_term_list_two_launches(bench):
    """The same size with two shifts per output (64 merged terms: beyond the kernel-argument capacity, so the term
    list is staged in device memory), full masks beside run tables, and a third, single term on some outputs."""
    specs = []
    for o in range(32):
        k, m = o % 4, (o // 4) % 4
        k2, m2 = (k + 1) % 4, (m + 2) % 4
        s0, s1 = (o // 2) % 4, (o // 2 + 1) % 4
        spec = [(s0, k, m, 0), (s1, k, m, 1), (s1, k2, m2, 0), (s0, k2, m2, 1)]
        if o % 5 == 0:
            spec.append((o % 4, (k + 2) % 4, m, 1))
        specs.append(tuple(spec))
    # the two halves of a shift use the same kind of mask (run table or full), so that they merge under their key
    groups = [[bench.term(*t, table=((i // 2) + o) % 3 != 0) for i, t in enumerate(spec)] for o, spec in enumerate(specs)]
    y = host(bench.ctx.hoisted_terms(groups, bench.nq))
    check_outputs(bench, specs, y)
    groups = [[bench.term(*t, table=((i // 2) + o) % 3 != 0, compact=True) for i, t in enumerate(spec)]
              for o, spec in enumerate(specs)]
    assert np.array_equal(host(bench.ctx.hoisted_terms(groups, bench.nq, compact_keys=True)), y)


def test_hoisted_sum_two_launches_every_operand_at_q_minus_one(bench):
    """Largest sums the reductions of both launches see: sources, b, key and masks all q - 1, at the split size."""
    orc, ctx, N, nq = bench.orc, bench.ctx, bench.N, bench.nq
    top = lambda primes, prefix: np.ascontiguousarray(
        np.stack([np.full(tuple(prefix) + (N,), q - 1, dtype=np.uint64) for q in primes], axis=len(prefix)))
    ext, b = top(bench.ext_mods, (bench.beta,)), top(orc.q[:nq], ())
    evk, mask = top(orc.mods, (orc.dnum, 2)), top(bench.ext_mods, ())
    dext, db, dk, dm = dev(ext), dev(b), dev(evk), dev(mask)
    tm = ctx.compact_mask(dm, bench.shift)
    assert tm is not None
    g1, g2 = bench.gal[1], bench.gal[2]
    kinds = [[(dext, db, dk, tm, g1, bench.shift), (dext, db, dk, tm, g1, bench.shift)],      # merged, run tables
             [(dext, db, dk, dm, g2), (dext, db, dk, dm, g2)],                                # merged, full masks
             [(dext, db, dk, dm, g1), (dext, db, dk, None, g2)]]                              # single terms
    groups = [kinds[o % 3] for o in range(32)]
    y = host(ctx.hoisted_terms(groups, nq))
    want = []
    for terms in ([(mask, g1), (mask, g1)], [(mask, g2), (mask, g2)], [(mask, g1), (None, g2)]):
        w = np.zeros((2, nq + orc.nP, N), dtype=np.uint64)
        for i, (mk, g) in enumerate(terms):
            orc.L.orc_hoisted_term(orc.h, _p(ext), _p(b), _p(evk), _p(mk) if mk is not None else None, g, nq, _p(w),
                                   int(i > 0))
        want.append(w)
    for o in range(32):
        assert np.array_equal(y[o], want[o % 3]), o
    # compact key with every residue q - 1: the high halves of the 12-byte records at their largest
    dkc = ctx.compact_key(dk)
    groups_c = [[(t[0], t[1], dkc) + tuple(t[3:]) for t in g] for g in groups]
    assert np.array_equal(host(ctx.hoisted_terms(groups_c, nq, compact_keys=True)), y)


@pytest.mark.parametrize("n_polys", [1, 2, 3])
def test_masked_sums_full_ring_both_paths(bench, n_polys):
    """out[o] = sum_t mask_t * ct_t over nq limbs at N = 2^16: a short list (kernel arguments) and a long one (staged),
    with unmasked terms and a mask read through an automorphism."""
    orc, ctx, N, nq = bench.orc, bench.ctx, bench.N, bench.nq
    rng = np.random.default_rng(5 + n_polys)
    mods = orc.q[:nq]
    cts = [rand_limbs(rng, mods, (n_polys,), N) for _ in range(3)]
    dcts = [dev(c) for c in cts]
    pts = [orc.encode(rng.uniform(-1, 1, orc.slots), nq - 1) for _ in range(3)]
    dpts = [dev(p.data) for p in pts]
    g = orc.galois(5)

    def one(spec):
        acc = None
        for (ci, pi, gal) in spec:
            x = O.Ct(cts[ci], 1.0)
            if pi is not None:
                p = pts[pi] if not gal else orc.left_rotate(pts[pi], 5)
                x = orc.mult_plain_no_rescale(x, p)
            acc = x if acc is None else orc.add(acc, x)
        return acc.data

    short = [((0, 0, 0), (1, None, 0)), ((2, 1, 1),), ((1, 2, 0), (2, 0, 0), (0, 1, 1))]
    long_ = [tuple(((o + t) % 3, (o + 2 * t) % 3 if (o + t) % 4 else None, (t % 5 == 1) and (o + t) % 4 != 0)
                   for t in range(5)) for o in range(8)]
    for specs in (short, long_):
        groups = [[(dcts[ci], dpts[pi] if pi is not None else None, g if gal else 0) for (ci, pi, gal) in spec]
                  for spec in specs]
        got = host(ctx.masked_sum_batch(groups, nq, n_polys))
        for o, spec in enumerate(specs):
            assert np.array_equal(got[o], one(spec)), (o, spec)


@pytest.fixture(scope="module")
def preset():
    """The preset evaluator and the oracle over the same primes with keys from the same seed."""
    load_package()
    from efla_amd import hellm
    H = hellm.HEMMer(preset=True, seed=3)
    qs, ps = O.ckks_chain(16, 13, 4)
    orc = O.Oracle(16, qs, ps, dnum=3, threads=THREADS)
    orc.gen_secret(3)
    orc.gen_mult_key(3)
    orc.gen_conj_key(3)
    orc.key_seed = 3
    assert np.array_equal(H.secret_coeffs(), orc.sk_coeffs)
    return H, orc, R.OracleEval(orc)


def as_oracle(orc, ct):
    i = ct.info()
    assert i["rescale_counter"] == 0
    return O.Ct(ct.residues(), orc.delta[i["level"]])


def test_preset_pcmm_residues_bit_exact(preset):
    """singleMatMul at N = 2^16 (the 127 shifts as terms of one sum dealt to 16 partial outputs, the weight read
    through a second automorphism, one ModDown): a single tile in the first block and the pair layout, residue for
    residue against the oracle's restatement of that schedule."""
    H, orc, ev = preset
    rng = np.random.default_rng(31)
    A, B, A2, B2 = (rng.uniform(-1, 1, (128, 128)) for _ in range(4))
    top = orc.delta[orc.nQ - 1]
    ca, pb = H.encrypt(A), H.encode(B)
    c = H.single_matmul(ca, pb, 4)
    want = R.mult_mat_mat_pc_lazy(orc, as_oracle(orc, ca), O.Pt(pb.residues(), top), 4, 128, 128)
    assert c.info()["level"] == 4 == want.level
    assert np.array_equal(c.residues(), want.data)
    assert np.abs(H.decrypt(c) - A @ B).max() < 2.0 ** -12
    ca2, pb2 = H.encrypt2(A, A2), H.encode2(B, B2)
    c2 = H.single_matmul(ca2, pb2, 4)
    want2 = R.mult_mat_mat_pc_lazy(orc, as_oracle(orc, ca2), O.Pt(pb2.residues(), top), 4, 128, 256)
    assert np.array_equal(c2.residues(), want2.data)
    d = H.decrypt2(c2)
    assert np.abs(d[0] - A @ B).max() < 2.0 ** -12 and np.abs(d[1] - A2 @ B2).max() < 2.0 ** -12


def test_preset_pair_layout_and_packed_ccmm_residues_bit_exact(preset):
    """singleCCMatMul on the pair layout (two products per call) and packedMatMul + repackCC at N = 2^16."""
    H, orc, ev = preset
    rng = np.random.default_rng(32)
    A, B, A2, B2 = (rng.uniform(-1, 1, (128, 128)) for _ in range(4))
    pa, pb = H.encrypt2(A, A2), H.encrypt2(B, B2)
    oa, ob = as_oracle(orc, pa), as_oracle(orc, pb)
    c = H.single_cc_matmul(pa, pb, 4)
    assert np.array_equal(c.residues(), R.mult_mat_mat_cc_packed_single(orc, oa, ob, 4, 128, 256).data)
    d = H.decrypt2(c)
    assert np.abs(d[0] - A @ B).max() < 2.0 ** -12 and np.abs(d[1] - A2 @ B2).max() < 2.0 ** -12
    H.complex_packing_inplace(pa)
    H.complex_packing_row_inplace(pb)
    oa, ob = R.complex_packing_cols(ev, oa, 128, 256), R.complex_packing_rows(ev, ob, 128, 256)
    assert np.array_equal(pa.residues(), oa.data) and np.array_equal(pb.residues(), ob.data)
    prod = H.packed_matmul(pa, pb, 4)
    want = R.mult_packed_mat_mat_fused(orc, oa, ob, 4, 128, 256)
    assert np.array_equal(prod.residues(), want.data)
    pc = H.repack_cc(prod)
    assert np.array_equal(pc.residues(), R.repack_cc(ev, want).data)
    d = H.decrypt2(pc)
    assert np.abs(d[0] - A @ B).max() < 2.0 ** -12 and np.abs(d[1] - A2 @ B2).max() < 2.0 ** -12


def test_preset_hoisted_pcmm_and_transpose_residues_bit_exact(preset):
    """matMulPre (all 128 shifted copies) + matMulReUse on a complex-packed activation pair, and transposeInplace of a
    pair-layout ciphertext, at N = 2^16."""
    H, orc, ev = preset
    n = 128
    rng = np.random.default_rng(33)
    X0, X1 = 0.1 * rng.normal(size=(n, n)), 0.1 * rng.normal(size=(n, n))
    W = [rng.normal(0, 0.02, (n, n)) for _ in range(4)]
    x = H.complex_packing(H.encrypt2(X0, X0), H.encrypt2(X1, X1))
    ox = as_oracle(orc, x)
    tmp = H.matmul_pre(x, 4)
    otmp = R.mult_mat_mat_pre_fused(orc, ox, 4, n, 2 * n)
    assert len(tmp) == n == len(otmp)
    for k in range(n):
        assert np.array_equal(tmp.get(k, n, n, 2 * n).residues(), otmp[k].data), k
    wp = H.encode_diagonal_to_row4(*W, level=5)
    owp = orc.encode(R.weights_diagonal_to_row4(*W, orc.slots), 5)
    assert np.array_equal(wp.residues(), owp.data)
    y = H.matmul_reuse(tmp, wp, 4)
    assert np.array_equal(y.residues(), R.mult_mat_mat_reuse(ev, otmp, owp, 4).data)
    z = H.decrypt2(H.repack_cc(y))
    assert np.abs(z[0] - (X0 @ W[0] + X1 @ W[2])).max() < 2.0 ** -12
    assert np.abs(z[1] - (X0 @ W[1] + X1 @ W[3])).max() < 2.0 ** -12
    A, A2 = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    t = H.encrypt2(A, A2)
    want = R.diagonal_transform_fused(orc, as_oracle(orc, t), R.DIAG_SIGNED, n, 2 * n)
    H.transpose_inplace(t)
    assert np.array_equal(t.residues(), want.data)
    d = H.decrypt2(t)
    assert np.abs(d[0] - A.T).max() < 2.0 ** -12 and np.abs(d[1] - A2.T).max() < 2.0 ** -12


def test_preset_ccmm_residues_bit_exact(preset):
    """singleCCMatMul of two fresh 128 x 128 tiles on the preset (N = 2^16, 13 + 4 primes, dnum 3, target level 4):
    every residue of the result equals the oracle's, which runs the same schedule with keys from the same seed."""
    H, orc, _ = preset
    rng = np.random.default_rng(1)
    A, B = rng.uniform(-1, 1, (128, 128)), rng.uniform(-1, 1, (128, 128))
    ca, cb = H.encrypt(A), H.encrypt(B)
    c = H.single_cc_matmul(ca, cb, 4)
    top = orc.delta[orc.nQ - 1]
    want = R.mult_mat_mat_cc_packed_single(orc, O.Ct(ca.residues(), top), O.Ct(cb.residues(), top), 4, 128, 128)
    assert c.info()["level"] == 4 == want.level
    assert np.array_equal(c.residues(), want.data)
    assert np.abs(H.decrypt(c) - A @ B).max() < 2.0 ** -12
    # the same operands three levels above the target with nothing known about their content (a raw upload): the
    # complex packing and the packed transform as one composite transform, then 63 + 63 masked cell shifts
    la, lb = H.level_down(ca, 7), H.level_down(cb, 7)
    ua, ub = H.upload(la.residues(), 128, 128, 128), H.upload(lb.residues(), 128, 128, 128)
    c3 = H.single_cc_matmul(ua, ub, 4)
    d7 = orc.delta[7]
    want3 = R.mult_mat_mat_cc_packed(orc, O.Ct(ua.residues(), d7), O.Ct(ub.residues(), d7), 4, 128, 128, single_tile=False)
    assert c3.info()["level"] == 4 == want3.level
    assert np.array_equal(c3.residues(), want3.data)
    assert np.abs(H.decrypt(c3) - A @ B).max() < 2.0 ** -12
    # three levels above the target as known single tiles: B's row shifts are exact rotations, so B takes the packing
    # and the first stage of tau as one composite map and then the second stage, beside A's composite transform
    c4 = H.single_cc_matmul(la, lb, 4)
    want4 = R.mult_mat_mat_cc_packed(orc, O.Ct(la.residues(), d7), O.Ct(lb.residues(), d7), 4, 128, 128, single_tile=True)
    assert c4.info()["level"] == 4 == want4.level
    assert np.array_equal(c4.residues(), want4.data)
    assert np.abs(H.decrypt(c4) - A @ B).max() < 2.0 ** -12


def test_preset_two_stream_products_repeat_bit_for_bit(preset):
    """The products whose operands take their own ways on two streams (singleCCMatMul of single tiles, packedMatMul)
    and the one-ModDown PCMM, called eight times in turn on the same operands: every call returns the residues of
    the first.  A launch of one chain that read what the other had not finished writing, or two users of one
    workspace, would show up as a call that differs."""
    H, orc, _ = preset
    rng = np.random.default_rng(41)
    A, B, A2, B2 = (rng.uniform(-1, 1, (128, 128)) for _ in range(4))
    ca, cb = H.encrypt(A), H.encrypt(B)
    pa, pb = H.encrypt2(A, A2), H.encrypt2(B, B2)
    H.complex_packing_inplace(pa)
    H.complex_packing_row_inplace(pb)
    wb = H.encode(B)
    first = None
    for it in range(8):
        got = (H.single_cc_matmul(ca, cb, 4).residues(), H.packed_matmul(pa, pb, 4).residues(),
               H.single_matmul(ca, wb, 4).residues())
        if first is None:
            first = got
            continue
        for k, (x, y) in enumerate(zip(got, first)):
            assert np.array_equal(x, y), (it, k)


def test_preset_polynomials_reductions_and_low_rank_product_residues_bit_exact(preset):
    """The rows around the matrix products at N = 2^16 on the preset, residue for residue against the oracle's
    restatements: Exp::exp_iter and its pairwise form, the reference's EXP_15_4 Chebyshev table (4 baby steps), the
    rotate-and-sum reductions of the pair layout, and a LoRA low-rank product (multMatMatHighLow) with its repacking."""
    from oracle import poly_ref as P
    from tests.test_poly_eval import EXP_15_4
    H, orc, ev = preset
    n, w, ld = 128, 256, R.LOW_DIM
    rng = np.random.default_rng(34)
    # polynomial evaluation
    M = rng.uniform(-1, 1, (n, n))
    ct = H.level_down(H.encrypt(M), 8)
    oct_ = as_oracle(orc, ct)
    got = H.exp_iter(ct, 3)
    assert np.array_equal(got.residues(), P.exp_iter(ev, oct_, 3).data)
    assert np.abs(H.decrypt(got) - (1 + M / 8) ** 8).max() < 2.0 ** -16
    pair = [H.level_down(H.encrypt(rng.uniform(-1, 1, (n, n))), 6) for _ in range(2)]
    opair = [as_oracle(orc, c) for c in pair]
    H.exp_iter_parallel(pair, 2)
    for c, want in zip(pair, P.exp_iter_parallel(ev, opair, 2)):
        assert np.array_equal(c.residues(), want.data)
    got = H.eval_chebyshev(ct, EXP_15_4, 4, 0.5)
    want = P.eval_chebyshev(ev, oct_, EXP_15_4, 4, 0.5)
    assert got.info()["level"] == want.level and np.array_equal(got.residues(), want.data)
    # reductions on the pair layout
    A, B = rng.normal(size=(n, n)), rng.normal(size=(n, n))
    x = H.encrypt2(A, B)
    ox = as_oracle(orc, x)
    scaled = np.zeros((n, n))
    scaled[:, 0] = 1.0 / (2 * n)
    red = x.clone()
    H.reduce_row_sum_with_scaled_mask(red, scaled, np.zeros((n, n)))
    want = R.reduce_row_sum_with_scaled_mask(ev, ox, R._message2(scaled, np.zeros((n, n)), orc.slots), 2 * n, True)
    assert np.array_equal(red.residues(), want.data)
    mean = np.concatenate([A, B], axis=1).mean(axis=1, keepdims=True)
    assert np.abs(H.decrypt2(red)[0] - mean).max() < 2.0 ** -18
    a, b = x.clone(), x.clone()
    H.one_mat_rot_sum_inplace(a, b)
    wa, wb = R.one_mat_rot_sum(ev, ox, ox, n, True)
    assert np.array_equal(a.residues(), wa.data) and np.array_equal(b.residues(), wb.data)
    # a low-rank product: X (two tiles) times the block of ld columns of the LoRA factor, then repacked into one column block
    blk = 3
    thin = lambda: np.pad(rng.normal(0, 0.5, (n, ld)), ((0, 0), (blk * ld, n - (blk + 1) * ld)))
    X0, X1, A0, A1 = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n)), thin(), thin()
    cx, ca = H.encrypt2(X0, X1), H.encrypt2(A0, A1)
    ocx, oca = as_oracle(orc, cx), as_oracle(orc, ca)
    low = H.get_low_col_block(ca, blk)
    olow = R.get_low_col_block(ev, oca, blk, n, n, w, ld)
    assert np.array_equal(low.residues(), olow.data)
    prod = H.matmul_high_low(cx, low, blk, 3)
    want = R.mult_mat_mat_high_low(ev, ocx, olow, blk, 3, (n, n), (n, n), w, ld, orc)
    assert prod.info()["level"] == 3 and np.array_equal(prod.residues(), want.data)
    one = H.repack_to_one_col(prod, 0)
    assert np.array_equal(one.residues(), R.repack_to_one_col(ev, want, 0, n, n, w, ld).data)
    XA = X0 @ A0[:, blk * ld:(blk + 1) * ld] + X1 @ A1[:, blk * ld:(blk + 1) * ld]
    for half in H.decrypt2(one):
        assert np.abs(half[:, :ld] - XA).max() < 2.0 ** -12 and np.abs(half[:, ld:]).max() < 2.0 ** -12


def test_preset_other_low_rank_forms_residues_bit_exact(preset):
    """multMatMatLowHigh with repackToMultiRow / OneRow, multMatMatLowLow and the element-wise rank-2 LoRA path
    (down and up projection) at N = 2^16 on the preset, residue for residue against the oracle."""
    H, orc, ev = preset
    n, w, ld = 128, 256, R.LOW_DIM
    rng = np.random.default_rng(35)
    rows_of = lambda blk: np.pad(rng.normal(0, 0.5, (ld, n)), ((blk * ld, n - (blk + 1) * ld), (0, 0)))
    cols_of = lambda blk: np.pad(rng.normal(0, 0.5, (n, ld)), ((0, 0), (blk * ld, n - (blk + 1) * ld)))
    blk = 2
    L0 = rows_of(blk)
    G0, G1 = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    ca, cg = H.encrypt2(L0, L0), H.encrypt2(G0, G1)
    oa, og = as_oracle(orc, ca), as_oracle(orc, cg)
    low = H.get_low_row_block(ca, blk)
    olow = R.get_low_row_block(ev, oa, blk, n, w, ld)
    assert np.array_equal(low.residues(), olow.data)
    got = H.matmul_low_high(low, cg, blk, 3)
    want = R.mult_mat_mat_low_high(ev, olow, og, blk, 3, (n, n), (n, n), w, ld, orc)
    assert np.array_equal(got.residues(), want.data)
    multi = H.repack_to_multi_row(got, 5)
    assert np.array_equal(multi.residues(), R.repack_to_multi_row(ev, want, 5, n, w, ld).data)
    thin = L0[blk * ld:(blk + 1) * ld]
    d = H.decrypt2(multi)
    assert np.abs(d[0][5 * ld:6 * ld] - thin @ G0).max() < 2.0 ** -12 and np.abs(d[1][5 * ld:6 * ld] - thin @ G1).max() < 2.0 ** -12
    one = H.repack_to_one_row(got, 1)
    assert np.array_equal(one.residues(), R.repack_to_one_row(ev, want, 1, n, n, w, ld).data)
    # low x low
    cb, rb = 0, 4
    A = cols_of(cb)
    B0, B1 = rows_of(rb), rows_of(rb)
    ca, cw = H.encrypt2(A, A), H.encrypt2(B0, B1)
    got = H.matmul_low_low(ca, cw, cb, rb, 2)
    want = R.mult_mat_mat_low_low(ev, as_oracle(orc, ca), as_oracle(orc, cw), cb, rb, 2, (n, n), (n, n), w, ld, orc)
    assert got.info()["level"] == 2 and np.array_equal(got.residues(), want.data)
    d = H.decrypt2(got)
    assert np.abs(d[0] - A[:, cb * ld:(cb + 1) * ld] @ B0[rb * ld:(rb + 1) * ld]).max() < 2.0 ** -12
    # the element-wise rank-2 path on one pair of tiles
    m = 1
    X = rng.uniform(-1, 1, (n, 2 * n * m))
    A2 = rng.normal(0, 0.3, (2 * n * m, 2))
    B2 = rng.normal(0, 0.3, (2, 2 * n * m))
    wa, wb = np.zeros((n, w)), np.zeros((n, w))
    for j in range(2):
        wa[j] = A2[:, j]
        wb[j] = B2[j]
    enc2 = lambda M: H.encrypt2(M[:, :n], M[:, n:])
    cur, cwa, cwb = [enc2(X)], enc2(wa), enc2(wb)
    ocur, owa, owb = [as_oracle(orc, c) for c in cur], as_oracle(orc, cwa), as_oracle(orc, cwb)
    xa = H.lora_rank2_down(cur, cwa, weight_level=7)
    oxa = R.lora_rank2_down(ev, ocur, owa, n, w, 7, True)
    for j in range(2):
        assert np.array_equal(xa[j].residues(), oxa[j].data)
    out = H.lora_rank2_up(xa, cwb, m, weight_level=4)
    oout = R.lora_rank2_up(ev, oxa, owb, m, n, w, 4, True)
    assert np.array_equal(out[0].residues(), oout[0].data)
    z = H.decrypt_slots(out[0]).real.reshape(n, w)
    assert np.abs(z - X @ A2 @ B2).max() < 2.0 ** -10


@pytest.fixture(scope="module")
def chain24():
    pkg = load_package()
    primes = pkg.primes_below(60, 16, 28)
    qs, ps = primes[:24], primes[24:]
    orc = O.Oracle(16, qs, ps, 3, threads=THREADS)
    ctx = pkg.Context(16, qs, ps, 3)
    orc.gen_secret(3)
    rng = np.random.default_rng(20)
    ct = rand_limbs(rng, qs[:21], (2,), 1 << 16)
    return orc, ctx, ct, dev(ct)


def test_rotation_stages_at_level_20_of_24(chain24):
    """ModUp, key inner product and ModDown one at a time at 21 active limbs + 4 special primes (3 digits of 8)."""
    orc, ctx, ct, dct = chain24
    nq, N = 21, 1 << 16
    E = nq + orc.nP
    orc.gen_rot_key(6, 1)
    evk = orc.keys[("gal", orc.galois(1))]
    ext = orc.modup(ct[1])
    dext = ctx.modup(dct[1].contiguous(), nq)
    assert np.array_equal(host(dext), ext)
    acc = np.empty((2, E, N), dtype=np.uint64)
    orc.L.orc_inner_product(orc.h, _p(ext), _p(evk), nq, _p(acc))
    dacc = ctx.inner_product(dext, dev(evk), nq)
    assert np.array_equal(host(dacc), acc)
    want = np.empty((2, nq, N), dtype=np.uint64)
    for p in range(2):
        orc.L.orc_moddown(orc.h, _p(acc[p]), nq, _p(want[p]))
    assert np.array_equal(host(ctx.moddown(dacc, nq)), want)


@pytest.mark.parametrize("step", [1, 2, 4, 8, 16, 32, 64] + [128 * j for j in (1, 2, 16, 48, 112, 128, 255)])
def test_rotation_step_set_at_level_20_of_24(chain24, step):
    orc, ctx, ct, dct = chain24
    orc.gen_rot_key(6, step)
    g = orc.galois(step)
    want = orc.left_rotate(O.Ct(ct, 1.0), step)
    got = host(ctx.rotate(dct, dev(orc.keys.pop(("gal", g))), g, 21))
    assert np.array_equal(got, want.data)


# ---- basis conversions at the upper end of their lazy accumulators ------------------------------------------------
def _product(ms):
    out = 1
    for m in ms:
        out *= int(m)
    return out


def _worst_case_limb(orc, prime_idx, basis):
    """NTT form of the polynomial whose every coefficient c satisfies [c (S / q)^-1]_q = q - 1 for the basis product
    S: the residue a fast basis conversion multiplies its constants with is then q - 1 at every position."""
    q = orc.mods[prime_idx]
    hat = _product(b for b in basis if b != q) % q
    x = np.full((1, orc.N), (q - 1) * hat % q, dtype=np.uint64)
    # what the conversion will see, checked before the transform hides it
    assert int(x[0, 0]) * pow(hat, -1, q) % q == q - 1
    orc.ntt(x, [prime_idx])
    return x[0]


def _mixed_chain():
    """8 chain primes just below 2^60 and 8 near 2^42 with 8 special primes below 2^60, two digits of 8 limbs: the
    widest conversions the fused transform pass takes, in both directions (eight 60-bit sources into primes below
    2^44, which finish in double precision, and into 60-bit primes)."""
    pkg = load_package()
    big = pkg.primes_below(60, 16, 16)
    qs = big[:8] + pkg.primes_below(42, 16, 8)
    ps = big[8:]
    return O.Oracle(16, qs, ps, 2, threads=THREADS), pkg.Context(16, qs, ps, 2)


def test_conversions_with_every_source_residue_at_q_minus_1(bench):
    """ModUp, ModDown merged with the rescale, plain ModDown and rescale on inputs whose scaled coefficient-form
    residues are q_i - 1 in every source limb and at every position: the lazy dot products of the fused conversion
    pass (16 products of 32 x 28 bits per 64-bit accumulator, finished in double precision for targets below 2^44)
    at the largest sources they can meet, 5 sources on the preset and 8 on a chain of two 8-limb digits."""
    rng = np.random.default_rng(77)
    for orc, ctx, nq in ((bench.orc, bench.ctx, 7), (bench.orc, bench.ctx, 13)) + tuple(
            (o, c, 16) for o, c in (_mixed_chain(),)):
        N, K, alpha = orc.N, orc.nP, orc.alpha
        # ModUp: limb j carries -(Q_d / q_j) for its digit d
        poly = np.empty((nq, N), dtype=np.uint64)
        for j in range(nq):
            d = j // alpha
            basis = orc.q[d * alpha:min(nq, (d + 1) * alpha)]
            poly[j] = _worst_case_limb(orc, j, basis)
        want = orc.modup(poly)
        assert np.array_equal(host(ctx.modup(dev(poly), nq)), want)
        assert np.array_equal(host(ctx.modup_batch(dev(np.stack([poly, poly])), nq)[1]), want)
        # ModDown (with and without the rescale merged in): dropped limbs at the worst case, the others random
        E = nq + K
        ext_mods = [orc.mods[orc.prime_of(j, nq)] for j in range(E)]
        for drop in (True, False):
            y = rand_limbs(rng, ext_mods, (2,), N)
            slots = ([nq - 1] if drop else []) + list(range(nq, E))
            basis = [ext_mods[l] for l in slots]
            for l in slots:
                y[:, l] = _worst_case_limb(orc, orc.prime_of(l, nq), basis)
            want = orc.moddown_drop(y, nq, drop)
            assert np.array_equal(host(ctx.moddown_batch(dev(y), nq, drop)), want), (nq, drop)
            if len(slots) in (4, 5):
                assert np.array_equal(host(ctx.moddown_batch(dev(y), nq, drop, column_slab=True)), want), (nq, drop)
        # rescale: the last limb's coefficients all q_last - 1
        ct = rand_limbs(rng, orc.q[:nq], (2,), N)
        ct[:, nq - 1] = _worst_case_limb(orc, nq - 1, [orc.q[nq - 1]])
        want = orc.rescale(O.Ct(ct, 1.0)).data
        assert np.array_equal(host(ctx.rescale(dev(ct), nq)), want)


def test_moddown_column_slab_form_same_residues(bench, chain24):
    """HEMM_MODDOWN_COLUMN_SLAB: the three-launch ModDown (inverse column pass, conversion and forward column pass in
    one kernel per slab) against the four-launch chain and the oracle; 4 and 5 dropped limbs, a 42-bit and a 60-bit
    last limb (the fifth source goes through LDS in either arithmetic)."""
    import torch
    rng = np.random.default_rng(78)
    for orc, ctx, nq, n_polys in ((bench.orc, bench.ctx, 7, 64), (bench.orc, bench.ctx, 13, 3), (chain24[0], chain24[1], 21, 2)):
        N, E = orc.N, nq + orc.nP
        ext_mods = [orc.mods[orc.prime_of(j, nq)] for j in range(E)]
        y = rand_limbs(rng, ext_mods, (n_polys,), N)
        for drop in (True, False):
            slab = ctx.moddown_batch(dev(y), nq, drop, column_slab=True)
            assert torch.equal(slab, ctx.moddown_batch(dev(y), nq, drop))
            assert np.array_equal(host(slab[-2:]), orc.moddown_drop(y[-2:], nq, drop))
