"""GPU parity, stage by stage, of the evaluator kernels (pointwise, tensor, automorphism, ModUp,
evk inner product, ModDown, key switch, rotate, relinearize, rescale) against the CPU oracle:
bit-exact residues on identical primes, keys and inputs."""
import numpy as np
import pytest

from __graft_entry__ import load_package
from oracle import oracle as O
from oracle.oracle import _p

pytestmark = pytest.mark.gpu


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


class Setup:
    def __init__(self, log_n, n_q, n_p, dnum, seed):
        pkg = load_package()
        self.pkg = pkg
        qs, ps = O.ckks_chain(log_n, n_q, n_p)
        self.orc = O.Oracle(log_n, qs, ps, dnum)
        self.ctx = pkg.Context(log_n, qs, ps, dnum)
        self.rng = np.random.default_rng(seed)
        self.N = 1 << log_n
        self.orc.gen_secret(3, hw=min(192, self.N // 4))


@pytest.fixture(scope="module", params=[(10, 6, 2, 3), (12, 7, 4, 2), (16, 5, 3, 2)],
                ids=["N1024", "N4096", "N65536"])
def S(request):
    return Setup(*request.param, seed=request.param[0])


def test_pointwise_ops(S):
    orc, ctx, pkg, N = S.orc, S.ctx, S.pkg, S.N
    nq = orc.nQ - 1
    mods = [orc.mods[orc.prime_of(j, nq)] for j in range(nq + orc.nP)]
    a = rand_limbs(S.rng, mods, (2,), N)
    b = rand_limbs(S.rng, mods, (2,), N)
    a[0, 0, :3] = [0, mods[0] - 1, 1]
    b[0, 0, :3] = [0, mods[0] - 1, mods[0] - 1]
    da, db = dev(a), dev(b)
    ref = {}
    for op in (0, 1, 2):
        ref[op] = np.empty_like(a)
        for p in range(2):
            for j in range(nq + orc.nP):
                orc.L.orc_pointwise(orc.h, op, _p(a[p, j]), _p(b[p, j]), _p(ref[op][p, j]), orc.prime_of(j, nq))
        assert np.array_equal(host(ctx.pointwise(op, da, db, nq, with_p=True)), ref[op])
    # negate, broadcast multiply (ct x pt), multiply-accumulate, aliasing output
    neg = host(ctx.pointwise(pkg.NEG, da, None, nq, with_p=True))
    assert np.array_equal((neg.astype(object) + a.astype(object)) % np.array(mods, dtype=object)[None, :, None], 0 * a)
    pt = db[0].contiguous()
    got = host(ctx.pointwise(pkg.MUL, da, pt, nq, with_p=True))
    want = np.empty_like(a)
    for p in range(2):
        for j in range(nq + orc.nP):
            orc.L.orc_pointwise(orc.h, 2, _p(a[p, j]), _p(b[0, j]), _p(want[p, j]), orc.prime_of(j, nq))
    assert np.array_equal(got, want)
    acc = da.clone()
    ctx.pointwise(pkg.MAC, da, db, nq, with_p=True, out=acc)
    want = (ref[2].astype(object) + a.astype(object)) % np.array(mods, dtype=object)[None, :, None]
    assert np.array_equal(host(acc).astype(object), want)
    # reading a 2-poly operand at a lower level through its stride
    lo = ctx.pointwise(pkg.ADD, da, db, 2, with_p=False)
    assert np.array_equal(host(lo), ref[0][:, :2])


def test_scalar_imag_tensor_automorphism(S):
    orc, ctx, N = S.orc, S.ctx, S.N
    nq = orc.nQ
    mods = orc.q[:nq]
    c1 = rand_limbs(S.rng, mods, (2,), N)
    c2 = rand_limbs(S.rng, mods, (2,), N)
    d1, d2 = dev(c1), dev(c2)
    want = np.empty((3, nq, N), dtype=np.uint64)
    orc.L.orc_tensor(orc.h, _p(c1), _p(c2), nq, _p(want))
    t = ctx.tensor(d1, d2, nq)
    assert np.array_equal(host(t), want)
    ctx.tensor(d2, d1, nq, out=t, accumulate=True)
    dbl = (want.astype(object) * 2) % np.array(mods, dtype=object)[None, :, None]
    assert np.array_equal(host(t).astype(object), dbl)
    # scalar (negative integer and a 60-bit constant) and imaginary unit
    for val in (-2, 123456789012345678):
        sc = [val % q for q in mods]
        got = host(ctx.mul_scalar(d1, sc, nq))
        assert np.array_equal(got, orc.mult_scalar_residues(O.Ct(c1, 1.0), val))
    assert np.array_equal(host(ctx.mul_imag_unit(d1, nq)), orc.mult_imag_unit(O.Ct(c1, 1.0)).data)
    for g in (5, pow(5, 77, 2 * N), 2 * N - 1):
        got = host(ctx.automorphism(d1, g, nq))
        want = np.empty_like(c1)
        for p in range(2):
            for j in range(nq):
                orc.L.orc_automorphism_ntt(orc.h, _p(c1[p, j]), _p(want[p, j]), g)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("drop", [0, 1, 2])
def test_keyswitch_stages(S, drop):
    """ModUp, inner product and ModDown one at a time, then the fused chain, at several levels
    (drop = limbs removed from the top, so partial last digits are covered)."""
    orc, ctx, N = S.orc, S.ctx, S.N
    nq = orc.nQ - drop
    E = nq + orc.nP
    if "mult" not in orc.keys:
        orc.gen_mult_key(6)
    evk = orc.keys["mult"]
    devk = dev(evk)
    x = rand_limbs(S.rng, orc.q[:nq], (), N)
    dx = dev(x)
    beta = (nq + orc.alpha - 1) // orc.alpha
    ext = np.empty((beta, E, N), dtype=np.uint64)
    orc.L.orc_modup(orc.h, _p(x), nq, _p(ext))
    dext = ctx.modup(dx, nq)
    assert np.array_equal(host(dext), ext)
    acc = np.empty((2, E, N), dtype=np.uint64)
    orc.L.orc_inner_product(orc.h, _p(ext), _p(evk), nq, _p(acc))
    dacc = ctx.inner_product(dext, devk, nq)
    assert np.array_equal(host(dacc), acc)
    want = np.empty((2, nq, N), dtype=np.uint64)
    for p in range(2):
        orc.L.orc_moddown(orc.h, _p(acc[p]), nq, _p(want[p]))
    assert np.array_equal(host(ctx.moddown(dacc, nq)), want)
    assert np.array_equal(host(ctx.keyswitch(dx, devk, nq)), want)
    ob, oa = orc.keyswitch(x, evk)
    assert np.array_equal(want[0], ob) and np.array_equal(want[1], oa)


@pytest.mark.parametrize("log_n", [10, 16])
def test_keyswitch_and_rescale_with_primes_above_2_60(log_n):
    """Primes of 2^60 and more leave the lazy dot products of the conversion kernels (8 terms of 60 x 60 bits) and the
    conversions inside the transforms: the generic conversion kernel and the separate launches must give the
    oracle's residues too."""
    pkg = load_package()
    big = O.primes_below(61, log_n, 6)
    assert all(q >> 60 for q in big)
    qs, ps = big[:4], big[4:]
    orc = O.Oracle(log_n, qs, ps, 2)
    ctx = pkg.Context(log_n, qs, ps, 2)
    N = 1 << log_n
    rng = np.random.default_rng(61 + log_n)
    orc.gen_secret(3, hw=min(192, N // 4))
    orc.gen_mult_key(6)
    evk = orc.keys["mult"]
    for nq in (4, 3):
        E = nq + orc.nP
        x = rand_limbs(rng, orc.q[:nq], (), N)
        beta = (nq + orc.alpha - 1) // orc.alpha
        ext = np.empty((beta, E, N), dtype=np.uint64)
        orc.L.orc_modup(orc.h, _p(x), nq, _p(ext))
        assert np.array_equal(host(ctx.modup(dev(x), nq)), ext)
        ob, oa = orc.keyswitch(x, evk)
        got = host(ctx.keyswitch(dev(x), dev(evk), nq))
        assert np.array_equal(got[0], ob) and np.array_equal(got[1], oa)
        ct = rand_limbs(rng, orc.q[:nq], (2,), N)
        want = orc.rescale(O.Ct(ct, 1.0)).data
        assert np.array_equal(host(ctx.rescale(dev(ct), nq)), want)


def test_rotate_relinearize_rescale(S):
    orc, ctx, N = S.orc, S.ctx, S.N
    nq = orc.nQ - 1
    if "mult" not in orc.keys:
        orc.gen_mult_key(6)
    rng = S.rng
    z = rng.uniform(-1, 1, orc.slots) + 1j * rng.uniform(-1, 1, orc.slots)
    ct = orc.encrypt(orc.encode(z, nq - 1), 4)
    dct = dev(ct.data)
    for r in (1, 7):
        orc.gen_rot_key(6, r)
        g = orc.galois(r)
        want = orc.left_rotate(ct, r)
        got = host(ctx.rotate(dct, dev(orc.keys[("gal", g)]), g, nq))
        assert np.array_equal(got, want.data)
        assert np.abs(orc.decrypt(O.Ct(got, ct.scale)) - np.roll(z, -r)).max() < 1e-6
    orc.gen_conj_key(6)
    g = 2 * N - 1
    assert np.array_equal(host(ctx.rotate(dct, dev(orc.keys[("gal", g)]), g, nq)), orc.conjugate(ct).data)
    # the result may replace the operand: every read of it is queued before the launch that writes the result
    # (at N = 2^16 no launch copies the rotated polynomials first: the ModUp and the key product read them through
    # the automorphism)
    same = dct.clone()
    ctx.rotate(same, dev(orc.keys[("gal", g)]), g, nq, out=same)
    assert np.array_equal(host(same), orc.conjugate(ct).data)
    t3 = orc.tensor(ct, ct)
    d3 = ctx.tensor(dct, dct, nq)
    assert np.array_equal(host(d3), t3.data)
    rl = orc.relinearize(t3)
    drl = ctx.relinearize(d3, dev(orc.keys["mult"]), nq)
    assert np.array_equal(host(drl), rl.data)
    rs = orc.rescale(rl)
    drs = ctx.rescale(drl, nq)
    assert np.array_equal(host(drs), rs.data)
    assert np.abs(orc.decrypt(O.Ct(host(drs), rs.scale)) - z * z).max() < 1e-6
    # 3-polynomial rescale (used on un-relinearised sums)
    assert np.array_equal(host(ctx.rescale(d3, nq)), orc.rescale(t3).data)


def test_batched_hoisted_forms(S):
    """ModUp of several polynomials, hoisted masked rotation terms, merged ModDown + rescale, masked
    sums and batched tensor accumulation against the oracle's one-at-a-time forms."""
    import torch
    orc, ctx, N = S.orc, S.ctx, S.N
    rng = S.rng
    nq = orc.nQ - 1
    orc.key_seed = 6
    E = nq + orc.nP
    mods = orc.q[:nq]
    cts = [rand_limbs(rng, mods, (2,), N) for _ in range(3)]
    dcts = [dev(c) for c in cts]
    # batched ModUp of the three a-polynomials == three single ModUps
    a_stack = torch.stack([d[1] for d in dcts]).contiguous()
    dext = ctx.modup_batch(a_stack, nq)
    exts = [orc.modup(c[1]) for c in cts]
    for k in range(3):
        assert np.array_equal(host(dext[k]), exts[k])
    # hoisted terms: group 0 = two masked rotations of ct0, group 1 = one unmasked rotation of ct1,
    # group 2 = conjugation of ct2
    z1 = rng.uniform(-1, 1, orc.slots)
    z2 = rng.uniform(-1, 1, orc.slots)
    m1, m2 = orc.encode_ext(z1, nq - 1), orc.encode_ext(z2, nq - 1)
    g1, g2, g3, gc = orc.galois(1), orc.galois(orc.slots - 5), orc.galois(16), 2 * N - 1
    dk = {g: dev(orc.galois_key(g)) for g in (g1, g2, g3, gc)}
    dm1, dm2 = dev(m1.data), dev(m2.data)
    groups = [[(dext[0], dcts[0][0], dk[g1], dm1, g1), (dext[0], dcts[0][0], dk[g2], dm2, g2)],
              [(dext[1], dcts[1][0], dk[g3], None, g3)],
              [(dext[2], dcts[2][0], dk[gc], None, gc)]]
    y = ctx.hoisted_terms(groups, nq)
    want = [orc.hoisted_sum([(exts[0], cts[0][0], ("g", g1), m1), (exts[0], cts[0][0], ("g", g2), m2)], nq),
            orc.hoisted_sum([(exts[1], cts[1][0], ("g", g3), None)], nq),
            orc.hoisted_sum([(exts[2], cts[2][0], ("g", gc), None)], nq)]
    for k in range(3):
        assert np.array_equal(host(y[k]), want[k])
    # two masked sources under one key (the kernel reads that key once for both), followed by a third
    # term of another key in the same group
    shared = [[(dext[0], dcts[0][0], dk[g1], dm1, g1), (dext[1], dcts[1][0], dk[g1], dm2, g1),
               (dext[2], dcts[2][0], dk[g3], dm1, g3)]]
    want_shared = orc.hoisted_sum([(exts[0], cts[0][0], ("g", g1), m1), (exts[1], cts[1][0], ("g", g1), m2),
                                   (exts[2], cts[2][0], ("g", g3), m1)], nq)
    assert np.array_equal(host(ctx.hoisted_terms(shared, nq)[0]), want_shared)
    # the same with P * b supplied by the caller
    Pq = [int(np.prod([int(p) for p in orc.p], dtype=object) % q) for q in mods]
    pbs = [dev(np.stack([(c[0][j].astype(object) * Pq[j] % mods[j]).astype(np.uint64) for j in range(nq)]))
           for c in cts]
    shared_pb = [[(dext[0], pbs[0], dk[g1], dm1, g1), (dext[1], pbs[1], dk[g1], dm2, g1),
                  (dext[2], pbs[2], dk[g3], dm1, g3)]]
    assert np.array_equal(host(ctx.hoisted_terms(shared_pb, nq, b_premultiplied=True)[0]), want_shared)
    # compact keys (6 bytes per residue of a prime below 2^44): the same sums, kernel-argument and staged term lists
    ck = {g: ctx.compact_key(k) for g, k in dk.items()}
    assert all(c.numel() < k.numel() for c, k in zip(ck.values(), dk.values()))
    swap = lambda gs: [[(t[0], t[1], ck[t[4]], t[3], t[4]) + tuple(t[5:]) for t in g] for g in gs]
    assert torch.equal(ctx.hoisted_terms(swap(groups), nq, compact_keys=True), y)
    assert np.array_equal(host(ctx.hoisted_terms(swap(shared), nq, compact_keys=True)[0]), want_shared)
    many = (groups + shared) * 12    # more than 32 terms: the staged list
    assert torch.equal(ctx.hoisted_terms(swap(many), nq, compact_keys=True), ctx.hoisted_terms(many, nq))
    # one layout per call: a mix is refused before anything is launched
    n_terms = sum(len(g) for g in groups)
    with pytest.raises(ValueError, match="same key layout"):
        ctx.hoisted_terms(swap(groups), nq, compact_keys=[True] + [False] * (n_terms - 1))
    # plain ModDown and ModDown merged with the rescale, batched over all outputs
    for drop in (False, True):
        got = host(ctx.moddown_batch(y.clone(), nq, drop))
        for k in range(3):
            assert np.array_equal(got[k], orc.moddown_drop(want[k], nq, drop))
    # both calls in one
    all_groups = (groups + shared) * 2
    all_want = (want + [want_shared]) * 2
    for drop in (False, True):
        got = host(ctx.hoisted_moddown(all_groups, nq, drop))
        for k in range(8):
            assert np.array_equal(got[k], orc.moddown_drop(all_want[k], nq, drop)), (k, drop)
    got = host(ctx.hoisted_moddown(shared_pb * 8, nq, True, b_premultiplied=True))
    assert np.array_equal(got[0], orc.moddown_drop(want_shared, nq, True))
    assert np.array_equal(got[7], got[0])
    got = host(ctx.hoisted_moddown(shared_pb, nq, True, b_premultiplied=True))
    assert np.array_equal(got[0], orc.moddown_drop(want_shared, nq, True))
    # masked sums: out0 = m*ct0 + ct1, out1 = m'*ct2
    p1, p2 = orc.encode(z1, nq - 1), orc.encode(z2, nq - 1)
    dp1, dp2 = dev(p1.data), dev(p2.data)
    ms = host(ctx.masked_sum_batch([[(dcts[0], dp1), (dcts[1], None)], [(dcts[2], dp2)]], nq, 2))
    w0 = orc.add(orc.mult_plain_no_rescale(O.Ct(cts[0], 1.0), p1), O.Ct(cts[1], 1.0)).data
    w1 = orc.mult_plain_no_rescale(O.Ct(cts[2], 1.0), p2).data
    assert np.array_equal(ms[0], w0) and np.array_equal(ms[1], w1)
    # batched tensor accumulation
    t1 = torch.stack(dcts).contiguous()
    t2 = torch.stack(dcts[::-1]).contiguous()
    acc = ctx.tensor_batch(t1, t2, nq)
    ctx.tensor_batch(t1[:1].contiguous(), t1[:1].contiguous(), nq, acc=acc)
    want3 = None
    for a, b in list(zip(cts, cts[::-1])) + [(cts[0], cts[0])]:
        t = orc.tensor(O.Ct(a, 1.0), O.Ct(b, 1.0))
        want3 = t if want3 is None else orc.add(want3, t)
    assert np.array_equal(host(acc), want3.data)
    # several sums in one launch, accumulators polynomial-major: group 0 stores 3 pairs into accumulator 1, group 1
    # adds 2 pairs to accumulator 0 (which holds the sum above), group 2 stores one pair into accumulator 2
    acc3 = torch.zeros((3, 3, nq, S.N), dtype=torch.int64, device="cuda")
    acc3[:, 0] = acc
    ctx.tensor_batch_groups([(t1, t2, 1, False), (t1[1:].contiguous(), t2[:2].contiguous(), 0, True),
                             (t2[:1].contiguous(), t2[:1].contiguous(), 2, False)], nq, acc3)
    single = [ctx.tensor_batch(t1, t2, nq),
              ctx.tensor_batch(t1[1:].contiguous(), t2[:2].contiguous(), nq, acc=acc.clone()),
              ctx.tensor_batch(t2[:1].contiguous(), t2[:1].contiguous(), nq)]
    for idx, want in zip((1, 0, 2), single):
        assert torch.equal(acc3[:, idx], want)
    with pytest.raises(ValueError, match="overlap"):
        ctx.tensor_batch_groups([(t1, t2, 1, False), (t1, t2, 1, True)], nq, acc3)


def test_hoisted_terms_extreme_residues(S):
    """Every operand of a hoisted sum at q - 1 (sources, b, key, masks): the largest sums of products the
    reductions of the integer and the double-precision paths ever see, for merged two-source terms (full masks and
    run tables), single terms and an unmasked term."""
    orc, ctx, N = S.orc, S.ctx, S.N
    nq = orc.nQ - 1
    beta = (nq + orc.alpha - 1) // orc.alpha
    ext_primes = [orc.mods[i] for i in orc.ext_primes(nq - 1)]
    top = lambda primes, prefix: np.stack([np.full(tuple(prefix) + (N,), q - 1, dtype=np.uint64) for q in primes],
                                          axis=len(prefix))
    ext = np.ascontiguousarray(top(ext_primes, (beta,)))                   # [beta][E][N]
    b = np.ascontiguousarray(top(orc.q[:nq], ()))                          # [nq][N]
    evk = np.ascontiguousarray(top(orc.mods, (orc.dnum, 2)))               # [dnum][2][nQ+nP][N]
    mask = O.Pt(np.ascontiguousarray(top(ext_primes, ())), 1.0)            # [E][N]
    g1, g2 = orc.galois(5), orc.galois(orc.slots - 3)
    dext, db, dk, dm = dev(ext), dev(b), dev(evk), dev(mask.data)
    groups = [[(dext, db, dk, dm, g1), (dext, db, dk, dm, g1)],            # merged: two sources under one key
              [(dext, db, dk, dm, g2), (dext, db, dk, None, g1)]]          # single terms, masked and unmasked
    shift = orc.log_n - 8
    tm = ctx.compact_mask(dm, shift)                                       # the same masks as run tables
    assert tm is not None
    groups.append([(dext, db, dk, tm, g1, shift), (dext, db, dk, tm, g1, shift)])
    y = host(ctx.hoisted_terms(groups, nq))
    L, h = orc.L, orc.h
    for k, terms in enumerate([[(mask, g1), (mask, g1)], [(mask, g2), (None, g1)], [(mask, g1), (mask, g1)]]):
        want = np.zeros((2, nq + orc.nP, N), dtype=np.uint64)
        for i, (mk, g) in enumerate(terms):
            L.orc_hoisted_term(h, O._p(ext), O._p(b), O._p(evk), O._p(mk.data) if mk is not None else None, g, nq,
                               O._p(want), int(i > 0))
        assert np.array_equal(y[k], want), k


def test_hoisted_terms_with_run_table_masks(S):
    """A slot pattern of period 128 is, in NTT form, constant over aligned runs of N/256 residues: the hoisted sums
    read such a mask from its run table and must give the residues of the full mask; a mask without that
    structure is reported as such."""
    orc, ctx, N = S.orc, S.ctx, S.N
    rng = np.random.default_rng(77)
    nq = orc.nQ - 1
    orc.key_seed = 6
    mods = orc.q[:nq]
    shift = orc.log_n - 8
    cts = [rand_limbs(rng, mods, (2,), N) for _ in range(2)]
    dcts = [dev(c) for c in cts]
    import torch
    dext = ctx.modup_batch(torch.stack([d[1] for d in dcts]).contiguous(), nq)
    exts = [orc.modup(c[1]) for c in cts]
    col = np.arange(orc.slots) % 128
    m_main = orc.encode_ext((col < 91).astype(float), nq - 1)
    m_wrap = orc.encode_ext((col >= 91).astype(float), nq - 1)
    m_rand = orc.encode_ext(rng.uniform(-1, 1, orc.slots), nq - 1)
    dmain, dwrap, drand = dev(m_main.data), dev(m_wrap.data), dev(m_rand.data)
    tmain, twrap = ctx.compact_mask(dmain, shift), ctx.compact_mask(dwrap, shift)
    assert tmain is not None and twrap is not None
    assert ctx.compact_mask(drand, shift) is None
    tab = host(tmain)
    assert np.array_equal(tab[:, :, 0], m_main.data[:, ::1 << shift])
    primes = [orc.mods[i] for i in orc.ext_primes(nq - 1)]
    for j in (0, nq - 1, len(primes) - 1):     # Shoup companions floor(v 2^64 / q), checked with Python integers
        for r in (0, 1, tab.shape[1] - 1):
            assert int(tab[j, r, 1]) == (int(tab[j, r, 0]) << 64) // int(primes[j])
    g1, g2 = orc.galois(37), orc.galois(orc.slots - 91)
    dk = {g: dev(orc.galois_key(g)) for g in (g1, g2)}
    # two sources under one key (merged), a single masked term, and a full mask beside a run table in one group
    groups = [[(dext[0], dcts[0][0], dk[g1], tmain, g1, shift), (dext[1], dcts[1][0], dk[g1], twrap, g1, shift)],
              [(dext[0], dcts[0][0], dk[g2], twrap, g2, shift)],
              [(dext[0], dcts[0][0], dk[g1], tmain, g1, shift), (dext[1], dcts[1][0], dk[g1], drand, g1)]]
    want = [orc.hoisted_sum([(exts[0], cts[0][0], ("g", g1), m_main), (exts[1], cts[1][0], ("g", g1), m_wrap)], nq),
            orc.hoisted_sum([(exts[0], cts[0][0], ("g", g2), m_wrap)], nq),
            orc.hoisted_sum([(exts[0], cts[0][0], ("g", g1), m_main), (exts[1], cts[1][0], ("g", g1), m_rand)], nq)]
    y = host(ctx.hoisted_terms(groups, nq))
    for k in range(3):
        assert np.array_equal(y[k], want[k]), k


def test_hoisted_terms_with_rotated_plaintext_factor(S):
    """A term may carry a plaintext over the extended basis, read through its own automorphism, as a further factor
    (the rotated weight of a plaintext-ciphertext product summed before the ModDown): with a mask, with two masked
    sources under one key, and alone."""
    import torch
    orc, ctx, N = S.orc, S.ctx, S.N
    rng = np.random.default_rng(78)
    nq = orc.nQ - 1
    orc.key_seed = 6
    mods = orc.q[:nq]
    shift = orc.log_n - 8
    cts = [rand_limbs(rng, mods, (2,), N) for _ in range(2)]
    dcts = [dev(c) for c in cts]
    dext = ctx.modup_batch(torch.stack([d[1] for d in dcts]).contiguous(), nq)
    exts = [orc.modup(c[1]) for c in cts]
    col = np.arange(orc.slots) % 128
    m_main = orc.encode_ext((col < 91).astype(float), nq - 1)
    m_wrap = orc.encode_ext((col >= 91).astype(float), nq - 1)
    weight = orc.encode_ext(rng.uniform(-1, 1, orc.slots), nq - 1)
    dmain, dwrap, dweight = dev(m_main.data), dev(m_wrap.data), dev(weight.data)
    tmain, twrap = ctx.compact_mask(dmain, shift), ctx.compact_mask(dwrap, shift)
    g1, g2 = orc.galois(37), orc.galois(orc.slots - 91)
    gp = orc.galois(5 * 128 % orc.slots)
    dk = {g: dev(orc.galois_key(g)) for g in (g1, g2)}
    groups = [[(dext[0], dcts[0][0], dk[g1], tmain, g1, shift, dweight, gp),
               (dext[1], dcts[1][0], dk[g1], twrap, g1, shift, dweight, gp)],
              [(dext[0], dcts[0][0], dk[g2], dwrap, g2, 0, dweight, gp), (dext[1], dcts[1][0], dk[g1], None, g1, 0, dweight, 1)]]
    e_main, e_wrap = orc.ext_plain_product(m_main, weight, gp), orc.ext_plain_product(m_wrap, weight, gp)
    want = [orc.hoisted_sum([(exts[0], cts[0][0], ("g", g1), e_main), (exts[1], cts[1][0], ("g", g1), e_wrap)], nq),
            orc.hoisted_sum([(exts[0], cts[0][0], ("g", g2), e_wrap),
                             (exts[1], cts[1][0], ("g", g1), orc.ext_plain_product(None, weight, 1))], nq)]
    y = host(ctx.hoisted_terms(groups, nq))
    for k in range(2):
        assert np.array_equal(y[k], want[k]), k


def test_hoisted_terms_without_a_key(S):
    """A term with no key is mask * pt * P * (b, a) on the chain limbs and nothing on the special limbs (the part of a masked
    sum that is not rotated joins the rotated parts before their common ModDown): alone, behind keyed terms of a
    group (plain and compact keys, argument and staged lists), and through the ModDown merged with the rescale."""
    import torch
    orc, ctx, N = S.orc, S.ctx, S.N
    rng = np.random.default_rng(79)
    nq = orc.nQ - 1
    orc.key_seed = 6
    ct = rand_limbs(rng, orc.q[:nq], (2,), N)
    dct = dev(ct)
    ext = orc.modup(ct[1])
    dext = ctx.modup_batch(dct[1:2].contiguous(), nq)[0]
    masks = [orc.encode_ext(rng.uniform(-1, 1, orc.slots), nq - 1) for _ in range(3)]
    dmasks = [dev(m.data) for m in masks]
    g1, g2 = orc.galois(3), orc.galois(orc.slots - 7)
    keys = {g: orc.galois_key(g) for g in (g1, g2)}
    dk = {g: dev(keys[g]) for g in keys}
    none = ("none",)
    weight = orc.encode_ext(rng.uniform(-1, 1, orc.slots), nq - 1)
    dweight = dev(weight.data)
    want = [orc.hoisted_sum([(ct[1], ct[0], none, masks[0])], nq),
            orc.hoisted_sum([(ext, ct[0], ("g", g1), masks[1]), (ext, ct[0], ("g", g2), masks[2]),
                             (ct[1], ct[0], none, masks[0])], nq),
            orc.hoisted_sum([(ct[1], ct[0], none, None), (ext, ct[0], ("g", g1), None)], nq)]
    assert not want[0][:, nq:].any() and want[0][:, :nq].any()
    chain_mask = dev(np.ascontiguousarray(masks[0].data[:nq]))       # a term without a key reads nq limbs of its mask
    groups = [[(dct[1], dct[0], None, chain_mask, 1)],
              [(dext, dct[0], dk[g1], dmasks[1], g1), (dext, dct[0], dk[g2], dmasks[2], g2), (dct[1], dct[0], None, chain_mask, 1)],
              [(dct[1], dct[0], None, None, 1), (dext, dct[0], dk[g1], None, g1)]]
    y = host(ctx.hoisted_terms(groups, nq))
    for k in range(3):
        assert np.array_equal(y[k], want[k]), k
    # without b (only the second polynomial receives P a); with a plaintext factor; with b premultiplied by the caller
    # (a is always taken as it is)
    pb = dev(orc.mul_p_residues(np.ascontiguousarray(ct[0])))
    got = host(ctx.hoisted_terms([[(dct[1], None, None, None, 1)], [(dct[1], dct[0], None, dmasks[0], 1, 0, dweight, 1)]], nq))
    assert np.array_equal(got[0], orc.hoisted_sum([(ct[1], None, none, None)], nq)) and not got[0][0].any()
    assert np.array_equal(got[1], orc.hoisted_sum([(ct[1], ct[0], none, orc.ext_plain_product(masks[0], weight, 1))], nq))
    got = host(ctx.hoisted_terms([[(dct[1], pb, None, chain_mask, 1)]], nq, b_premultiplied=True))
    assert np.array_equal(got[0], want[0])
    # compact keys; a list too long for the kernel arguments (staged); the merged ModDown + rescale behind the sum
    ck = {g: ctx.compact_key(dk[g]) for g in dk}
    groups_c = [[(dext, dct[0], ck[g1], dmasks[1], g1), (dext, dct[0], ck[g2], dmasks[2], g2), (dct[1], dct[0], None, dmasks[0], 1)]]
    assert np.array_equal(host(ctx.hoisted_terms(groups_c, nq, compact_keys=True))[0], want[1])
    long_group = [(dext, dct[0], dk[g1], dmasks[1], g1), (dext, dct[0], dk[g2], dmasks[2], g2)] * 20 + [(dct[1], dct[0], None, dmasks[0], 1)]
    long_want = orc.hoisted_sum([(ext, ct[0], ("g", g1), masks[1]), (ext, ct[0], ("g", g2), masks[2])] * 20 +
                                [(ct[1], ct[0], none, masks[0])], nq)
    assert np.array_equal(host(ctx.hoisted_terms([long_group], nq))[0], long_want)
    got = host(ctx.hoisted_moddown(groups[1:2], nq, True))[0]
    assert np.array_equal(got, orc.moddown_drop(want[1], nq, True))
    # what a term without a key may not carry
    with pytest.raises(ValueError, match="without a key"):
        ctx.hoisted_terms([[(dct[1], dct[0], None, dmasks[0], g1)]], nq)


def test_rotation_24_limb_chain_of_60_bit_primes():
    """One key-switched rotation at the shape of the reference's rotation benchmark: N = 2^16, a chain of 24
    60-bit primes + 4 special primes, dnum = 3 (digits of 8 limbs), ciphertext at level 20, steps from the
    power-of-two set HEMMer uses.  Residues bit-exact against the oracle, ModUp and ModDown included."""
    pkg = load_package()
    log_n, N = 16, 1 << 16
    primes = pkg.primes_below(60, log_n, 28)
    qs, ps = primes[:24], primes[24:]
    orc = O.Oracle(log_n, qs, ps, 3)
    ctx = pkg.Context(log_n, qs, ps, 3)
    orc.gen_secret(3)
    rng = np.random.default_rng(20)
    nq = 21
    ct = rand_limbs(rng, qs[:nq], (2,), N)
    dct = dev(ct)
    # stages on the a-polynomial
    ext = orc.modup(ct[1])
    assert np.array_equal(host(ctx.modup(dct[1].contiguous(), nq)), ext)
    for r in (1, 64, 128 * 5):
        orc.gen_rot_key(6, r)
        g = orc.galois(r)
        want = orc.left_rotate(O.Ct(ct, 1.0), r)
        got = host(ctx.rotate(dct, dev(orc.keys[("gal", g)]), g, nq))
        assert np.array_equal(got, want.data), r


def test_device_samplers_match_oracle(S):
    """The uniform and error samplers on the device reproduce the oracle's counter-based streams."""
    orc, ctx, N = S.orc, S.ctx, S.N
    tot = orc.nQ + orc.nP
    idx = list(range(tot))
    keys = [orc.stream(9, O.TAG_EVK_A, 77, j) for j in idx]
    got = host(ctx.sample_uniform(keys, idx))
    for j in idx:
        assert np.array_equal(got[j], orc.uniform(keys[j], j)), j
        assert got[j].max() < orc.mods[j]
    ek = orc.stream(9, O.TAG_EVK_E, 77, 1)
    e = orc.error(ek)
    got = host(ctx.sample_error(ek, idx))
    for j in idx:
        assert np.array_equal(got[j], np.mod(e.astype(np.int64), orc.mods[j]).astype(np.uint64)), j


def test_batched_entry_points_refuse_what_the_kernels_cannot_take():
    """Compact keys with more than six digits (there the limbs of primes below 2^44 run through the integer path,
    which reads whole words), more groups than one grouped tensor launch holds, and a flag the library does not know:
    each refused on the host, nothing launched."""
    import torch
    pkg = load_package()
    log_n, N = 10, 1 << 10
    qs, ps = O.ckks_chain(log_n, 8, 1)
    ctx = pkg.Context(log_n, qs, ps, 8)            # digits of one limb: a sum at nq = 8 has 8 digits
    nq, E = 8, 9
    z = lambda *shape: torch.zeros(shape, dtype=torch.int64, device="cuda")
    ext, b, evk = z(8, E, N), z(nq, N), z(8, 2, 9, N)
    groups = [[(ext, b, evk, None, 5)]]
    assert int(ctx.hoisted_terms(groups, nq).abs().sum().item()) == 0          # the plain layout runs
    ck = ctx.compact_key(evk)
    with pytest.raises(ValueError, match="at most 6 digits"):
        ctx.hoisted_terms([[(ext, b, ck, None, 5)]], nq, compact_keys=True)
    with pytest.raises(ValueError, match="unknown flag"):
        ctx.hoisted_terms(groups, nq, compact_keys=[2])
    t = z(1, 2, nq, N)
    acc = z(3, 9, nq, N)
    with pytest.raises(ValueError, match="groups per call"):
        ctx.tensor_batch_groups([(t, t, i, False) for i in range(9)], nq, acc)
    ctx.tensor_batch_groups([(t, t, i, False) for i in range(8)], nq, acc)
    torch.cuda.synchronize()
    assert int(acc.abs().sum().item()) == 0
