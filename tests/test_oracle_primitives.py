"""Pins the CPU oracle's ring primitives against what the mathematics fixes: Python big
integers, the O(N^2) definition of the negacyclic transform, exact CRT, and published
splitmix64 outputs.  Nothing here retypes the oracle's own formulas."""
import numpy as np
import pytest

from oracle import oracle as O
from oracle.oracle import _p


def bitrev(x, bits):
    return int(format(x, "0%db" % bits)[::-1], 2)


@pytest.fixture(scope="module")
def small():
    qs, ps = O.ckks_chain(6, 5, 2)       # N = 64
    return O.Oracle(6, qs, ps, dnum=2)


@pytest.fixture(scope="module")
def mid():
    qs, ps = O.ckks_chain(10, 6, 2)      # N = 1024
    return O.Oracle(10, qs, ps, dnum=3)


def rand_res(rng, q, n):
    return np.array([int(rng.integers(0, 1 << 62)) % q for _ in range(n)], dtype=np.uint64)


def test_splitmix64_known_answers():
    L = O.lib()
    # first three outputs of the published splitmix64 generator seeded with 0
    g = 0x9E3779B97F4A7C15
    exp = [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    got = [L.orc_sm64((k * g) & (2**64 - 1)) for k in range(3)]
    assert got == exp


def test_prime_chain_properties():
    qs, ps = O.ckks_chain(16, 13, 4)
    assert len(set(qs + ps)) == 17
    for p in qs + ps:
        assert O.is_prime(p) and p % (1 << 17) == 1 and p < (1 << 61)
    assert all(abs(q / 2**42 - 1) < 2**-17 for q in qs[1:])
    assert qs[0] < 2**60 and all(2**59 < p < 2**60 for p in ps)
    # 24 largest 60-bit NTT-friendly primes: strictly descending, no prime skipped
    big = O.primes_below(60, 16, 24)
    assert big == sorted(big, reverse=True)
    skipped = [c for c in range(big[-1], 1 << 60, 1 << 17) if c not in big and O.is_prime(c)]
    assert skipped == []


def test_pointwise_vs_bigint(mid):
    rng = np.random.default_rng(1)
    for pi in (0, 1, mid.nQ):          # 60-bit base, 42-bit scale prime, special prime
        q = mid.mods[pi]
        a = rand_res(rng, q, mid.N)
        b = rand_res(rng, q, mid.N)
        edge = [0, 1, q - 1, q - 2, q // 2, (1 << 32) - 1, (1 << 32) + 1]
        a[: len(edge)] = edge
        b[: len(edge)] = edge[::-1]
        out = np.empty_like(a)
        for op, f in ((0, lambda x, y: (x + y) % q), (1, lambda x, y: (x - y) % q),
                      (2, lambda x, y: x * y % q)):
            mid.L.orc_pointwise(mid.h, op, _p(a), _p(b), _p(out), pi)
            assert [int(v) for v in out] == [f(int(x), int(y)) for x, y in zip(a, b)]


def test_ntt_matches_definition(small):
    """out[k] = sum_j a_j psi^{(2 br(k)+1) j}  (bit-reversed output order)."""
    rng = np.random.default_rng(2)
    N, lg = small.N, small.log_n
    for pi in (0, 2, small.nQ + 1):
        q = small.mods[pi]
        psi = small.L.orc_psi(small.h, pi)
        assert pow(psi, N, q) == q - 1                      # primitive 2N-th root
        a = rand_res(rng, q, N)
        a[:3] = [q - 1, 0, q - 1]
        x = a.copy()
        small.L.orc_ntt(small.h, _p(x), pi, 0)
        for k in range(N):
            e = 2 * bitrev(k, lg) + 1
            want = sum(int(a[j]) * pow(psi, e * j, q) for j in range(N)) % q
            assert int(x[k]) == want
        small.L.orc_ntt(small.h, _p(x), pi, 1)
        assert np.array_equal(x, a)


def test_ntt_full_size_spot_and_monomial():
    qs = O.primes_below(60, 16, 2)
    orc = O.Oracle(16, qs, [], dnum=1)
    rng = np.random.default_rng(3)
    q = qs[1]
    psi = orc.L.orc_psi(orc.h, 1)
    N = orc.N
    # closed form: NTT(X^j)[k] = psi^{(2 br(k)+1) j}
    j = 40961
    a = np.zeros(N, dtype=np.uint64)
    a[j] = 1
    orc.L.orc_ntt(orc.h, _p(a), 1, 0)
    for k in [0, 1, 2, 77, 32768, 65535] + [int(v) for v in rng.integers(0, N, 20)]:
        assert int(a[k]) == pow(psi, (2 * bitrev(k, 16) + 1) * j, q)
    # random input, definition at a few output indices, and bit-exact round trip
    b = rng.integers(0, q, N, dtype=np.uint64)
    x = b.copy()
    orc.L.orc_ntt(orc.h, _p(x), 1, 0)
    bi = [int(v) for v in b]
    for k in [0, 65535] + [int(v) for v in rng.integers(0, N, 4)]:
        e = 2 * bitrev(k, 16) + 1
        w, acc, step = 1, 0, pow(psi, e, q)
        for v in bi:
            acc += v * w
            w = w * step % q
        assert int(x[k]) == acc % q
    orc.L.orc_ntt(orc.h, _p(x), 1, 1)
    assert np.array_equal(x, b)


def test_negacyclic_convolution(mid):
    rng = np.random.default_rng(4)
    N, pi = 256, 1
    qs = O.primes_below(60, 8, 1)
    orc = O.Oracle(8, qs, [], dnum=1)
    q = qs[0]
    a = rand_res(rng, q, N)
    b = rand_res(rng, q, N)
    want = [0] * N
    for i in range(N):
        for j in range(N):
            k = i + j
            if k < N:
                want[k] += int(a[i]) * int(b[j])
            else:
                want[k - N] -= int(a[i]) * int(b[j])
    want = [w % q for w in want]
    x, y, z = a.copy(), b.copy(), np.empty_like(a)
    orc.L.orc_ntt(orc.h, _p(x), 0, 0)
    orc.L.orc_ntt(orc.h, _p(y), 0, 0)
    orc.L.orc_pointwise(orc.h, 2, _p(x), _p(y), _p(z), 0)
    orc.L.orc_ntt(orc.h, _p(z), 0, 1)
    assert [int(v) for v in z] == want


def test_automorphism(small):
    rng = np.random.default_rng(5)
    N, q = small.N, small.mods[1]
    a = rand_res(rng, q, N)
    for g in (5, 25, 2 * N - 1, pow(5, 7, 2 * N)):
        # brute-force substitution X -> X^g in Z_q[X]/(X^N+1)
        want = [0] * N
        for i in range(N):
            e = i * g % (2 * N)
            if e < N:
                want[e] = (want[e] + int(a[i])) % q
            else:
                want[e - N] = (want[e - N] - int(a[i])) % q
        out = np.empty_like(a)
        small.L.orc_automorphism_coeff(small.h, _p(a), _p(out), g, 1)
        assert [int(v) for v in out] == want
        # NTT-domain permutation == INTT -> substitution -> NTT
        x = a.copy()
        small.L.orc_ntt(small.h, _p(x), 1, 0)
        y = np.empty_like(x)
        small.L.orc_automorphism_ntt(small.h, _p(x), _p(y), g)
        small.L.orc_ntt(small.h, _p(y), 1, 1)
        assert [int(v) for v in y] == want


def crt(res, mods):
    M = 1
    for m in mods:
        M *= m
    x = 0
    for r, m in zip(res, mods):
        Mi = M // m
        x += int(r) * Mi * pow(Mi, -1, m)
    return x % M, M


def test_modup_is_fast_basis_conversion(mid):
    """Every extended limb equals x + u*Q_d with 0 <= u < |digit|, u given by the
    float-free formula sum_i [x_i qhat_i^-1]_{q_i} qhat_i."""
    rng = np.random.default_rng(6)
    N, nq = mid.N, 5                      # alpha = 2 -> digits {0,1},{2,3},{4}
    coef = np.stack([rand_res(rng, mid.q[j], N) for j in range(nq)])
    x = coef.copy()
    mid.ntt(x, list(range(nq)))
    beta = (nq + mid.alpha - 1) // mid.alpha
    ext = np.empty((beta, nq + mid.nP, N), dtype=np.uint64)
    mid.L.orc_modup(mid.h, _p(x), nq, _p(ext))
    primes = [mid.prime_of(j, nq) for j in range(nq + mid.nP)]
    back = ext.copy()
    for d in range(beta):
        mid.ntt(back[d], primes, inverse=True)
    for d in range(beta):
        dig = list(range(d * mid.alpha, min(nq, (d + 1) * mid.alpha)))
        mods = [mid.q[j] for j in dig]
        Qd = 1
        for m in mods:
            Qd *= m
        for n in range(0, N, 37):
            s = 0
            for j, m in zip(dig, mods):
                qh = Qd // m
                s += (int(coef[j, n]) * pow(qh, -1, m) % m) * qh
            exact, _ = crt([coef[j, n] for j in dig], mods)
            assert s % Qd == exact and 0 <= (s - exact) // Qd < len(dig)
            for l, pi in enumerate(primes):
                assert int(back[d, l, n]) == s % mid.mods[pi]


def test_moddown_divides_by_P(mid):
    rng = np.random.default_rng(7)
    N, nq = mid.N, 4
    primes = [mid.prime_of(j, nq) for j in range(nq + mid.nP)]
    coef = np.stack([rand_res(rng, mid.mods[pi], N) for pi in primes])
    acc = coef.copy()
    mid.ntt(acc, primes)
    out = np.empty((nq, N), dtype=np.uint64)
    mid.L.orc_moddown(mid.h, _p(acc), nq, _p(out))
    mid.ntt(out, list(range(nq)), inverse=True)
    P = 1
    for p in mid.p:
        P *= p
    for n in range(0, N, 29):
        s = 0
        for k, p in enumerate(mid.p):
            ph = P // p
            s += (int(coef[nq + k, n]) * pow(ph, -1, p) % p) * ph
        for j in range(nq):
            q = mid.q[j]
            want = (int(coef[j, n]) - s) * pow(P, -1, q) % q
            assert int(out[j, n]) == want


def test_rescale_is_exact_division(mid):
    rng = np.random.default_rng(8)
    N, nq = mid.N, 4
    coef = np.stack([rand_res(rng, mid.q[j], N) for j in range(nq)])
    x = coef.copy()
    mid.ntt(x, list(range(nq)))
    out = np.empty((nq - 1, N), dtype=np.uint64)
    mid.L.orc_rescale(mid.h, _p(x), nq, _p(out))
    mid.ntt(out, list(range(nq - 1)), inverse=True)
    mods = mid.q[:nq]
    for n in range(0, N, 31):
        c, _ = crt(coef[:, n], mods)
        want = (c - c % mods[-1]) // mods[-1]              # floor(c / q_last)
        for j in range(nq - 1):
            assert int(out[j, n]) == want % mods[j]


@pytest.mark.parametrize("drop_last", [0, 1])
def test_moddown_drop_vs_crt(mid, drop_last):
    """Division by P, or by P q_last in one conversion, against big integers: with D the product of the dropped
    primes and s the float-free lift of the dropped residues (s = y mod D up to a multiple u D, 0 <= u < number of
    dropped limbs), every kept limb is (y_j - s) / D mod q_j -- the floor of y / D shifted down by u, never rounded."""
    rng = np.random.default_rng(17)
    N, nq = mid.N, 5
    primes = [mid.prime_of(j, nq) for j in range(nq + mid.nP)]
    coef = np.stack([rand_res(rng, mid.mods[pi], N) for pi in primes])
    y = coef.copy()
    mid.ntt(y, primes)
    nq_out = nq - drop_last
    out = np.empty((nq_out, N), dtype=np.uint64)
    mid.L.orc_moddown_drop(mid.h, _p(y), nq, drop_last, _p(out))
    mid.ntt(out, list(range(nq_out)), inverse=True)
    dropped = ([nq - 1] if drop_last else []) + list(range(nq, nq + mid.nP))      # limb slots
    dmods = [mid.mods[primes[l]] for l in dropped]
    D = 1
    for m in dmods:
        D *= m
    kept = [mid.q[j] for j in range(nq_out)]
    for n in range(0, N, 23):
        s = 0
        for l, m in zip(dropped, dmods):
            dh = D // m
            s += (int(coef[l, n]) * pow(dh, -1, m) % m) * dh
        exact, _ = crt([coef[l, n] for l in dropped], dmods)
        u = (s - exact) // D
        assert s % D == exact and 0 <= u < len(dropped)
        full, _ = crt([coef[j, n] for j in range(nq_out)] + [coef[l, n] for l in dropped], kept + dmods)
        assert (full - exact) % D == 0
        for j, q in enumerate(kept):
            assert int(out[j, n]) == (int(coef[j, n]) - s) * pow(D, -1, q) % q
            assert int(out[j, n]) == ((full - exact) // D - u) % q          # floor(y / D) - u


def test_inner_product_vs_bigint(mid):
    rng = np.random.default_rng(18)
    N, nq = mid.N, 5
    E, full = nq + mid.nP, mid.nQ + mid.nP
    beta = (nq + mid.alpha - 1) // mid.alpha
    primes = [mid.prime_of(j, nq) for j in range(E)]
    ext = np.stack([[rand_res(rng, mid.mods[pi], N) for pi in primes] for _ in range(beta)])
    evk = np.stack([[[rand_res(rng, m, N) for m in mid.mods] for _ in range(2)] for _ in range(mid.dnum)])
    ext[0, 0, :4] = np.uint64(mid.mods[0] - 1)          # both factors at q - 1
    evk[0, :, 0, :4] = np.uint64(mid.mods[0] - 1)
    acc = np.empty((2, E, N), dtype=np.uint64)
    mid.L.orc_inner_product(mid.h, _p(ext), _p(evk), nq, _p(acc))
    for pol in range(2):
        for j, pi in enumerate(primes):
            q = mid.mods[pi]
            for n in list(range(4)) + list(range(5, N, 97)):
                want = sum(int(ext[d, j, n]) * int(evk[d, pol, pi, n]) for d in range(beta)) % q
                assert int(acc[pol, j, n]) == want


def test_hoisted_term_vs_bigint(small):
    """y (+)= mask * (<rot_g(ext), evk> + P rot_g(b)): the automorphism is checked through the coefficient domain
    (X -> X^g by brute-force substitution), the products with big integers."""
    o = small
    rng = np.random.default_rng(19)
    N, nq = o.N, 5                    # two digits
    E, full = nq + o.nP, o.nQ + o.nP
    beta = (nq + o.alpha - 1) // o.alpha
    assert beta == 2
    primes = [o.prime_of(j, nq) for j in range(E)]
    g = pow(5, 7, 2 * N)
    P = 1
    for p in o.p:
        P *= p

    def substitute(poly, q):          # X -> X^g on coefficients, sign from X^N = -1
        out = [0] * N
        for i, v in enumerate(poly):
            e = i * g % (2 * N)
            out[e % N] = int(v) % q if e < N else (q - int(v)) % q
        return np.array(out, dtype=np.uint64)

    def rotated_ntt(x, pi):           # NTT form of the substituted polynomial
        c = x.copy()
        o.ntt(c.reshape(1, N), [pi], inverse=True)
        c = substitute(c, o.mods[pi])
        o.ntt(c.reshape(1, N), [pi])
        return c

    ext = np.stack([[rand_res(rng, o.mods[pi], N) for pi in primes] for _ in range(beta)])
    b = np.stack([rand_res(rng, o.q[j], N) for j in range(nq)])
    evk = np.stack([[[rand_res(rng, m, N) for m in o.mods] for _ in range(2)] for _ in range(o.dnum)])
    mask = np.stack([rand_res(rng, o.mods[pi], N) for pi in primes])
    y0 = np.stack([[rand_res(rng, o.mods[pi], N) for pi in primes] for _ in range(2)])
    for accumulate, with_b, with_mask in ((0, True, True), (1, True, False), (1, False, True)):
        y = y0.copy()
        o.L.orc_hoisted_term(o.h, _p(ext), _p(b) if with_b else None, _p(evk), _p(mask) if with_mask else None,
                             g, nq, _p(y), accumulate)
        for j, pi in enumerate(primes):
            q = o.mods[pi]
            rext = [rotated_ntt(ext[d, j], pi) for d in range(beta)]
            rb = rotated_ntt(b[j], pi) if (with_b and j < nq) else None
            for pol in range(2):
                for n in range(N):
                    s = sum(int(rext[d][n]) * int(evk[d, pol, pi, n]) for d in range(beta))
                    if pol == 0 and rb is not None:
                        s += P * int(rb[n])
                    if with_mask:
                        s *= int(mask[j, n])
                    if accumulate:
                        s += int(y0[pol, j, n])
                    assert int(y[pol, j, n]) == s % q, (accumulate, j, pol, n)


def test_tensor_and_imag_unit(mid):
    rng = np.random.default_rng(9)
    N, nq = mid.N, 3
    c1 = np.stack([[rand_res(rng, mid.q[j], N) for j in range(nq)] for _ in range(2)])
    c2 = np.stack([[rand_res(rng, mid.q[j], N) for j in range(nq)] for _ in range(2)])
    out = np.empty((3, nq, N), dtype=np.uint64)
    mid.L.orc_tensor(mid.h, _p(c1), _p(c2), nq, _p(out))
    for j in range(nq):
        q = mid.q[j]
        for n in range(0, N, 101):
            b1, a1, b2, a2 = (int(c1[0, j, n]), int(c1[1, j, n]), int(c2[0, j, n]), int(c2[1, j, n]))
            assert [int(out[k, j, n]) for k in range(3)] == [b1 * b2 % q, (a1 * b2 + a2 * b1) % q,
                                                              a1 * a2 % q]
    # multImagUnit == multiplication by X^{N/2} in coefficient form
    a = rand_res(rng, mid.q[1], N)
    x = a.copy()
    mid.L.orc_ntt(mid.h, _p(x), 1, 0)
    y = np.empty_like(x)
    mid.L.orc_mul_imag_unit(mid.h, _p(x), _p(y), 1)
    mid.L.orc_ntt(mid.h, _p(y), 1, 1)
    want = np.concatenate([(mid.q[1] - a[N // 2:]) % np.uint64(mid.q[1]), a[: N // 2]])
    assert np.array_equal(y, want)


def test_samplers(mid):
    k = mid.stream(11, O.TAG_SK)
    s = mid.ternary(k, 192)
    assert np.count_nonzero(s) == 192 and set(np.unique(s)) <= {-1, 0, 1}
    assert abs(int(s.sum())) < 60
    assert np.array_equal(s, mid.ternary(k, 192))
    assert not np.array_equal(s, mid.ternary(mid.stream(12, O.TAG_SK), 192))
    e = mid.error(mid.stream(11, O.TAG_ENC_E))
    assert abs(e.mean()) < 0.5 and 8 < e.var() < 13 and np.abs(e).max() <= 21
    u = mid.uniform(mid.stream(11, O.TAG_ENC_A, 3), 1)
    assert u.max() < mid.q[1] and u.min() >= 0 and abs(u.mean() / mid.q[1] - 0.5) < 0.05
