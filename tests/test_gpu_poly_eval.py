"""GPU parity of the polynomial evaluation routines: residues bit-exact against the oracle restatement on a
small ring, decrypted values against numpy on the full ring."""
import numpy as np
import pytest
from numpy.polynomial import chebyshev as C

from __graft_entry__ import load_package
from oracle import hemmer_ref as R
from oracle import oracle as O
from oracle import poly_ref as P
from tests.test_poly_eval import EXP_15_4, EXP_2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def small():
    load_package()
    from efla_amd import hellm
    qs, ps = O.ckks_chain(10, 9, 3)
    H = hellm.HEMMer(10, qs, ps, dnum=3, min_bootstrap_level=0, seed=7)
    orc = O.Oracle(10, qs, ps, dnum=3)
    orc.gen_secret(7)
    orc.gen_mult_key(7)
    return H, orc, R.OracleEval(orc)


def test_residues_match_oracle(small):
    H, orc, ev = small
    rng = np.random.default_rng(2)
    M = rng.uniform(-1, 1, (16, 16))
    ct = H.encrypt(M)
    i = ct.info()
    oct_ = O.Ct(ct.residues(), orc.delta[i["level"]])
    got = H.exp_iter(ct, 4)
    want = P.exp_iter(ev, oct_, 4)
    assert np.array_equal(got.residues(), want.data)
    assert np.abs(H.decrypt(got) - (1 + M / 16) ** 16).max() < 2 ** -18
    # HELLM::Exp::exp_iter_Parallel on three tensors: one pair and an unpaired last one
    Ms = [rng.uniform(-1, 1, (16, 16)) for _ in range(3)]
    cts = [H.encrypt(m) for m in Ms]
    octs = [O.Ct(c.residues(), orc.delta[c.info()["level"]]) for c in cts]
    H.exp_iter_parallel(cts, 4)
    wants = P.exp_iter_parallel(ev, octs, 4)
    for c, w in zip(cts, wants):
        assert np.array_equal(c.residues(), w.data)
    assert np.abs(H.decrypt(cts[1]) - (1 + Ms[1] / 16) ** 16).max() < 2 ** -18
    assert np.abs(H.decrypt(cts[2]) - (1 + Ms[2] / 16)).max() < 2 ** -20
    poly = [0, 1.5, 0, -0.7, 0, 0.3, 0, -0.11, 0, 0.05, 0, -0.02, 0, 0.008, 0, -0.003]
    for k, l in ((2, 3), (4, 2)):
        got = H.eval_odd_polynomial(ct, poly, k, l)
        want = P.eval_odd_polynomial(ev, oct_, poly, k, l)
        assert np.array_equal(got.residues(), want.data), (k, l)
        assert np.abs(H.decrypt(got) - np.polynomial.polynomial.polyval(M, poly)).max() < 2 ** -16
    # tables in the product basis of HEaaN-math: the reference's own EXP_15_4, random tables, a plain series as one
    # block, a sparse one
    for coef, baby in ((EXP_15_4, 4), (list(rng.normal(size=16)), 4), (list(rng.normal(size=8)), 2),
                       (list(rng.normal(size=11)), 8), (list(rng.normal(size=6)), 0), ([0.5, 0, 0, 0, 2.0], 4)):
        got = H.eval_chebyshev(ct, coef, baby, 0.5)
        want = P.eval_chebyshev(ev, oct_, coef, baby, 0.5)
        assert np.array_equal(got.residues(), want.data), (len(coef), baby)
        assert np.abs(H.decrypt(got) - 0.5 * P.cheb_product_value(coef, baby, M)).max() < 2 ** -14
    # exp on [-2, 2] as the reference computes it (src/Loss.cpp:41-56): linearTransform, then the table
    M2 = rng.uniform(-2, 2, (16, 16))
    c2 = H.encrypt(M2)
    o2 = O.Ct(c2.residues(), orc.delta[c2.info()["level"]])
    u, ou = H.linear_transform(c2, -2.0, 2.0), P.linear_transform(ev, o2, -2.0, 2.0)
    assert np.array_equal(u.residues(), ou.data)
    got, want = H.eval_chebyshev(u, EXP_15_4, 4), P.eval_chebyshev(ev, ou, EXP_15_4, 4)
    assert np.array_equal(got.residues(), want.data)
    assert got.info()["level"] == u.info()["level"] - 4
    assert np.abs(H.decrypt(got) - np.exp(M2)).max() < 2 ** -16
    with pytest.raises(ValueError):
        H.eval_chebyshev(ct, EXP_2, 3)          # baby steps must be a power of two
    low = H.level_down(ct, 2)
    with pytest.raises(load_package().HemmError):
        H.exp_iter(low, 4)                      # not enough levels: the reference would bootstrap here
    with pytest.raises(load_package().HemmError):
        H.exp_iter_parallel([H.level_down(ct, 2), H.level_down(ct, 2)], 4)


def test_full_ring_values():
    load_package()
    from efla_amd import hellm
    H = hellm.HEMMer(preset=True, seed=3)
    rng = np.random.default_rng(3)
    M = rng.uniform(-1, 1, (128, 128))
    ct = H.encrypt(M)
    e = H.eval_chebyshev(ct, EXP_15_4, 4)   # the reference's table, 4 levels (its level_cost)
    assert e.info()["level"] == 12 - 4
    assert np.abs(H.decrypt(e) - np.exp(2 * M)).max() < 2 ** -12
    r = H.exp_iter(ct, 6)
    assert np.abs(H.decrypt(r) - (1 + M / 64) ** 64).max() < 2 ** -12
