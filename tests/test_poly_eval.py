"""Polynomial evaluation on ciphertexts: the restated algorithms on the exact slot simulator (values against
numpy) and over the CPU RNS-CKKS oracle (decrypted values), which pins the sequences the GPU residues are
compared against in test_gpu_poly_eval.py."""
import numpy as np
import pytest
from numpy.polynomial import chebyshev as C

from oracle import hemmer_ref as R
from oracle import oracle as O
from oracle import poly_ref as P

# Chebyshev coefficients of exp on [-2, 2] in the variable x / 2: exp(2t) = I_0(2) + 2 sum_k I_k(2) T_k(t).  The
# reference's EXP_15_4 table (include/HELLM/LossRemezCoeff.hpp:18-35) starts 2.27958530, 3.18083..., 1.37469...:
# the same expansion up to its minimax adjustment.
from scipy.special import iv

EXP_2 = [float(iv(0, 2.0))] + [float(2.0 * iv(k, 2.0)) for k in range(1, 16)]


def test_slot_values():
    ev = R.SlotSim(9, 12)
    rng = np.random.default_rng(0)
    x = rng.uniform(-1, 1, 512)
    ct = ev.encrypt(x)
    r = P.exp_iter(ev, ct, 6)
    assert r.level == 12 - 7
    assert np.abs(ev.decrypt(r).real - (1 + x / 64) ** 64).max() < 1e-12
    poly = [0, 1.5, 0, -0.7, 0, 0.3, 0, -0.11, 0, 0.05, 0, -0.02, 0, 0.008, 0, -0.003]
    for k, l in ((2, 3), (4, 2), (8, 1)):
        r = P.eval_odd_polynomial(ev, ct, poly, k, l)
        assert np.abs(ev.decrypt(r).real - np.polynomial.polynomial.polyval(x, poly)).max() < 1e-13
    for deg in (1, 3, 4, 7, 8, 10, 15, 16, 31):
        coef = rng.normal(size=deg + 1)
        for baby in (2, 4, 8):
            r = P.eval_chebyshev(ev, ct, coef, baby)
            assert np.abs(ev.decrypt(r).real - C.chebval(x, coef)).max() < 1e-11, (deg, baby)
    # sparse expansions: only T_4 / only T_8 above the constant, and an inner zero
    for coef in ([0.5, 0, 0, 0, 2.0], [0.5, 0, 0, 0, 0, 0, 0, 0, 2.0], [1, 2, 0, 0, 0, 0, 3, 0, 0, 0, 0.5]):
        r = P.eval_chebyshev(ev, ct, coef, 4)
        assert np.abs(ev.decrypt(r).real - C.chebval(x, coef)).max() < 1e-12
    # degree 15, 4 baby steps: depth 5 (T_8 at depth 3, two nested giant-step products above the baby sums)
    r = P.eval_chebyshev(ev, ct, rng.normal(size=16), 4)
    assert r.level == 12 - 5


@pytest.fixture(scope="module")
def env():
    qs, ps = O.ckks_chain(10, 9, 3)
    orc = O.Oracle(10, qs, ps, dnum=3)
    orc.gen_secret(7)
    orc.gen_mult_key(7)
    return orc, R.OracleEval(orc)


def test_over_oracle(env):
    orc, ev = env
    rng = np.random.default_rng(1)
    x = rng.uniform(-1, 1, orc.slots)
    ct = orc.encrypt(orc.encode(x.astype(np.complex128), orc.nQ - 1), 5)
    r = P.exp_iter(ev, ct, 4)
    assert np.abs(orc.decrypt(r).real - (1 + x / 16) ** 16).max() < 2 ** -18
    poly = [0, 1.5, 0, -0.7, 0, 0.3, 0, -0.11]
    r = P.eval_odd_polynomial(ev, ct, poly, 2, 2)
    assert r.data.shape[0] == 2
    assert np.abs(orc.decrypt(r).real - np.polynomial.polynomial.polyval(x, poly)).max() < 2 ** -18
    r = P.eval_chebyshev(ev, ct, EXP_2, 4)
    assert np.abs(orc.decrypt(r).real - C.chebval(x, EXP_2)).max() < 2 ** -16
    assert np.abs(orc.decrypt(r).real - np.exp(2 * x)).max() < 1e-6
