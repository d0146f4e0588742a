"""Polynomial evaluation on ciphertexts: the restated algorithms on the exact slot simulator (values against
numpy) and over the CPU RNS-CKKS oracle (decrypted values), which pins the sequences the GPU residues are
compared against in test_gpu_poly_eval.py."""
import numpy as np
import pytest
from numpy.polynomial import chebyshev as C

from oracle import hemmer_ref as R
from oracle import oracle as O
from oracle import poly_ref as P

from scipy.special import iv

# Plain Chebyshev series of exp on [-2, 2] in the variable t = x / 2: exp(2t) = I_0(2) + 2 sum_k I_k(2) T_k(t).
EXP_2 = [float(iv(0, 2.0))] + [float(2.0 * iv(k, 2.0)) for k in range(1, 16)]

# The reference's own table for the same function (include/HELLM/LossRemezCoeff.hpp:18-35, EXP_15_4: 16 numbers,
# 4 baby steps, input range [-2, 2] through linearTransform, src/Loss.cpp:41-56), typed in as data.  It is stored in
# the baby-step / giant-step product basis of HEaaN-math (PolynomialEvaluator.hpp:49-58), not as a plain series:
# entry 5 is 0.0393..., twice the plain coefficient 2 I_5(2) = 0.01965....
EXP_15_4 = [2.2795853023344534449279308319091796875, 3.18083051935939664645047741942107677459716796875,
            1.374697152038709457855247819679789245128631591796875, 0.405828613932481874204682981144287623465061187744140625,
            0.1014571354501081767995884774791193194687366485595703125,
            0.0393026084044210063939139843114389805123209953308105469,
            0.0063994866685381495557960462861046835314482450485229492,
            0.0008863798243944620569578773938701488077640533447265625,
            0.000055398739024659082730295267538167536258697509765625,
            0.0000121767403431454263913616756220825720902212196961045,
            0.0000012067365124407632469223693519322360145906714024022,
            0.0000001081982869352056945326870374124439422303112223744,
            0.0000000090165239110433833408242421114664466585963964462,
            0.0000000013796130076531036481174430363694227708037942648,
            0.0000000000980785986734873695678561811295281813727342524,
            0.0000000000065353935470404213923091649857122220623750763]


def test_reference_table_is_in_the_product_basis():
    """The reference's EXP_15_4 numbers, read in the product basis, give exp on [-2, 2] to 1e-10 -- and 4e-2 when
    misread as a plain Chebyshev series; the plain series of exp converted to the product basis lands on the table
    (up to the table's minimax adjustment)."""
    t = np.linspace(-1, 1, 4001)
    assert np.abs(P.cheb_product_value(EXP_15_4, 4, t) - np.exp(2 * t)).max() < 1e-10
    assert np.abs(C.chebval(t, EXP_15_4) - np.exp(2 * t)).max() > 1e-2
    conv = P.cheb_plain_to_product(EXP_2, 4)
    assert np.abs(np.array(conv) - np.array(EXP_15_4)).max() < 1e-9
    assert abs(conv[5] - 2 * EXP_2[5]) < 1e-6 and abs(conv[3] - (EXP_2[3] - EXP_2[5])) < 1e-6   # up to c_11, c_13
    # conversion and definition agree for random series and every power-of-two block size
    rng = np.random.default_rng(5)
    for deg in (3, 7, 10, 15, 31, 63):
        c = rng.normal(size=deg + 1)
        for bs in (2, 4, 8, 16):
            d = P.cheb_plain_to_product(c, bs)
            assert np.abs(P.cheb_product_value(d, bs, t) - C.chebval(t, c)).max() < 1e-9, (deg, bs)


def test_slot_values():
    ev = R.SlotSim(9, 12)
    rng = np.random.default_rng(0)
    x = rng.uniform(-1, 1, 512)
    ct = ev.encrypt(x)
    r = P.exp_iter(ev, ct, 6)
    assert r.level == 12 - 7
    assert np.abs(ev.decrypt(r).real - (1 + x / 64) ** 64).max() < 1e-12
    # the list form squares pair by pair; a trailing tensor without a partner is only scaled and shifted
    ys = [rng.uniform(-1, 1, 512) for _ in range(5)]
    rs = P.exp_iter_parallel(ev, [ev.encrypt(y) for y in ys], 5)
    for y, r in zip(ys[:4], rs[:4]):
        assert r.level == 12 - 6
        assert np.abs(ev.decrypt(r).real - (1 + y / 32) ** 32).max() < 1e-12
    assert rs[4].level == 12 - 1 and np.abs(ev.decrypt(rs[4]).real - (1 + ys[4] / 32)).max() < 1e-12
    poly = [0, 1.5, 0, -0.7, 0, 0.3, 0, -0.11, 0, 0.05, 0, -0.02, 0, 0.008, 0, -0.003]
    for k, l in ((2, 3), (4, 2), (8, 1)):
        r = P.eval_odd_polynomial(ev, ct, poly, k, l)
        assert np.abs(ev.decrypt(r).real - np.polynomial.polynomial.polyval(x, poly)).max() < 1e-13
    t = x
    for deg in (1, 3, 4, 7, 8, 10, 15, 16, 31):
        coef = rng.normal(size=deg + 1)
        for baby in (2, 4, 8):
            r = P.eval_chebyshev(ev, ct, P.cheb_plain_to_product(coef, baby), baby)
            assert np.abs(ev.decrypt(r).real - C.chebval(x, coef)).max() < 1e-11, (deg, baby)
        # one block (baby = 0): the coefficients are a plain series
        r = P.eval_chebyshev(ev, ct, coef, 0)
        assert np.abs(ev.decrypt(r).real - C.chebval(x, coef)).max() < 1e-11, deg
    # product-basis coefficients as the reference's tables hold them: random tables against the definition
    for n, baby in ((16, 4), (64, 8), (128, 16), (11, 8), (13, 4)):
        d = rng.normal(size=n)
        r = P.eval_chebyshev(ev, ct, d, baby, multiplier=0.75)
        assert np.abs(ev.decrypt(r).real - 0.75 * P.cheb_product_value(d, baby, t)).max() < 1e-9, (n, baby)
        levels = max(0, (baby - 1).bit_length()) + max(0, (-(-n // baby) - 1).bit_length())
        assert r.level == 12 - levels                         # the header's level_cost = log_bs + log_gs
    # sparse expansions: only T_4 / only T_8 above the constant, and an inner zero
    for coef in ([0.5, 0, 0, 0, 2.0], [0.5, 0, 0, 0, 0, 0, 0, 0, 2.0], [1, 2, 0, 0, 0, 0, 3, 0, 0, 0, 0.5]):
        r = P.eval_chebyshev(ev, ct, P.cheb_plain_to_product(coef, 4), 4)
        assert np.abs(ev.decrypt(r).real - C.chebval(x, coef)).max() < 1e-12
    # the reference's table: exp on [-2, 2] after linearTransform, to the table's accuracy, in level_cost = 4 levels
    x2 = rng.uniform(-2, 2, 512)
    c2 = ev.encrypt(x2)
    u = P.linear_transform(ev, c2, -2.0, 2.0)
    r = P.eval_chebyshev(ev, u, EXP_15_4, 4)
    assert np.abs(ev.decrypt(r).real - np.exp(x2)).max() < 1e-10
    assert r.level == u.level - 4


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
    r = P.eval_chebyshev(ev, ct, EXP_15_4, 4)
    assert np.abs(orc.decrypt(r).real - np.exp(2 * x)).max() < 1e-6
    x2 = rng.uniform(-2, 2, orc.slots)
    c2 = orc.encrypt(orc.encode(x2.astype(np.complex128), orc.nQ - 1), 6)
    r = P.eval_chebyshev(ev, P.linear_transform(ev, c2, -2.0, 2.0), EXP_15_4, 4)
    assert r.level == orc.nQ - 1 - 1 - 4
    assert np.abs(orc.decrypt(r).real - np.exp(x2)).max() < 1e-6
