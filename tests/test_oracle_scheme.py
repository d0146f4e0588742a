"""Pins the oracle's CKKS layer (encode/decode, encrypt/decrypt, key switching, rescale,
level handling) through identities the scheme fixes: the canonical embedding evaluated
directly, and decrypt(op(enc(z))) == op(z) on the slots."""
import numpy as np
import pytest

from oracle import oracle as O


@pytest.fixture(scope="module")
def orc():
    qs, ps = O.ckks_chain(10, 6, 2)
    o = O.Oracle(10, qs, ps, dnum=3)
    o.gen_secret(3, hw=64)
    o.gen_mult_key(6)
    for r in (1, 2, 5, o.slots - 3):
        o.gen_rot_key(6, r)
    o.gen_conj_key(6)
    return o


@pytest.fixture(scope="module")
def z(orc):
    rng = np.random.default_rng(0)
    return rng.uniform(-1, 1, orc.slots) + 1j * rng.uniform(-1, 1, orc.slots)


def test_encode_is_inverse_canonical_embedding():
    """m(zeta^{5^j}) = Delta * z_j for zeta = exp(i pi / N), evaluated directly (O(N^2))."""
    qs, ps = O.ckks_chain(6, 3, 1)
    o = O.Oracle(6, qs, ps, dnum=1)
    rng = np.random.default_rng(1)
    zz = rng.uniform(-1, 1, o.slots) + 1j * rng.uniform(-1, 1, o.slots)
    pt = o.encode(zz, 2)
    d = pt.data[:1].copy()
    o.ntt(d, [0], inverse=True)
    q0 = o.q[0]
    coeffs = np.array([int(v) if int(v) < q0 // 2 else int(v) - q0 for v in d[0]], dtype=np.float64)
    zeta = np.exp(1j * np.pi / o.N)
    for j in range(o.slots):
        x = zeta ** pow(5, j, 2 * o.N)
        val = np.sum(coeffs * x ** np.arange(o.N)) / pt.scale
        assert abs(val - zz[j]) < 1e-9
    # basis vector: slot 0 = 1 -> coefficients (2/N) Re(zeta^{-k}) * Delta / 2 ... check via decode
    e0 = np.zeros(o.slots, dtype=np.complex128)
    e0[0] = 1
    assert np.abs(o.decode(o.encode(e0, 1)) - e0).max() < 1e-9
    # constant message -> constant polynomial
    c = o.encode(np.full(o.slots, 0.75), 0)
    dc = c.data.copy()
    o.ntt(dc, [0], inverse=True)
    assert int(dc[0, 0]) == round(0.75 * c.scale) and not dc[0, 1:].any()


def test_encode_decode_and_encrypt(orc, z):
    pt = orc.encode(z, 5)
    assert np.abs(orc.decode(pt) - z).max() < 1e-9
    ct = orc.encrypt(pt, 4)
    assert ct.level == 5 and np.abs(orc.decrypt(ct) - z).max() < 1e-8
    # b + a*s = m + e exactly, with e the small sampled error
    diff = orc.decrypt_pt(ct).data[0].copy()
    diff = (diff.astype(object) - pt.data[0].astype(object)) % orc.q[0]
    d = np.array(diff, dtype=np.uint64)[None]
    orc.ntt(d, [0], inverse=True)
    e = np.array([int(v) if int(v) < orc.q[0] // 2 else int(v) - orc.q[0] for v in d[0]])
    assert np.abs(e).max() <= 21


def test_rotation_conjugation_composition(orc, z):
    ct = orc.encrypt(orc.encode(z, 5), 4)
    for r in (1, 2, 5):
        assert np.abs(orc.decrypt(orc.left_rotate(ct, r)) - np.roll(z, -r)).max() < 1e-7
    assert np.abs(orc.decrypt(orc.right_rotate(ct, 3)) - np.roll(z, 3)).max() < 1e-7
    assert np.abs(orc.decrypt(orc.conjugate(ct)) - np.conj(z)).max() < 1e-7
    r12 = orc.left_rotate(orc.left_rotate(ct, 1), 2)
    assert np.abs(orc.decrypt(r12) - np.roll(z, -3)).max() < 1e-7
    # plaintext rotation needs no key
    pt = orc.left_rotate(orc.encode(z, 3), 7)
    assert np.abs(orc.decode(pt) - np.roll(z, -7)).max() < 1e-9


def test_mult_rescale_leveldown(orc, z):
    ct = orc.encrypt(orc.encode(z, 5), 4)
    c3 = orc.mult(ct, ct)
    assert c3.level == 4 and abs(c3.scale / orc.delta[4] - 1) < 1e-12
    assert np.abs(orc.decrypt(c3) - z * z).max() < 1e-7
    t = orc.tensor(ct, ct)                       # 3-poly decrypts with s^2
    assert np.abs(orc.decrypt(t) - z * z).max() < 1e-7
    w = np.random.default_rng(5).uniform(-1, 1, orc.slots)
    assert np.abs(orc.decrypt(orc.mult_msg(ct, w)) - z * w).max() < 1e-7
    c5 = orc.level_down(ct, 2)
    assert c5.level == 2 and np.abs(orc.decrypt(c5) - z).max() < 1e-7
    assert np.abs(orc.decrypt(orc.mult_imag_unit(ct)) - 1j * z).max() < 1e-8
    s = orc.add(c3, orc.level_down(ct, 4))
    assert np.abs(orc.decrypt(s) - (z * z + z)).max() < 1e-7
    assert np.abs(orc.decrypt(orc.mult_const(ct, 0.37)) - 0.37 * z).max() < 1e-7
    assert np.abs(orc.decrypt(orc.mult_integer(ct, -2)) + 2 * z).max() < 1e-7
    assert np.abs(orc.decrypt(orc.sub(ct, ct))).max() < 1e-7
    assert np.abs(orc.decrypt(orc.negate(ct)) + z).max() < 1e-7


@pytest.mark.parametrize("c", [0.37, -1.25, 0.5 - 0.75j, -3.0j])
def test_constant_added_on_the_residues_equals_an_encoded_constant_message(orc, z, c):
    """add(ct, constant) without a plaintext: the residues must be those of adding the encoding of the message that
    holds the constant in every slot (the embedding of a constant is re Delta + im Delta X^(N/2)), and the
    ciphertext must decrypt to z + c."""
    ct = orc.encrypt(orc.encode(z, orc.nQ - 1), 21)
    direct = orc.add_constant_residues(ct.data, complex(c), ct.level)
    via_message = orc.add(ct, orc.encode(np.full(orc.slots, c, dtype=np.complex128), ct.level))
    assert np.array_equal(direct, via_message.data)
    assert np.abs(orc.decrypt(O.Ct(direct, ct.scale)) - (z + c)).max() < 1e-6
