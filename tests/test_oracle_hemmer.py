"""The restated algorithms over the CPU RNS-CKKS oracle (N = 1024, 16 x 16 tiles): decrypted
products equal float64 A @ B, which pins the composition of oracle primitives that the GPU residues
are later compared against."""
import numpy as np
import pytest

from oracle import hemmer_ref as R
from oracle import oracle as O


@pytest.fixture(scope="module")
def env():
    qs, ps = O.ckks_chain(10, 8, 3)
    orc = O.Oracle(10, qs, ps, dnum=3)
    orc.gen_secret(7)
    orc.gen_mult_key(7)
    orc.gen_conj_key(7)
    n = 16
    orc.key_seed = 7
    return orc, R.OracleEval(orc), n


def enc(orc, M, seed):
    z = np.zeros(orc.slots, dtype=np.complex128)
    z[: M.size] = M.reshape(-1)
    return orc.encrypt(orc.encode(z, orc.nQ - 1), seed)


def test_ccmm_over_oracle(env):
    orc, ev, n = env
    rng = np.random.default_rng(0)
    A, B = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    c = R.mult_mat_mat_cc(ev, enc(orc, A, 11), enc(orc, B, 12), 2, n, n)
    assert c.level == 2
    z = orc.decrypt(c)
    assert np.abs(z[: n * n].real.reshape(n, n) - A @ B).max() < 2 ** -20
    assert np.abs(z[n * n:]).max() < 2 ** -20


@pytest.mark.parametrize("T", [1, 2, 3])
def test_complex_packed_single_ccmm_over_oracle(env, T):
    """One product through the complex-packed route.  With T = 1 the fresh operands (level 7) sit above the packing
    level T + 5: they are only truncated, and the packing masks carry the change of scale.  With T = 3 they sit at
    T + 4: the packing and the first transform stage are one composite map."""
    orc, ev, n = env
    rng = np.random.default_rng(5)
    A, B = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    c = R.mult_mat_mat_cc_packed_single(orc, enc(orc, A, 21), enc(orc, B, 22), T, n, n)
    assert c.level == T and c.scale == orc.delta[T]
    z = orc.decrypt(c)
    assert np.abs(z[: n * n].real.reshape(n, n) - A @ B).max() < 2 ** -18
    assert np.abs(z[: n * n].imag).max() < 2 ** -18
    assert np.abs(z[n * n:]).max() < 2 ** -18


def test_packed_ccmm_over_oracle(env):
    orc, ev, n = env
    rng = np.random.default_rng(1)
    A1, A2, B1, B2 = (rng.uniform(-1, 1, (n, n)) for _ in range(4))
    a = R.complex_packing_cols(ev, enc(orc, np.concatenate([A1, A2], 1), 13), n, 2 * n)
    b = R.complex_packing_rows(ev, enc(orc, np.concatenate([B1, B2], 1), 14), n, 2 * n)
    c = R.repack_cc(ev, R.mult_packed_mat_mat(ev, a, b, 2, n, 2 * n))
    z = orc.decrypt(c).reshape(n, 2 * n)
    assert np.abs(z.real[:, :n] - A1 @ B1).max() < 2 ** -18
    assert np.abs(z.real[:, n:] - A2 @ B2).max() < 2 ** -18
    assert np.abs(z.imag).max() < 2 ** -18


def test_lazy_pcmm_over_oracle(env):
    """The plaintext x ciphertext product with one ModDown (all shifts, masks and rotated weights multiplied and summed
    in the extended basis) decrypts to A @ B at the target level, for a single matrix in the first tile block (the
    other blocks stay empty) and for the pair layout."""
    orc, ev, n = env
    rng = np.random.default_rng(2)
    A, B = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    zb = np.zeros(orc.slots, dtype=np.complex128)
    zb[: n * n] = B.reshape(-1)
    c = R.mult_mat_mat_pc_lazy(orc, enc(orc, A, 15), orc.encode(zb, orc.nQ - 1), 2, n, n)
    assert c.level == 2 and c.scale == orc.delta[2]
    z = orc.decrypt(c)
    assert np.abs(z[: n * n].real.reshape(n, n) - A @ B).max() < 2 ** -20
    assert np.abs(z[n * n:]).max() < 2 ** -20
    A2, B2 = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    zb = np.concatenate([B, B2], 1).reshape(-1).astype(np.complex128)
    c = R.mult_mat_mat_pc_lazy(orc, enc(orc, np.concatenate([A, A2], 1), 16), orc.encode(zb, orc.nQ - 1), 2, n, 2 * n)
    z = orc.decrypt(c).reshape(n, 2 * n)
    assert np.abs(z.real[:, :n] - A @ B).max() < 2 ** -18 and np.abs(z.real[:, n:] - A2 @ B2).max() < 2 ** -18
    # stacked different matrices have no whole-rotation row shift: not handled by this route
    zb = np.concatenate([B.reshape(-1), B2.reshape(-1)]).astype(np.complex128)
    zfull = np.zeros(orc.slots, dtype=np.complex128)
    zfull[: zb.size] = zb
    assert R.mult_mat_mat_pc_lazy(orc, enc(orc, A, 17), orc.encode(zfull, orc.nQ - 1), 2, n, n) is None


@pytest.mark.parametrize("T", [2, 3])
def test_complex_packed_ccmm_on_stacked_tiles_over_oracle(env, T):
    """Two tiles stacked in one ciphertext (block width n, 2 n rows) through the complex-packed product with masked
    shifts of its two-column / two-row cells: each tile block of the result is the product of the operands' blocks.
    T = 3 leaves the fresh operands (level 7) four levels: the packing and the first transform stage are one map."""
    orc, ev, n = env
    rng = np.random.default_rng(6)
    A, B = rng.uniform(-1, 1, (2 * n, n)), rng.uniform(-1, 1, (2 * n, n))
    c = R.mult_mat_mat_cc_packed(orc, enc(orc, A, 23), enc(orc, B, 24), T, n, n, single_tile=False)
    assert c.level == T and c.scale == orc.delta[T]
    z = orc.decrypt(c)
    d = z[: 2 * n * n].real.reshape(2 * n, n)
    assert np.abs(d[:n] - A[:n] @ B[:n]).max() < 2 ** -18
    assert np.abs(d[n:] - A[n:] @ B[n:]).max() < 2 ** -18
    assert np.abs(z.imag).max() < 2 ** -18


@pytest.mark.parametrize("single_tile", [True, False])
def test_complex_packed_ccmm_three_levels_above_target_over_oracle(env, single_tile):
    """Operands only three levels above the target: the packing and the packed transform run as one composite transform
    (one level), the rest of the complex-packed product is unchanged."""
    orc, ev, n = env
    rng = np.random.default_rng(8)
    rows = n if single_tile else 2 * n
    A, B = rng.uniform(-1, 1, (rows, n)), rng.uniform(-1, 1, (rows, n))
    a, b = orc.level_down(enc(orc, A, 25), 5), orc.level_down(enc(orc, B, 26), 5)
    c = R.mult_mat_mat_cc_packed(orc, a, b, 2, n, n, single_tile=single_tile)
    assert c.level == 2 and c.scale == orc.delta[2]
    z = orc.decrypt(c)
    d = z[: rows * n].real.reshape(rows, n)
    assert np.abs(d[:n] - A[:n] @ B[:n]).max() < 2 ** -18
    if not single_tile:
        assert np.abs(d[n:] - A[n:] @ B[n:]).max() < 2 ** -18
    assert np.abs(z.imag).max() < 2 ** -18


@pytest.mark.parametrize("unit,count", [(1, 16), (-1, 32), (-16, 8), (3, 4), (5, 2), (32, 16)])
def test_rotate_sum_as_hoisted_sums_over_oracle(env, unit, count):
    """OracleEval.rotate_sum (at most two stages of one hoisted sum each, the unrotated input as a term without a
    key) decrypts to the sum of the count rotations of its input; (32, 16) wraps round the 512 slots, so one of its
    rotations is a whole turn."""
    orc, ev, _ = env
    rng = np.random.default_rng(9)
    z = rng.uniform(-1, 1, orc.slots) + 1j * rng.uniform(-1, 1, orc.slots)
    x = orc.encrypt(orc.encode(z, 5), 31)
    got = orc.decrypt(ev.rotate_sum(x, unit, count))
    want = sum(np.roll(z, -((i * unit) % orc.slots)) for i in range(count))
    assert np.abs(got - want).max() < 2 ** -20
    assert [c for c, _ in R.rotate_sum_stages(count)] == ([count] if count <= 4 else
                                                          [1 << ((count.bit_length()) // 2), count >> ((count.bit_length()) // 2)])
