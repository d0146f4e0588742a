"""GPU parity of the LoRA low-rank path (rank 2): products with a thin operand, block selection and
repacking.  Small ring (N = 1024, 16 x 16 tiles in the pair layout): every residue must equal the CPU oracle
running the same schedule; decrypted values are checked against float64 products."""
import numpy as np
import pytest

from __graft_entry__ import load_package
from oracle import hemmer_ref as R
from oracle import oracle as O

pytestmark = pytest.mark.gpu
N_TILE, W, LD = 16, 32, 2


@pytest.fixture(scope="module")
def small():
    load_package()
    from efla_amd import hellm
    qs, ps = O.ckks_chain(10, 8, 3)
    H = hellm.HEMMer(10, qs, ps, dnum=3, min_bootstrap_level=0, seed=11)
    orc = O.Oracle(10, qs, ps, dnum=3)
    orc.gen_secret(11)
    orc.gen_mult_key(11)
    orc.gen_conj_key(11)
    orc.key_seed = 11
    return H, orc, R.OracleEval(orc)


def to_oracle(orc, ct):
    i = ct.info()
    assert i["rescale_counter"] == 0
    return O.Ct(ct.residues(), orc.delta[i["level"]])


def transform_of(orc, fused):
    """The oracle runs the batched transforms (through `orc`) or the reference order (None)."""
    return orc if fused else None


def thin_cols(rng, block, n=N_TILE):
    m = np.zeros((n, n))
    m[:, block * LD:(block + 1) * LD] = rng.normal(0, 0.5, (n, LD))
    return m


def thin_rows(rng, block, n=N_TILE):
    m = np.zeros((n, n))
    m[block * LD:(block + 1) * LD] = rng.normal(0, 0.5, (LD, n))
    return m


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_high_low_and_one_col(small, fused):
    H, orc, ev = small
    n, w = N_TILE, W
    H.set_schedule(fused, batch=4)
    rng = np.random.default_rng(21)
    X0, X1 = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    blk = 3
    A0, A1 = thin_cols(rng, blk), thin_cols(rng, blk)
    cx, ca = H.encrypt2(X0, X1), H.encrypt2(A0 + thin_cols(rng, 1), A1 + thin_cols(rng, 5))
    ox, oa = to_oracle(orc, cx), to_oracle(orc, ca)
    low = H.get_low_col_block(ca, blk)
    olow = R.get_low_col_block(ev, oa, blk, n, n, w, LD)
    assert np.array_equal(low.residues(), olow.data)
    got = H.matmul_high_low(cx, low, blk, 3)
    want = R.mult_mat_mat_high_low(ev, ox, olow, blk, 3, (n, n), (n, n), w, LD, transform_of(orc, fused))
    H.set_schedule(True)
    assert got.info()["level"] == 3
    assert np.array_equal(got.residues(), want.data)
    one = H.repack_to_one_col(got, 0)
    assert np.array_equal(one.residues(), R.repack_to_one_col(ev, want, 0, n, n, w, LD).data)
    d = H.decrypt2(one)
    XA = X0 @ A0[:, blk * LD:(blk + 1) * LD] + X1 @ A1[:, blk * LD:(blk + 1) * LD]
    for half in d:
        assert np.abs(half[:, :LD] - XA).max() < 2 ** -16 and np.abs(half[:, LD:]).max() < 2 ** -16
    multi = H.repack_to_multi_col(got, 2)
    assert np.array_equal(multi.residues(), R.repack_to_multi_col(ev, want, 2, n, n, w, LD).data)
    d = H.decrypt2(multi)
    assert np.abs(d[0][:, 2 * LD:3 * LD] - X0 @ A0[:, blk * LD:(blk + 1) * LD]).max() < 2 ** -16
    assert np.abs(d[1][:, 2 * LD:3 * LD] - X1 @ A1[:, blk * LD:(blk + 1) * LD]).max() < 2 ** -16


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_low_high_and_rows(small, fused):
    H, orc, ev = small
    n, w = N_TILE, W
    H.set_schedule(fused, batch=4)
    rng = np.random.default_rng(22)
    blk = 2
    L0 = thin_rows(rng, blk)
    G0, G1 = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    ca, cg = H.encrypt2(L0 + thin_rows(rng, 0), L0 + thin_rows(rng, 7)), H.encrypt2(G0, G1)
    oa, og = to_oracle(orc, ca), to_oracle(orc, cg)
    low = H.get_low_row_block(ca, blk)
    olow = R.get_low_row_block(ev, oa, blk, n, w, LD)
    assert np.array_equal(low.residues(), olow.data)
    got = H.matmul_low_high(low, cg, blk, 3)
    want = R.mult_mat_mat_low_high(ev, olow, og, blk, 3, (n, n), (n, n), w, LD, transform_of(orc, fused))
    H.set_schedule(True)
    assert np.array_equal(got.residues(), want.data)
    thin = L0[blk * LD:(blk + 1) * LD]
    multi = H.repack_to_multi_row(got, 5)
    assert np.array_equal(multi.residues(), R.repack_to_multi_row(ev, want, 5, n, w, LD).data)
    d = H.decrypt2(multi)
    assert np.abs(d[0][5 * LD:6 * LD] - thin @ G0).max() < 2 ** -16
    assert np.abs(d[1][5 * LD:6 * LD] - thin @ G1).max() < 2 ** -16
    assert np.abs(d[0][:5 * LD]).max() < 2 ** -16 and np.abs(d[0][6 * LD:]).max() < 2 ** -16
    one = H.repack_to_one_row(got, 1)
    assert np.array_equal(one.residues(), R.repack_to_one_row(ev, want, 1, n, n, w, LD).data)
    d = H.decrypt2(one)
    for half in d:
        assert np.abs(half[LD:2 * LD] - (thin @ G0 + thin @ G1)).max() < 2 ** -16


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_low_low(small, fused):
    H, orc, ev = small
    n, w = N_TILE, W
    H.set_schedule(fused, batch=4)
    rng = np.random.default_rng(23)
    cb, rb = 0, 4
    A = thin_cols(rng, cb)
    B0, B1 = thin_rows(rng, rb), thin_rows(rng, rb)
    ca, cw = H.encrypt2(A, A), H.encrypt2(B0, B1)
    oa, ow = to_oracle(orc, ca), to_oracle(orc, cw)
    got = H.matmul_low_low(ca, cw, cb, rb, 2)
    want = R.mult_mat_mat_low_low(ev, oa, ow, cb, rb, 2, (n, n), (n, n), w, LD, transform_of(orc, fused))
    H.set_schedule(True)
    assert got.info()["level"] == 2
    assert np.array_equal(got.residues(), want.data)
    d = H.decrypt2(got)
    thin = A[:, cb * LD:(cb + 1) * LD]
    assert np.abs(d[0] - thin @ B0[rb * LD:(rb + 1) * LD]).max() < 2 ** -16
    assert np.abs(d[1] - thin @ B1[rb * LD:(rb + 1) * LD]).max() < 2 ** -16


def test_repack_lora_opti(small):
    H, orc, ev = small
    n = N_TILE
    rng = np.random.default_rng(24)
    A0, A1, B0, B1 = (rng.uniform(-1, 1, (n, n)) for _ in range(4))
    x1 = H.complex_packing(H.encrypt2(A0, A1), H.encrypt2(B0, B1))
    x2 = H.complex_packing(H.encrypt2(B1, A0), H.encrypt2(A1, B0))
    o1, o2 = to_oracle(orc, x1), to_oracle(orc, x2)
    got = H.repack_lora_opti(x1, x2)
    # rescale counters are zero here, so the oracle skips the two leading rescales as the product does
    class NoRescale:
        def __getattr__(self, name):
            return getattr(ev, name)
        def rescale(self, x):
            return x
    want = R.repack_lora_opti(NoRescale(), o1, o2, n)
    assert np.array_equal(got.residues(), want.data)
    out = H.decrypt_slots(got).reshape(n, 2 * n)
    assert np.abs(out[:, :n] - 2 * (A0 + A1)).max() < 2 ** -16
    assert np.abs(out[:, n:] - (2 * A0 + B1 + 1j * A0)).max() < 2 ** -16


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_lora_rank2_elementwise_path(small, fused):
    """Element-wise rank-2 form: residues against the oracle, values against float64; the rotate-and-sum steps in the
    reference's order and as hoisted sums."""
    H, orc, ev = small
    H.set_schedule(fused)
    try:
        _lora_rank2_elementwise_path(H, orc, ev, fused)
    finally:
        H.set_schedule(True)


def _lora_rank2_elementwise_path(H, orc, ev, fused):
    n, w, m = N_TILE, W, 2
    rng = np.random.default_rng(25)
    X = rng.uniform(-1, 1, (n, 2 * n * m))
    A = rng.normal(0, 0.3, (2 * n * m, 2))
    B = rng.normal(0, 0.3, (2, 2 * n * m))
    wa, wb = np.zeros((n, w)), np.zeros((n, w))
    for i in range(m):
        for j in range(2):
            wa[2 * i + j] = A[2 * n * i:2 * n * (i + 1), j]
            wb[2 * i + j] = B[j, 2 * n * i:2 * n * (i + 1)]
    enc2 = lambda M: H.encrypt2(M[:, :n], M[:, n:])
    cur = [enc2(X[:, 2 * n * i:2 * n * (i + 1)]) for i in range(m)]
    cwa, cwb = enc2(wa), enc2(wb)
    ocur, owa, owb = [to_oracle(orc, c) for c in cur], to_oracle(orc, cwa), to_oracle(orc, cwb)
    xa = H.lora_rank2_down(cur, cwa, weight_level=7)
    oxa = R.lora_rank2_down(ev, ocur, owa, n, w, 7, fused)
    for j in range(2):
        assert np.array_equal(xa[j].residues(), oxa[j].data)
        z = H.decrypt_slots(xa[j]).real.reshape(n, w)
        assert np.abs(z[:, 0] - X @ A[:, j]).max() < 2 ** -16 and np.abs(z[:, 1:]).max() < 2 ** -16
    out = H.lora_rank2_up(xa, cwb, m, weight_level=4)
    oout = R.lora_rank2_up(ev, oxa, owb, m, n, w, 4, fused)
    want = X @ A @ B
    for i in range(m):
        assert np.array_equal(out[i].residues(), oout[i].data)
        z = H.decrypt_slots(out[i]).real.reshape(n, w)
        assert np.abs(z - want[:, 2 * n * i:2 * n * (i + 1)]).max() < 2 ** -16
