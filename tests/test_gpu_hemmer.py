"""GPU parity of the HEMMer layer.

Small ring (N = 1024, 16 x 16 tiles): the GPU path and the CPU oracle share primes, seed-derived
secret / evaluation keys and input ciphertexts, run the same operation sequence, and must agree on
every residue (bit-exact).  Full ring (N = 2^16, 128 x 128 tiles, 13 + 4 primes, dnum 3, scale 2^42):
decrypted products are checked against float64 A @ B within 2^-12 max-abs (tolerance asked for the
128 x 128 CCMM on U(-1,1) inputs; the reference's own checks use 2^-15 .. 2^-10)."""
import numpy as np
import pytest

from __graft_entry__ import load_package
from oracle import hemmer_ref as R
from oracle import oracle as O

pytestmark = pytest.mark.gpu
TOL = 2.0 ** -12


def gen_oracle_keys(orc, seed, n):
    orc.gen_secret(seed)
    orc.gen_mult_key(seed)
    orc.gen_conj_key(seed)
    orc.key_seed = seed          # rotation keys are derived from (seed, Galois element) on first use


@pytest.fixture(scope="module")
def small():
    pkg = load_package()
    from efla_amd import hellm
    qs, ps = O.ckks_chain(10, 8, 3)
    H = hellm.HEMMer(10, qs, ps, dnum=3, min_bootstrap_level=0, seed=7)
    orc = O.Oracle(10, qs, ps, dnum=3)
    gen_oracle_keys(orc, 7, H.dim)
    return H, orc, R.OracleEval(orc)


@pytest.fixture(scope="module")
def full():
    load_package()
    from efla_amd import hellm
    return hellm.HEMMer(preset=True, seed=3)


def to_oracle(orc, ct):
    i = ct.info()
    assert i["rescale_counter"] == 0
    return O.Ct(ct.residues(), orc.delta[i["level"]])


def test_keys_and_encoding_match_oracle(small):
    H, orc, _ = small
    assert np.array_equal(H.secret_coeffs(), orc.sk_coeffs)
    assert np.array_equal(H.export_key(0), orc.keys["mult"])
    H.ensure_rotation_keys([1, 5])
    for r in (1, 5):
        orc.gen_rot_key(7, r)
        g = orc.galois(r)
        assert np.array_equal(H.export_key(g), orc.keys[("gal", g)])
    assert np.array_equal(H.export_key(2 * H.N - 1), orc.keys[("gal", 2 * H.N - 1)])
    # host-side encoding (embedding FFT + rounding) gives the oracle's residues
    rng = np.random.default_rng(1)
    M = rng.uniform(-1, 1, (16, 16))
    z = np.zeros(orc.slots, dtype=np.complex128)
    z[:256] = M.reshape(-1)
    for level in (7, 3):
        assert np.array_equal(H.encode(M, level).residues(), orc.encode(z, level).data)


def test_plaintext_pair_packing_bit_exact(small):
    """HEMMer::complexPacking(PtxtTensor, PtxtTensor): 0.5 a - 0.5 i b, decoded, combined and encoded again at the lower
    level -- the oracle's decode / encode of the same residues gives the same plaintext."""
    H, orc, _ = small
    rng = np.random.default_rng(17)
    A, B = rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
    a, b = H.encode(A, 5), H.encode(B, 3)
    p = H.complex_packing_pt(a, b)
    za = orc.decode(O.Pt(a.residues(), orc.delta[5]))
    zb = orc.decode(O.Pt(b.residues(), orc.delta[3]))
    want = orc.encode(0.5 * za - 0.5j * zb, 3)
    assert np.array_equal(p.residues(), want.data)
    got = orc.decode(O.Pt(p.residues(), orc.delta[3]))[:256].reshape(16, 16)
    assert np.abs(got - (0.5 * A - 0.5j * B)).max() < 1e-9


def test_evaluator_calls_bit_exact(small):
    H, orc, ev = small
    rng = np.random.default_rng(2)
    A, B = rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
    ca, cb = H.encrypt(A), H.encrypt(B)
    oa, ob = to_oracle(orc, ca), to_oracle(orc, cb)
    assert np.abs(orc.decrypt(oa)[:256].real.reshape(16, 16) - A).max() < 1e-8
    assert np.array_equal(H.left_rotate(ca, 1).residues(), ev.left_rotate(oa, 1).data)
    assert np.array_equal(H.conjugate(ca).residues(), ev.conjugate(oa).data)
    assert np.array_equal(H.mult(ca, cb).residues(), ev.mult(oa, ob).data)
    assert np.array_equal(H.level_down(ca, 3).residues(), ev.level_down(oa, 3).data)
    assert np.array_equal(H.mult_imag_unit(ca).residues(), ev.mult_imag_unit(oa).data)
    lo = H.level_down(cb, 4)
    assert np.array_equal(H.add(ca, lo).residues(), ev.add(oa, ev.level_down(ob, 4)).data)


def test_sigma_tau_bit_exact(small):
    H, orc, ev = small
    rng = np.random.default_rng(3)
    A = rng.uniform(-1, 1, (16, 16))
    ca = H.encrypt(A)
    oa = to_oracle(orc, ca)
    H.set_schedule(False)
    s = H.diagonal_to_column(ca)
    assert np.array_equal(s.residues(), R.diagonal_transform(ev, oa, R.H, 16, 16).data)
    t = H.diagonal_to_row(ca)
    assert np.array_equal(t.residues(), R.diagonal_transform(ev, oa, R.V, 16, 16).data)
    H.set_schedule(True)
    sb, tb = H.diagonal_to_column(ca), H.diagonal_to_row(ca)
    assert np.array_equal(sb.residues(), R.diagonal_transform_fused(orc, oa, R.H, 16, 16).data)
    assert np.array_equal(tb.residues(), R.diagonal_transform_fused(orc, oa, R.V, 16, 16).data)
    assert np.abs(H.decrypt(sb) - H.decrypt(s)).max() < 1e-7 and np.abs(H.decrypt(tb) - H.decrypt(t)).max() < 1e-7
    i, j = np.meshgrid(np.arange(16), np.arange(16), indexing="ij")
    assert np.abs(H.decrypt(s) - A[i, (i + j) % 16]).max() < 1e-7
    tr = ca.clone()
    H.set_schedule(False)
    H.transpose_inplace(tr)
    H.set_schedule(True)
    assert np.array_equal(tr.residues(), R.transpose(ev, oa, 16, 16).data)
    # batched schedule: the diagonals in sigma / tau's grouping through the batched transform
    tb = ca.clone()
    H.transpose_inplace(tb)
    assert np.array_equal(tb.residues(), R.diagonal_transform_fused(orc, oa, R.DIAG_SIGNED, 16, 16).data)
    assert np.abs(H.decrypt(tb) - A.T).max() < 1e-7


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_ccmm_residues_bit_exact_and_decrypts(small, fused):
    """Both schedules of singleCCMatMul against the oracle running the same schedule."""
    H, orc, ev = small
    rng = np.random.default_rng(4)
    A, B = rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
    ca, cb = H.encrypt(A), H.encrypt(B)
    H.set_schedule(fused, batch=4)
    try:
        c = H.single_cc_matmul(ca, cb, 2)
    finally:
        H.set_schedule(True)
    oa, ob = to_oracle(orc, ca), to_oracle(orc, cb)
    # operands straight from encrypt() are known to hold a single tile and have levels to spare: the batched schedule
    # takes the complex-packed route (half the column shifts) with tau(B) spread over the blocks
    want = (R.mult_mat_mat_cc_packed_single(orc, oa, ob, 2, 16, 16) if fused
            else R.mult_mat_mat_cc(ev, oa, ob, 2, 16, 16))
    assert c.info()["level"] == 2
    assert np.array_equal(c.residues(), want.data)
    assert np.abs(H.decrypt(c) - A @ B).max() < 2 ** -20


def test_ccmm_single_tile_promise(small):
    """With the promise that the operands hold one tile block and nothing else, tau(B) is spread over every block
    and the product takes the baby-step / giant-step route; the result still lives in the first block only."""
    H, orc, ev = small
    rng = np.random.default_rng(15)
    A, B = rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
    ca, cb = H.encrypt(A), H.encrypt(B)
    H.set_schedule(True, batch=3)
    H.assume_single_tile(True)
    try:
        c = H.single_cc_matmul(ca, cb, 2)
    finally:
        H.assume_single_tile(False)
        H.set_schedule(True)
    want = R.mult_mat_mat_cc_packed_single(orc, to_oracle(orc, ca), to_oracle(orc, cb), 2, 16, 16)
    assert c.info()["level"] == 2
    assert np.array_equal(c.residues(), want.data)
    assert np.abs(H.decrypt(c) - A @ B).max() < 2 ** -20
    assert np.abs(H.decrypt_slots(c)[256:]).max() < 2 ** -20
    # without a level to spare for a separate packing (operands at T+3) the packing and the packed transform run as
    # one composite transform
    H.assume_single_tile(True)
    try:
        la, lb = H.level_down(ca, 5), H.level_down(cb, 5)
        c5 = H.single_cc_matmul(la, lb, 2)
    finally:
        H.assume_single_tile(False)
    want5 = R.mult_mat_mat_cc_packed_single(orc, to_oracle(orc, la), to_oracle(orc, lb), 2, 16, 16)
    assert np.array_equal(c5.residues(), want5.data)
    assert np.abs(H.decrypt(c5) - A @ B).max() < 2 ** -20


def test_ccmm_packed_route_at_lower_and_mixed_levels(small):
    """The complex-packed route away from its preferred levels (A >= T+5, B >= T+4: separate packing, two-stage
    transforms).  An A at T+4 or a B at T+3 takes the packing and the first transform stage as one composite map and
    then the second stage, an A at T+3 the composite one-stage transform; operands above the level their way starts
    from are truncated to it, the first masks on the way absorbing the change of scale."""
    H, orc, ev = small
    rng = np.random.default_rng(23)
    A, B = rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
    ca, cb = H.encrypt(A), H.encrypt(B)
    top = ca.info()["level"]
    assert top == 7
    for T, la, lb in ((2, 6, 6), (2, 7, 6), (2, 6, 7), (1, 7, 7), (1, 7, 6), (1, 5, 7), (2, 7, 5), (2, 6, 5), (2, 5, 7),
                      (3, 7, 6)):
        a = H.level_down(ca, la) if la < top else ca
        b = H.level_down(cb, lb) if lb < top else cb
        c = H.single_cc_matmul(a, b, T)
        want = R.mult_mat_mat_cc_packed_single(orc, to_oracle(orc, a), to_oracle(orc, b), T, 16, 16)
        assert c.info()["level"] == T
        assert np.array_equal(c.residues(), want.data), (T, la, lb)
        assert np.abs(H.decrypt(c) - A @ B).max() < 2 ** -20


def test_ccmm_stacked_tiles_keep_block_products(small):
    """Two 16 x 16 tiles stacked in one ciphertext (block width 16, 32 rows): nothing is known about which slots
    are empty, so the batched schedule must keep the masked row shifts and return both block products."""
    H, orc, ev = small
    rng = np.random.default_rng(16)
    A, B = rng.uniform(-1, 1, (32, 16)), rng.uniform(-1, 1, (32, 16))
    ea, eb = H.encrypt(A), H.encrypt(B)
    ca = H.upload(ea.residues(), 16, 16, 16)       # same residues, declared as 16 x 16 tiles
    cb = H.upload(eb.residues(), 16, 16, 16)
    H.set_schedule(True, batch=5)
    c = H.single_cc_matmul(ca, cb, 2)
    H.set_schedule(True)
    # four levels to spare: the complex-packed product with masked shifts of its two-column / two-row cells
    want = R.mult_mat_mat_cc_packed(orc, to_oracle(orc, ca), to_oracle(orc, cb), 2, 16, 16, single_tile=False)
    assert np.array_equal(c.residues(), want.data)
    d = H.decrypt_slots(c).real[:512].reshape(32, 16)
    assert np.abs(d[:16] - A[:16] @ B[:16]).max() < 2 ** -18
    assert np.abs(d[16:] - A[16:] @ B[16:]).max() < 2 ** -18
    # (the same at T+4: packing and first transform stage as one composite map for both operands, then the second stage)
    c4 = H.single_cc_matmul(H.level_down(ca, 6), cb, 2)
    want4 = R.mult_mat_mat_cc_packed(orc, to_oracle(orc, H.level_down(ca, 6)), to_oracle(orc, cb), 2, 16, 16, single_tile=False)
    assert np.array_equal(c4.residues(), want4.data)
    d = H.decrypt_slots(c4).real[:512].reshape(32, 16)
    assert np.abs(d[:16] - A[:16] @ B[:16]).max() < 2 ** -18 and np.abs(d[16:] - A[16:] @ B[16:]).max() < 2 ** -18
    # three levels to spare: packing and packed transform as one composite transform, then the same masked shifts
    la, lb = H.level_down(ca, 5), H.level_down(cb, 5)
    c1 = H.single_cc_matmul(la, lb, 2)
    want1 = R.mult_mat_mat_cc_packed(orc, to_oracle(orc, la), to_oracle(orc, lb), 2, 16, 16, single_tile=False)
    assert np.array_equal(c1.residues(), want1.data)
    d = H.decrypt_slots(c1).real[:512].reshape(32, 16)
    assert np.abs(d[:16] - A[:16] @ B[:16]).max() < 2 ** -18
    assert np.abs(d[16:] - A[16:] @ B[16:]).max() < 2 ** -18
    # mixed levels with the lower operand three above the target
    c3 = H.single_cc_matmul(ca, lb, 2)
    want3 = R.mult_mat_mat_cc_packed(orc, to_oracle(orc, ca), to_oracle(orc, lb), 2, 16, 16, single_tile=False)
    assert np.array_equal(c3.residues(), want3.data)
    # a rotation forgets what was known about a single tile: with such a B the masked route again
    ea16 = H.encrypt(A[:16])
    rb = H.left_rotate(H.left_rotate(H.encrypt(B[:16]), 3), 512 - 3)
    c2 = H.single_cc_matmul(ea16, rb, 2)
    want2 = R.mult_mat_mat_cc_packed(orc, to_oracle(orc, ea16), to_oracle(orc, rb), 2, 16, 16, single_tile=False)
    assert np.array_equal(c2.residues(), want2.data)
    assert np.abs(H.decrypt(c2) - A[:16] @ B[:16]).max() < 2 ** -18


def test_ccmm_only_the_right_operand_has_to_be_a_known_single_tile(small):
    """A carries a second tile (or anything else) beyond its first block and nothing is known about it; B comes from
    encrypt.  tau(B) can still be spread over the blocks, so the product takes the single-tile route (residues of the
    oracle's restatement of it), the first block of the result is A1 B, and the result is not taken for a single
    tile afterwards: used as the right operand of another product it goes through the masked route."""
    H, orc, ev = small
    rng = np.random.default_rng(41)
    A, B, C = rng.uniform(-1, 1, (32, 16)), rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
    ea = H.encrypt(A)
    ca = H.upload(ea.residues(), 16, 16, 16)        # two stacked tiles declared as one 16 x 16 tensor
    cb = H.encrypt(B)
    for la, lb in ((7, 7), (6, 7), (5, 5)):          # separate packing at T+5 / T+4, composite transform at T+3
        a = H.level_down(ca, la) if la < 7 else ca
        b = H.level_down(cb, lb) if lb < 7 else cb
        c = H.single_cc_matmul(a, b, 2)
        want = R.mult_mat_mat_cc_packed(orc, to_oracle(orc, a), to_oracle(orc, b), 2, 16, 16, single_tile=True)
        assert np.array_equal(c.residues(), want.data), (la, lb)
        assert np.abs(H.decrypt(c) - A[:16] @ B).max() < 2 ** -18
    assert np.abs(H.decrypt_slots(c)[256:]).max() > 2 ** -6          # the other block is not empty ...
    cc = H.encrypt(C)
    # ... and the result does not pass for a single tile: as a right operand it takes the masked route
    hi = H.single_cc_matmul(ca, cb, 4)
    d = H.single_cc_matmul(H.level_down(cc, 4), hi, 1)
    want = R.mult_mat_mat_cc_packed(orc, to_oracle(orc, H.level_down(cc, 4)), to_oracle(orc, hi), 1, 16, 16, single_tile=False)
    assert np.array_equal(d.residues(), want.data)
    assert np.abs(H.decrypt(d) - C @ (A[:16] @ B)).max() < 2 ** -16


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_ccmm_pair_layout(small, fused):
    """Two products per call on the pair layout [A1 | A2] x [B1 | B2] (rows fill the slot vector, so the
    row wrap is a whole turn)."""
    H, orc, ev = small
    H.set_schedule(fused, batch=4)
    rng = np.random.default_rng(9)
    A1, A2, B1, B2 = (rng.uniform(-1, 1, (16, 16)) for _ in range(4))
    ca, cb = H.encrypt2(A1, A2), H.encrypt2(B1, B2)
    c = H.single_cc_matmul(ca, cb, 2)
    H.set_schedule(True)
    oa, ob = to_oracle(orc, ca), to_oracle(orc, cb)
    # tile block = slot vector and levels to spare: the batched schedule takes the complex-packed route
    want = R.mult_mat_mat_cc_packed_single(orc, oa, ob, 2, 16, 32) if fused else R.mult_mat_mat_cc(ev, oa, ob, 2, 16, 32)
    assert np.array_equal(c.residues(), want.data)
    d = H.decrypt2(c)
    assert np.abs(d[0] - A1 @ B1).max() < 2 ** -18 and np.abs(d[1] - A2 @ B2).max() < 2 ** -18


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_pcmm_pair_layout(small, fused):
    """Plaintext x ciphertext product on the pair layout (two products per call); the batched schedule takes the
    hoisted route because the plaintext's row shifts are whole rotations there."""
    H, orc, ev = small
    H.set_schedule(fused, batch=5)
    rng = np.random.default_rng(14)
    A1, A2, B1, B2 = (rng.uniform(-1, 1, (16, 16)) for _ in range(4))
    ca = H.encrypt2(A1, A2)
    pb = H.encode2(B1, B2)
    c = H.single_matmul(ca, pb, 2)
    H.set_schedule(True)
    opb = O.Pt(pb.residues(), orc.delta[orc.nQ - 1])
    oa = to_oracle(orc, ca)
    want = R.mult_mat_mat_pc_lazy(orc, oa, opb, 2, 16, 32) if fused else R.mult_mat_mat_pc(ev, oa, opb, 2, 16, 32)
    assert np.array_equal(c.residues(), want.data)
    d = H.decrypt2(c)
    assert np.abs(d[0] - A1 @ B1).max() < 2 ** -18 and np.abs(d[1] - A2 @ B2).max() < 2 ** -18


def test_pcmm_weight_preparation_follows_the_weight_content(small):
    """The batched plaintext product keeps tau of a weight under a hash of the weight's residues: the same weight gives
    the same residues on every call, and another weight -- also one that lands in the device buffer the first one
    left -- gives its own product."""
    H, orc, ev = small
    H.set_schedule(True)
    rng = np.random.default_rng(21)
    A, B1, B2 = (rng.uniform(-1, 1, (16, 16)) for _ in range(3))
    ca = H.encrypt(A)
    p1 = H.encode(B1)
    first = H.single_matmul(ca, p1, 2).residues()
    again = H.single_matmul(ca, p1, 2).residues()
    assert np.array_equal(first, again)
    del p1
    p2 = H.encode(B2)
    c2 = H.single_matmul(ca, p2, 2)
    assert np.abs(H.decrypt(c2) - A @ B2).max() < 2 ** -20
    p1 = H.encode(B1)
    assert np.array_equal(H.single_matmul(ca, p1, 2).residues(), first)


def test_batch_size_does_not_change_residues(small):
    H, _, _ = small
    rng = np.random.default_rng(14)
    A, B = rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
    ca, cb = H.encrypt(A), H.encrypt(B)
    outs = []
    for batch in (1, 5, 16):
        H.set_schedule(True, batch=batch)
        outs.append(H.single_cc_matmul(ca, cb, 2).residues())
    H.set_schedule(True)
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_pcmm_and_packed_bit_exact(small, fused):
    H, orc, ev = small
    H.set_schedule(fused, batch=3)
    rng = np.random.default_rng(5)
    A, B = rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
    ca = H.encrypt(A)
    pb = H.encode(B)
    c = H.single_matmul(ca, pb, 2)
    opb = O.Pt(pb.residues(), orc.delta[orc.nQ - 1])
    if fused:   # single matrix in the first tile block: tau(B) copied into every block, masks on the first block
        want = R.mult_mat_mat_pc_lazy(orc, to_oracle(orc, ca), opb, 2, 16, 16)
    else:
        want = R.mult_mat_mat_pc(ev, to_oracle(orc, ca), opb, 2, 16, 16)
    assert np.array_equal(c.residues(), want.data)
    assert np.abs(H.decrypt(c) - A @ B).max() < 2 ** -20
    assert np.abs(H.decrypt_slots(c)[256:]).max() < 2 ** -20      # nothing outside the first tile block
    A2, B2 = rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
    pa, pbb = H.encrypt2(A, A2), H.encrypt2(B, B2)
    oa, ob = to_oracle(orc, pa), to_oracle(orc, pbb)
    H.complex_packing_inplace(pa)
    H.complex_packing_row_inplace(pbb)
    oa = R.complex_packing_cols(ev, oa, 16, 32)
    ob = R.complex_packing_rows(ev, ob, 16, 32)
    assert np.array_equal(pa.residues(), oa.data) and np.array_equal(pbb.residues(), ob.data)
    pc = H.repack_cc(H.packed_matmul(pa, pbb, 2))
    H.set_schedule(True)
    prod = R.mult_packed_mat_mat_fused(orc, oa, ob, 2, 16, 32) if fused else R.mult_packed_mat_mat(ev, oa, ob, 2, 16, 32)
    want = R.repack_cc(ev, prod)
    assert np.array_equal(pc.residues(), want.data)
    d = H.decrypt2(pc)
    assert np.abs(d[0] - A @ B).max() < 2 ** -18 and np.abs(d[1] - A2 @ B2).max() < 2 ** -18


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_hoisted_products_bit_exact(small, fused):
    H, orc, ev = small
    n = 16
    H.set_schedule(fused, batch=6)
    rng = np.random.default_rng(6)
    X0, X1 = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    W = [rng.normal(0, 0.02, (n, n)) for _ in range(4)]
    x = H.complex_packing(H.encrypt2(X0, X0), H.encrypt2(X1, X1))
    ox = to_oracle(orc, x)
    tmp = H.matmul_pre(x, 2)
    H.set_schedule(True)
    otmp = R.mult_mat_mat_pre_fused(orc, ox, 2, n, 2 * n) if fused else R.mult_mat_mat_pre(ev, ox, 2, n, 2 * n)
    assert len(tmp) == n
    for k in (0, 1, n - 1):
        assert np.array_equal(tmp.get(k, n, n, 2 * n).residues(), otmp[k].data)
    wp = H.encode_diagonal_to_row4(*W, level=3)
    owp = orc.encode(R.weights_diagonal_to_row4(*W, orc.slots), 3)
    assert np.array_equal(wp.residues(), owp.data)
    y = H.matmul_reuse(tmp, wp, 2)
    assert np.array_equal(y.residues(), R.mult_mat_mat_reuse(ev, otmp, owp, 2).data)
    z = H.decrypt2(H.repack_cc(y))
    assert np.abs(z[0] - (X0 @ W[0] + X1 @ W[2])).max() < 2 ** -18
    assert np.abs(z[1] - (X0 @ W[1] + X1 @ W[3])).max() < 2 ** -18


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_reuse_variants_and_repacking(small, fused):
    """The ciphertext x ciphertext re-use forms (matMulPre + matMulPreRev + matMulCCReUse and their packed
    counterparts), splitInTwo, complexPackingRev and repack_notBTS against float64 algebra on the slots."""
    H, orc, ev = small
    n, T = 16, 2
    H.set_schedule(fused, batch=5)
    rng = np.random.default_rng(8)
    A0, A1, B0, B1 = (rng.uniform(-1, 1, (n, n)) for _ in range(4))
    a, b = H.encrypt2(A0, A1), H.encrypt2(B0, B1)
    # sigma(A) shifts once, tau(B) once, then sum_k shift_k(sigma A) (x) rowrot_k(tau B)
    tmp = H.matmul_pre(a, T)
    bt = H.matmul_pre_rev(b, T)
    c = H.matmul_cc_reuse(tmp, bt, T)
    d = H.decrypt2(c)
    assert np.abs(d[0] - A0 @ B0).max() < 2 ** -18 and np.abs(d[1] - A1 @ B1).max() < 2 ** -18
    otmp = [to_oracle(orc, tmp.get(k, n, n, 2 * n)) for k in range(len(tmp))]
    if fused:   # tau(B) through the batched transform, then all its rotations from one ModUp: residues
        assert np.array_equal(bt.residues(), R.lower_and_transform_fused(orc, to_oracle(orc, b), R.V, n, 2 * n, T + 1).data)
        want = R.mult_mat_mat_cc_reuse_fused(orc, otmp, to_oracle(orc, bt), 2 * n)
        assert np.array_equal(c.residues(), want.data)
    else:       # reference order: levelDown + tau, then the chained rotations of tau(B)
        assert np.array_equal(bt.residues(), R.mult_mat_mat_pre_rev(ev, to_oracle(orc, b), T, n, 2 * n).data)
        assert np.array_equal(c.residues(), R.mult_mat_mat_cc_reuse(ev, otmp, to_oracle(orc, bt), 2 * n).data)
    # packed counterparts: the same product as packedMatMul
    pa, pb = H.encrypt2(A0, A1), H.encrypt2(B0, B1)
    H.complex_packing_inplace(pa)
    H.complex_packing_row_inplace(pb)
    sa = H.packed_matmul_pre(pa, T)
    ptmp = H.packed_matmul_pre_rot(sa, T)
    pbt = H.packed_matmul_pre_rev(pb, T)
    pprod = H.packed_matmul_cc_reuse(ptmp, pbt, T)
    pc = H.repack_cc(pprod)
    d = H.decrypt2(pc)
    assert np.abs(d[0] - A0 @ B0).max() < 2 ** -18 and np.abs(d[1] - A1 @ B1).max() < 2 ** -18
    if not fused:
        osa = R.mult_mat_mat_pre_rev(ev, to_oracle(orc, pa), T + 1, n, 2 * n, kind=R.PH)   # multPackedMatMatPre: T + 3
        assert np.array_equal(sa.residues(), osa.data)
        want_rot = R.mult_packed_mat_mat_pre_rot(ev, osa, T, n, 2 * n)
        assert len(ptmp) == len(want_rot) == n // 2
        for k in range(len(ptmp)):
            assert np.array_equal(ptmp.get(k, n, n, 2 * n).residues(), want_rot[k].data), k
        assert np.array_equal(pbt.residues(), R.mult_mat_mat_pre_rev(ev, to_oracle(orc, pb), T, n, 2 * n, kind=R.PV).data)
        want = R.mult_mat_mat_cc_reuse(ev, want_rot, to_oracle(orc, pbt), 4 * n, rescale_after=True)
        assert np.array_equal(pprod.residues(), want.data)
    if fused:
        osa = R.lower_and_transform_fused(orc, to_oracle(orc, pa), R.PH, n, 2 * n, T + 2)
        assert np.array_equal(sa.residues(), osa.data)
        want_rot = R.mult_packed_mat_mat_pre_rot_fused(orc, osa, T, n, 2 * n)
        assert len(ptmp) == len(want_rot) == n // 2
        for k in range(len(ptmp)):
            assert np.array_equal(ptmp.get(k, n, n, 2 * n).residues(), want_rot[k].data), k
        assert np.array_equal(pbt.residues(), R.lower_and_transform_fused(orc, to_oracle(orc, pb), R.PV, n, 2 * n, T + 1).data)
        optmp = [to_oracle(orc, ptmp.get(k, n, n, 2 * n)) for k in range(len(ptmp))]
        want = R.mult_mat_mat_cc_reuse_fused(orc, optmp, to_oracle(orc, pbt), 4 * n, rescale_after=True)
        assert np.array_equal(pprod.residues(), want.data)
    H.set_schedule(True)
    # splitInTwo: [A0 | A1] -> [A0 | A0], [A1 | A1]
    both = H.encrypt2(A0, A1)
    t1, t2 = H.split_in_two(both)
    w1, w2 = R.split_in_two(ev, to_oracle(orc, both), n)
    assert np.array_equal(t1.residues(), w1.data) and np.array_equal(t2.residues(), w2.data)
    d1, d2 = H.decrypt2(t1), H.decrypt2(t2)
    for got, want in ((d1[0], A0), (d1[1], A0), (d2[0], A1), (d2[1], A1)):
        assert np.abs(got - want).max() < 2 ** -20
    # complexPackingRev: x - i y
    ra, rb = H.encrypt2(A0, A1), H.encrypt2(B0, B1)
    rev = H.complex_packing_rev(ra, rb)
    # HEMMer::complexPackingRev (HEMMer.cpp:987-994): multImagUnit of the second operand, subtracted from the first
    assert np.array_equal(rev.residues(), ev.sub(to_oracle(orc, ra), ev.mult_imag_unit(to_oracle(orc, rb))).data)
    z = H.decrypt_slots(rev)
    want = np.concatenate([A0, A1], axis=1).ravel() - 1j * np.concatenate([B0, B1], axis=1).ravel()
    assert np.abs(z - want).max() < 2 ** -20
    # repack_notBTS: o = 2 Re(t1) + 2i Re(t2); left half <- o + rot(o, n) on the left columns, right half <-
    # the left columns of rot(o, n)
    x1 = H.complex_packing(H.encrypt2(A0, A1), H.encrypt2(B0, B1))     # A + iB
    x2 = H.complex_packing(H.encrypt2(B1, A0), H.encrypt2(A1, B0))
    repacked = H.repack_not_bts(x1, x2)
    want_ct = R.repack_not_bts(ev, to_oracle(orc, x1), to_oracle(orc, x2), n, rescale_first=False)
    assert np.array_equal(repacked.residues(), want_ct.data)
    out = H.decrypt_slots(repacked)
    s1 = np.concatenate([A0, A1], axis=1).ravel()
    s2 = np.concatenate([B1, A0], axis=1).ravel()
    o = 2 * s1 + 2j * s2
    rot = np.roll(o, -n)
    m = np.concatenate([np.ones((n, n)), np.zeros((n, n))], axis=1).ravel()
    want = (o + rot) * m + np.roll(rot * m, n)
    assert np.abs(out - want).max() < 2 ** -18


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
@pytest.mark.parametrize("target_level", [0, 3])
def test_transpose_complex_packing_inplace(small, fused, target_level):
    """HEMMer::transposeComplexPackingInplace: columns (2c, 2c+1) -> a - i b written to both, optional levelDown,
    transpose; residues against the restatement, slots against the closed form."""
    H, orc, ev = small
    n = 16
    rng = np.random.default_rng(21)
    A0, A1 = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    x = H.encrypt2(A0, A1)
    ox = to_oracle(orc, x)
    H.set_schedule(fused)
    try:
        H.transpose_complex_packing_inplace(x, target_level)
    finally:
        H.set_schedule(True)
    want = R.transpose_complex_packing(ev, ox, n, 2 * n, target_level, fused_orc=orc if fused else None)
    assert x.info()["level"] == want.level
    assert np.array_equal(x.residues(), want.data)
    M = np.concatenate([A0, A1], axis=1)                      # rows of the pair layout, 2n wide
    P = np.empty_like(M, dtype=np.complex128)
    P[:, 0::2] = M[:, 0::2] - 1j * M[:, 1::2]
    P[:, 1::2] = P[:, 0::2]
    z = H.decrypt_slots(x).reshape(n, 2 * n)
    for half in (0, 1):
        assert np.abs(z[:, half * n:(half + 1) * n] - P[:, half * n:(half + 1) * n].T).max() < 2 ** -18


@pytest.mark.parametrize("fused", [False, True], ids=["reference-order", "batched"])
def test_rotate_and_sum_reductions(small, fused):
    """Row reductions on the pair layout: residues against the oracle restatement, values against numpy.  The
    reference's order adds log2 rotations one after the other; the batched schedule takes the same sums as hoisted sums
    of all their rotations (HELLM::rotateSumFused)."""
    H, orc, ev = small
    H.set_schedule(fused)
    try:
        _rotate_and_sum_reductions(H, orc, ev, fused)
    finally:
        H.set_schedule(True)


def _rotate_and_sum_reductions(H, orc, ev, fused):
    n = 16
    rng = np.random.default_rng(13)
    A, B = rng.normal(size=(n, n)), rng.normal(size=(n, n))
    x = H.encrypt2(A, B)
    ox = to_oracle(orc, x)
    scaled = np.zeros((n, n))
    scaled[:, 0] = 1.0 / (2 * n)
    got = x.clone()
    H.reduce_row_sum_with_scaled_mask(got, scaled, np.zeros((n, n)))
    want = R.reduce_row_sum_with_scaled_mask(ev, ox, R._message2(scaled, np.zeros((n, n)), orc.slots), 2 * n, fused)
    assert np.array_equal(got.residues(), want.data)
    d = H.decrypt2(got)
    mean = np.concatenate([A, B], axis=1).mean(axis=1, keepdims=True)
    assert np.abs(d[0] - mean).max() < 2 ** -20 and np.abs(d[1] - mean).max() < 2 ** -20
    a, b = x.clone(), x.clone()
    H.one_mat_rot_sum_inplace(a, b)
    wa, wb = R.one_mat_rot_sum(ev, ox, ox, n, fused)
    assert np.array_equal(a.residues(), wa.data) and np.array_equal(b.residues(), wb.data)
    assert np.abs(H.decrypt2(a)[1] - B[:, : n // 2].sum(axis=1, keepdims=True)).max() < 2 ** -18
    l, r = H.mask_right_left(x)
    wl, wr = R.mask_right_left(ev, ox, n)
    assert np.array_equal(l.residues(), wl.data) and np.array_equal(r.residues(), wr.data)
    assert np.abs(H.decrypt2(l)[0][:, : n // 2] - A[:, : n // 2]).max() < 2 ** -20
    assert np.abs(H.decrypt2(l)[0][:, n // 2:]).max() < 2 ** -20
    tiles = [H.encrypt2(rng.normal(size=(n, n)), rng.normal(size=(n, n))) for _ in range(3)]
    rows = np.concatenate([np.concatenate(H.decrypt2(t), axis=1) for t in tiles], axis=1)
    m, sq = H.row_moments(tiles, 1.0 / rows.shape[1])
    wm, wsq = R.row_moments(ev, [to_oracle(orc, t) for t in tiles], 1.0 / rows.shape[1], n, fused)
    assert np.array_equal(m.residues(), wm.data) and np.array_equal(sq.residues(), wsq.data)
    assert np.abs(H.decrypt2(m)[0] - rows.mean(axis=1, keepdims=True)).max() < 2 ** -18
    assert np.abs(H.decrypt2(sq)[1] - (rows ** 2).mean(axis=1, keepdims=True)).max() < 2 ** -16


def test_weight_and_ciphertext_stores(small, tmp_path):
    """encodeWeight / getWeight and the ciphertext store: what is read back is what was written."""
    H, orc, ev = small
    n = 16
    rng = np.random.default_rng(10)
    grid = rng.normal(0, 0.02, (6, 2, n, n))                 # 6 tile rows (one full group of 4 + a trailing pair) x 2
    H.encode_weight(grid, str(tmp_path / "w_"))
    for i, j, rows in ((0, 0, (0, 1, 2, 3)), (0, 1, (0, 1, 2, 3)), (1, 0, (4, 5, None, None))):
        w = [grid[r][j] if r is not None else np.zeros((n, n)) for r in rows]
        got = H.get_weight(str(tmp_path / ("w_%d_%d.msg" % (i, j))), 3)
        want = H.encode_diagonal_to_row4(*w, level=3)
        assert np.array_equal(got.residues(), want.residues())
    H.encode_weight(grid[:4, 0], str(tmp_path / "v_"))       # list of tiles -> pairs
    got = H.get_weight(str(tmp_path / "v_1.msg"), 2)
    assert np.array_equal(got.residues(), H.encode2(grid[2, 0], grid[3, 0], level=2).residues())
    with pytest.raises(pkg_error()):
        H.get_weight(str(tmp_path / "missing.msg"), 2)
    A, B = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    ct = H.level_down(H.encrypt2(A, B), 5)
    H.save_ct(ct, str(tmp_path / "ct.bin"))
    back = H.load_ct(str(tmp_path / "ct.bin"))
    assert back.info() == ct.info()
    assert np.array_equal(back.residues(), ct.residues())
    c = H.single_cc_matmul(back, H.encrypt2(B, A), 2)          # the loaded tensor keeps its tile shape
    d = H.decrypt2(c)
    assert np.abs(d[0] - A @ B).max() < 2 ** -18 and np.abs(d[1] - B @ A).max() < 2 ** -18


def test_error_behaviour(small):
    H, _, _ = small
    A = np.ones((16, 16))
    ca = H.encrypt(A)
    low = H.level_down(ca, 3)
    zero = H.level_down(ca, 0)
    with pytest.raises(ValueError):            # std::invalid_argument("[multMatMat] level >= 1 is needed.")
        H.single_cc_matmul(zero, zero, 2)
    with pytest.raises(pkg_error()):           # level < 4 + minimum bootstrap level: the reference would
        H.single_cc_matmul(low, low, 2)        # bootstrap here; this build raises instead
    mid = H.level_down(ca, 4)
    with pytest.raises(ValueError):            # enough to skip bootstrapping, too low for target level 2
        H.single_cc_matmul(mid, mid, 2)
    pa = H.encrypt2(A, A)
    with pytest.raises(ValueError):            # block widths differ
        H.single_cc_matmul(ca, pa, 2)
    with pytest.raises(pkg_error()):           # rescale / level errors surface as runtime errors
        H.level_down(low, 5)


def pkg_error():
    return load_package().HemmError


# ---- full size -----------------------------------------------------------------------------------
@pytest.mark.parametrize("fused", [True, False], ids=["batched", "reference-order"])
def test_full_ccmm_128(full, fused):
    H = full
    H.set_schedule(fused)
    rng = np.random.default_rng(1)
    A, B = rng.uniform(-1, 1, (128, 128)), rng.uniform(-1, 1, (128, 128))
    ca, cb = H.encrypt(A), H.encrypt(B)
    assert ca.info()["level"] == 12
    c = H.single_cc_matmul(ca, cb, 4)
    assert c.info()["level"] == 4
    err = np.abs(H.decrypt(c) - A @ B).max()
    assert err < TOL, err
    z = H.decrypt_slots(c)
    assert np.abs(z[128 * 128:]).max() < TOL           # upper half of the slots stays empty
    # linearity in the encrypted operand: (2A) B = 2 (A B)
    c2 = H.single_cc_matmul(H.add(ca, ca), cb, 4)
    H.set_schedule(True)
    assert np.abs(H.decrypt(c2) - 2 * (A @ B)).max() < TOL


def test_full_ccmm_batch_sizes_give_the_same_residues(full):
    """The batch size only decides how the shifts are cut into launch chains (two concurrent chains of kernel-argument
    term lists at the default 16; one chain with a staged term list at 32; four chains one after the other at 8): every
    residue of the product is the same."""
    H = full
    rng = np.random.default_rng(5)
    A, B = rng.uniform(-1, 1, (128, 128)), rng.uniform(-1, 1, (128, 128))
    ca, cb = H.encrypt(A), H.encrypt(B)
    ref = None
    try:
        for batch in (16, 32, 8):
            H.set_schedule(True, batch=batch)
            c = H.single_cc_matmul(ca, cb, 4)
            r = c.residues()
            if ref is None:
                ref = r
                assert np.abs(H.decrypt(c) - A @ B).max() < TOL
            else:
                assert np.array_equal(r, ref), batch
    finally:
        H.set_schedule(True)


def test_full_pcmm_packed_and_hoisted(full):
    H = full
    rng = np.random.default_rng(2)
    A, B = rng.uniform(-1, 1, (128, 128)), rng.uniform(-1, 1, (128, 128))
    A2, B2 = rng.uniform(-1, 1, (128, 128)), rng.uniform(-1, 1, (128, 128))
    c = H.single_matmul(H.encrypt(A), H.encode(B), 4)
    assert np.abs(H.decrypt(c) - A @ B).max() < TOL
    pa, pb = H.encrypt2(A, A2), H.encrypt2(B, B2)
    H.complex_packing_inplace(pa)
    H.complex_packing_row_inplace(pb)
    d = H.decrypt2(H.repack_cc(H.packed_matmul(pa, pb, 4)))
    assert np.abs(d[0] - A @ B).max() < TOL and np.abs(d[1] - A2 @ B2).max() < TOL
    W = [rng.normal(0, 0.02, (128, 128)) for _ in range(4)]
    X0, X1 = 0.1 * rng.normal(size=(128, 128)), 0.1 * rng.normal(size=(128, 128))
    x = H.complex_packing(H.encrypt2(X0, X0), H.encrypt2(X1, X1))
    tmp = H.matmul_pre(x, 4)
    y = H.matmul_reuse(tmp, H.encode_diagonal_to_row4(*W, level=5), 4)
    z = H.decrypt2(H.repack_cc(y))
    assert np.abs(z[0] - (X0 @ W[0] + X1 @ W[2])).max() < 2 ** -10
    assert np.abs(z[1] - (X0 @ W[1] + X1 @ W[3])).max() < 2 ** -10
    t = H.encrypt2(A, A2)
    H.transpose_inplace(t)
    d = H.decrypt2(t)
    assert np.abs(d[0] - A.T).max() < TOL and np.abs(d[1] - A2.T).max() < TOL


def test_two_parameter_sets_take_turns(small):
    """Two HEMMers over different prime chains with the same tile shape, used in turn: the mask caches behind the
    products belong to one parameter set at a time (masks are keyed by kind, shape and level, all of which the two sets
    share), so each product must still give the residues of its own oracle."""
    from efla_amd import hellm
    H1, orc1, _ = small
    qs, ps = O.ckks_chain(10, 9, 3)
    assert len(qs) == len(orc1.q) + 1
    H2 = hellm.HEMMer(10, qs, ps, dnum=3, min_bootstrap_level=0, seed=9)
    orc2 = O.Oracle(10, qs, ps, dnum=3)
    gen_oracle_keys(orc2, 9, H2.dim)
    rng = np.random.default_rng(77)
    A, B = rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
    for H, orc in ((H1, orc1), (H2, orc2), (H1, orc1), (H2, orc2)):
        ca, cb = H.encrypt(A), H.encrypt(B)
        a = H.level_down(ca, 6) if ca.info()["level"] > 6 else ca
        b = H.level_down(cb, 6) if cb.info()["level"] > 6 else cb
        c = H.single_cc_matmul(a, b, 2)
        want = R.mult_mat_mat_cc_packed_single(orc, to_oracle(orc, a), to_oracle(orc, b), 2, 16, 16)
        assert np.array_equal(c.residues(), want.data)
        assert np.abs(H.decrypt(c) - A @ B).max() < 2 ** -18
        w = H.encode(B)
        p = H.single_matmul(ca, w, 2)
        assert np.abs(H.decrypt(p) - A @ B).max() < 2 ** -18
