"""Pins the restated HEMMer algorithms (oracle/hemmer_ref.py) on exact slot vectors: every mask and
rotation index must reproduce float64 matrix algebra, at the reference's 128 x 128 / 2^15-slot shape
and on a small tile.  No cryptography involved."""
import numpy as np
import pytest

from oracle import hemmer_ref as R


def setup(n, top=12):
    slots = 2 * n * n
    ev = R.SlotSim(slots.bit_length() - 1, top)
    rng = np.random.default_rng(n)
    return ev, rng


def single(ev, M, n):
    return ev.encrypt(M.reshape(-1))


def pair(ev, M1, M2):
    return ev.encrypt(np.concatenate([M1, M2], axis=1).reshape(-1))


@pytest.mark.parametrize("n", [8, 128])
def test_sigma_tau_transpose(n):
    ev, rng = setup(n)
    A = rng.uniform(-1, 1, (n, n))
    i, j = np.meshgrid(np.arange(n), np.arange(n), indexing="ij")
    for w, enc in ((n, lambda M: single(ev, M, n)), (2 * n, lambda M: pair(ev, M, 2 * M))):
        s = R.diagonal_transform(ev, enc(A), R.H, n, w)
        got = ev.decrypt(s).real.reshape(-1, w)[:n, :n]
        assert np.array_equal(got, A[i, (i + j) % n]) and s.level == 11 and s.rc == 0
        t = R.diagonal_transform(ev, enc(A), R.V, n, w)
        assert np.array_equal(ev.decrypt(t).real.reshape(-1, w)[:n, :n], A[(i + j) % n, j])
        tr = R.transpose(ev, enc(A), n, w)
        assert np.array_equal(ev.decrypt(tr).real.reshape(-1, w)[:n, :n], A.T)
        # the same diagonals in sigma / tau's grouping (what the batched transform walks)
        ts = R.diagonal_transform(ev, enc(A), R.DIAG_SIGNED, n, w)
        assert np.array_equal(ev.decrypt(ts).real.reshape(-1, w), ev.decrypt(tr).real.reshape(-1, w))
        if w == 2 * n:   # the second tile of the pair is transformed independently
            assert np.array_equal(ev.decrypt(tr).real.reshape(-1, w)[:n, n:], 2 * A.T)


@pytest.mark.parametrize("n", [8, 128])
def test_ccmm_single_and_pair_layout(n):
    ev, rng = setup(n)
    A, B = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    c = R.mult_mat_mat_cc(ev, single(ev, A, n), single(ev, B, n), 4, n, n)
    z = ev.decrypt(c)
    assert c.level == 4 and c.rc == 0
    assert np.abs(z[: n * n].real.reshape(n, n) - A @ B).max() < 1e-12
    assert np.abs(z[n * n:]).max() == 0           # upper half of the slots stays empty
    A2, B2 = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    c = R.mult_mat_mat_cc(ev, pair(ev, A, A2), pair(ev, B, B2), 4, n, 2 * n)
    z = ev.decrypt(c).real.reshape(n, 2 * n)
    assert np.abs(z[:, :n] - A @ B).max() < 1e-12 and np.abs(z[:, n:] - A2 @ B2).max() < 1e-12


@pytest.mark.parametrize("n", [8, 128])
def test_pcmm_unhoisted(n):
    ev, rng = setup(n)
    A, B = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    bp = ev.encode(single(ev, B, n).z, 12)
    c = R.mult_mat_mat_pc(ev, single(ev, A, n), bp, 4, n, n)
    assert np.abs(ev.decrypt(c)[: n * n].real.reshape(n, n) - A @ B).max() < 1e-12


@pytest.mark.parametrize("n", [8, 128])
def test_packed_ccmm_two_products_per_call(n):
    ev, rng = setup(n)
    A1, A2, B1, B2 = (rng.uniform(-1, 1, (n, n)) for _ in range(4))
    a = R.complex_packing_cols(ev, pair(ev, A1, A2), n, 2 * n)
    b = R.complex_packing_rows(ev, pair(ev, B1, B2), n, 2 * n)
    # packing: both slots of a column pair hold a + i b; both rows of a row pair hold a - i b
    za = ev.decrypt(a).reshape(n, 2 * n)
    assert np.allclose(za[:, 0:n:2], A1[:, 0::2] + 1j * A1[:, 1::2]) and np.allclose(za[:, 0:n:2], za[:, 1:n:2])
    zb = ev.decrypt(b).reshape(n, 2 * n)
    assert np.allclose(zb[0::2, :n], B1[0::2] - 1j * B1[1::2]) and np.allclose(zb[0::2], zb[1::2])
    c = R.repack_cc(ev, R.mult_packed_mat_mat(ev, a, b, 4, n, 2 * n))
    z = ev.decrypt(c).reshape(n, 2 * n)
    assert np.abs(z.imag).max() < 1e-12
    assert np.abs(z.real[:, :n] - A1 @ B1).max() < 1e-12 and np.abs(z.real[:, n:] - A2 @ B2).max() < 1e-12
    assert c.level == 4


@pytest.mark.parametrize("n", [8, 128])
def test_hoisted_plaintext_product(n):
    """complexPacking(x0, x1) -> matMulPre -> matMulReUse(encodeDiagonalToRow4(W..)) gives
    Re = X0 W1 + X1 W3 (left) | X0 W2 + X1 W4 (right) after x + conj(x)."""
    ev, rng = setup(n)
    X0, X1 = rng.uniform(-1, 1, (n, n)), rng.uniform(-1, 1, (n, n))
    W = [rng.normal(0, 0.02, (n, n)) for _ in range(4)]
    x0 = pair(ev, X0, X0)
    x1 = pair(ev, X1, X1)
    x = ev.add(x0, ev.mult_imag_unit(x1))                     # HEMMer::complexPacking(ct, ct)
    tmp = R.mult_mat_mat_pre(ev, x, 4, n, 2 * n)
    assert len(tmp) == n and all(t.level == 5 for t in tmp)
    wp = ev.encode(R.weights_diagonal_to_row4(*W, ev.slots), 5)
    y = R.mult_mat_mat_reuse(ev, tmp, wp, 4)
    z = ev.decrypt(R.repack_cc(ev, y)).real.reshape(n, 2 * n)
    assert y.level == 4
    assert np.abs(z[:, :n] - (X0 @ W[0] + X1 @ W[2])).max() < 1e-12
    assert np.abs(z[:, n:] - (X0 @ W[1] + X1 @ W[3])).max() < 1e-12


def test_assemble_masks_are_complementary():
    n, slots = 8, 128
    cm, rm = R.col_masks(n, slots), R.row_masks(n, n, slots)
    for i in range(n):
        assert np.array_equal(cm[2 * i] + cm[2 * i + 1], np.ones(slots))
        assert np.array_equal(rm[2 * i] + rm[2 * i + 1], np.ones(slots))
        assert cm[2 * i].sum() == i * slots // n and rm[2 * i].sum() == i * slots // n


@pytest.mark.parametrize("hoisted", [False, True], ids=["log-steps", "hoisted-sums"])
def test_rotate_and_sum_reductions(hoisted):
    """Row reductions on the pair layout against numpy (exact slot arithmetic), in the reference's order (log2 steps)
    and as the sums of all rotations the batched schedule takes."""
    n = 8
    ev = R.SlotSim(7, 12)                     # 2 n^2 = 128 slots
    rng = np.random.default_rng(5)
    A, B = rng.normal(size=(n, n)), rng.normal(size=(n, n))
    x = ev.encrypt(R._message2(A, B, ev.slots))
    scaled = np.zeros((n, n))
    scaled[:, 0] = 1.0 / (2 * n)
    out = R.reduce_row_sum_with_scaled_mask(ev, x, R._message2(scaled, np.zeros((n, n)), ev.slots), 2 * n, hoisted)
    z = ev.decrypt(out).real.reshape(n, 2 * n)
    want = np.concatenate([A, B], axis=1).mean(axis=1, keepdims=True)
    assert np.abs(z - want).max() < 1e-12       # every slot of a row holds the row mean over both halves
    a, b = R.one_mat_rot_sum(ev, x, x, n, hoisted)
    za, zb = ev.decrypt(a).real.reshape(n, 2 * n), ev.decrypt(b).real.reshape(n, 2 * n)
    # a: sums of the first half of each tile row, spread over the tile row; b: sums of the second half
    assert np.abs(za[:, :n] - A[:, : n // 2].sum(axis=1, keepdims=True)).max() < 1e-12
    assert np.abs(za[:, n:] - B[:, : n // 2].sum(axis=1, keepdims=True)).max() < 1e-12
    assert np.abs(zb[:, :n] - A[:, n // 2:].sum(axis=1, keepdims=True)).max() < 1e-12
    assert np.abs(zb[:, n:] - B[:, n // 2:].sum(axis=1, keepdims=True)).max() < 1e-12
    tiles = [ev.encrypt(R._message2(rng.normal(size=(n, n)), rng.normal(size=(n, n)), ev.slots)) for _ in range(3)]
    rows = np.concatenate([ev.decrypt(t).real.reshape(n, 2 * n) for t in tiles], axis=1)
    mean, sq = R.row_moments(ev, tiles, 1.0 / rows.shape[1], n, hoisted)
    assert np.abs(ev.decrypt(mean).real.reshape(n, 2 * n) - rows.mean(axis=1, keepdims=True)).max() < 1e-12
    assert np.abs(ev.decrypt(sq).real.reshape(n, 2 * n) - (rows ** 2).mean(axis=1, keepdims=True)).max() < 1e-12


@pytest.mark.parametrize("n,w,log_slots", [(8, 16, 7), (8, 8, 7), (16, 32, 9)])
def test_two_stage_transform_masks(n, w, log_slots):
    """The two-stage sigma / tau (rows rotated by i mod b, then by b (i div b)) built from its masks and plain
    rotations equals the one-stage transform of the reference for all four kinds."""
    sim = R.SlotSim(log_slots, 12)
    rng = np.random.default_rng(n * w)
    x0 = rng.normal(size=sim.slots) + 1j * rng.normal(size=sim.slots)
    rot = lambda v, r: np.roll(v, -r)
    for kind in (R.H, R.V, R.PH, R.PV):
        cell = 2 if kind in (R.PH, R.PV) else 1
        u = n // cell
        b = R.two_stage_split(u)
        step = cell * (w if kind in (R.V, R.PV) else 1)
        wrap = n * (w if kind in (R.V, R.PV) else 1)
        x = x0
        for stage, count, mul in ((1, b, 1), (2, u // b, b)):
            x2 = rot(x, -wrap)
            y = R.two_stage_mask(kind, n, w, sim.slots, stage, 0, 0) * x
            for r in range(1, count):
                y = y + R.two_stage_mask(kind, n, w, sim.slots, stage, r, 1) * rot(x, r * mul * step)
                y = y + R.two_stage_mask(kind, n, w, sim.slots, stage, r, 2) * rot(x2, r * mul * step)
            x = y
        want = R.diagonal_transform(sim, sim.encrypt(x0), kind, n, w).z
        assert np.abs(x - want).max() < 1e-12, kind


@pytest.mark.parametrize("n,w,log_slots", [(8, 16, 7), (8, 8, 7), (16, 32, 9), (16, 16, 9)])
def test_composite_packing_transform_masks(n, w, log_slots):
    """The complex packing followed by the packed sigma / tau as ONE one-stage transform (kinds PKH / PKV, diagonals
    over single columns / rows): equal to the packing and then the packed transform on arbitrary slot vectors,
    stacked tile blocks included."""
    sim = R.SlotSim(log_slots, 12)
    rng = np.random.default_rng(n + w)
    x0 = rng.normal(size=sim.slots) + 1j * rng.normal(size=sim.slots)
    for merged, packed, pack in ((R.PKH, R.PH, R.complex_packing_cols), (R.PKV, R.PV, R.complex_packing_rows)):
        two_steps = R.diagonal_transform(sim, pack(sim, sim.encrypt(x0), n, w), packed, n, w)
        one_step = R.diagonal_transform(sim, sim.encrypt(x0), merged, n, w)
        assert np.abs(one_step.z - two_steps.z).max() < 1e-12, merged
        assert sim.level_of(one_step) == sim.level_of(two_steps) + 1      # one level instead of two


@pytest.mark.parametrize("n,w,log_slots", [(8, 16, 7), (8, 8, 7), (16, 32, 9), (16, 16, 9)])
def test_packing_and_first_stage_as_one_map(n, w, log_slots):
    """packing_stage_one_maps: sum_a mask_a (.) rho^a(x) equals the complex packing followed by the first stage of
    the two-stage packed transform, and the second stage then completes the packed transform of the packed operand
    (arbitrary slot vectors; tiles that fill the slot vector, where main and wrapped rotations coincide, and tiles
    that leave other blocks)."""
    sim = R.SlotSim(log_slots, 12)
    rng = np.random.default_rng(3 * n + w)
    x0 = rng.normal(size=sim.slots) + 1j * rng.normal(size=sim.slots)
    rot = lambda v, r: np.roll(v, -r)
    for kind, pack in ((R.PH, R.complex_packing_cols), (R.PV, R.complex_packing_rows)):
        maps = R.packing_stage_one_maps(kind, n, w, sim.slots)
        assert len({a for a, _ in maps}) == len(maps) and all(0 <= a < sim.slots for a, _ in maps)
        x = sum(m * rot(x0, a) for a, m in maps)
        # the second stage alone (its masks and rotations as in the two-stage transform)
        u = n // 2
        b = R.two_stage_split(u)
        step = 2 * (w if kind == R.PV else 1)
        wrap = n * (w if kind == R.PV else 1)
        y = R.two_stage_mask(kind, n, w, sim.slots, 2, 0, 0) * x
        for r in range(1, u // b):
            y = y + R.two_stage_mask(kind, n, w, sim.slots, 2, r, 1) * rot(x, r * b * step)
            y = y + R.two_stage_mask(kind, n, w, sim.slots, 2, r, 2) * rot(x, r * b * step - wrap)
        want = R.diagonal_transform(sim, pack(sim, sim.encrypt(x0), n, w), kind, n, w).z
        assert np.abs(y - want).max() < 1e-12, kind


def test_composite_packed_ccmm_three_levels_above_the_target():
    """A whole product through the composite transform on the slot simulator: operands three levels above the target,
    single tile and stacked tiles."""
    n = 8
    sim = R.SlotSim(7, 12)
    rng = np.random.default_rng(3)
    A, B = rng.uniform(-1, 1, (2 * n, n)), rng.uniform(-1, 1, (2 * n, n))
    a, b = sim.encrypt(A.reshape(-1), 5), sim.encrypt(B.reshape(-1), 5)
    for kind, unit in ((R.PKH, 1), (R.PKV, n)):
        assert R.geometry(kind, n, n)[4] == unit
    pa = R.diagonal_transform(sim, a, R.PKH, n, n)
    pb = R.diagonal_transform(sim, b, R.PKV, n, n)
    want_a = R.diagonal_transform(sim, R.complex_packing_cols(sim, a, n, n), R.PH, n, n)
    want_b = R.diagonal_transform(sim, R.complex_packing_rows(sim, b, n, n), R.PV, n, n)
    assert np.abs(pa.z - want_a.z).max() < 1e-12 and np.abs(pb.z - want_b.z).max() < 1e-12
