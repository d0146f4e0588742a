"""Index logic of the LoRA low-rank path on exact slot vectors (no encryption): the restatement of the
reference's multMatMatHighLow / LowHigh / LowLow, getLow*Block and repackTo* (oracle/hemmer_ref.py) must
reproduce the matrix products it is used for, in the layouts its callers rely on
(reference src/TransformerBlock.cpp:1785-1835 forward, :8399-8410, :8573-8583, :8641-8653 gradients).
Also the rectangular sigma / tau transforms those products run, against their index formulas."""
import numpy as np
import pytest

from oracle import hemmer_ref as R

N_TILE, W, LD, LOG_SLOTS = 8, 16, 2, 7


@pytest.fixture()
def sim():
    return R.SlotSim(LOG_SLOTS, 12)


def tile2(sim, a, b):
    return R._message2(a, b, sim.slots)


def halves(z):
    m = np.real(z).reshape(N_TILE, W)
    return m[:, :N_TILE], m[:, N_TILE:]


@pytest.mark.parametrize("rows,cols", [(8, 2), (2, 8), (8, 4), (4, 8), (8, 8)])
def test_rectangular_sigma_tau(sim, rows, cols):
    """sigma(A)[i, j] = A[i, (i + j) mod cols] on the first min(rows, cols) rows of every row group;
    tau(B)[i, j] = B[(i + j) mod rows, j] likewise on columns (MatrixUtils.cpp:776-848, 924-996)."""
    rng = np.random.default_rng(rows * 16 + cols)
    sub = min(rows, cols)
    M = rng.normal(size=(sim.slots // W, W))
    x = sim.encrypt(M.reshape(-1))
    s = R.diagonal_transform(sim, x, R.H, (rows, cols), W).z.real.reshape(-1, W)
    t = R.diagonal_transform(sim, x, R.V, (rows, cols), W).z.real.reshape(-1, W)
    r, c = np.meshgrid(np.arange(M.shape[0]), np.arange(W), indexing="ij")
    cb, j = c - c % cols, c % cols
    rb, i = r - r % rows, r % rows
    assert np.abs(s - M[r, cb + (j + i % sub) % cols]).max() < 1e-12
    assert np.abs(t - M[rb + (i + j % sub) % rows, c]).max() < 1e-12


def test_lora_forward_chain(sim):
    """x (n x 4n, two pair-layout tiles) times A (4n x 2) times B (2 x 4n): sum of HighLow partial products,
    repackToOneCol, then one LowLow per output tile."""
    n, w, ld = N_TILE, W, LD
    rng = np.random.default_rng(0)
    m = 2
    Xs = [(rng.normal(size=(n, n)), rng.normal(size=(n, n))) for _ in range(m)]
    A = rng.normal(size=(2 * m * n, ld))
    W0, W1 = rng.normal(size=(n, n)), rng.normal(size=(n, n))      # other column blocks hold other data
    for i in range(m):
        W0[:, i * ld:(i + 1) * ld] = A[(2 * i) * n:(2 * i + 1) * n]
        W1[:, i * ld:(i + 1) * ld] = A[(2 * i + 1) * n:(2 * i + 2) * n]
    wa = sim.encrypt(tile2(sim, W0, W1))
    acc = None
    for i in range(m):
        x = sim.encrypt(tile2(sim, *Xs[i]))
        low = R.get_low_col_block(sim, wa, i, n, n, w, ld)
        r = R.mult_mat_mat_high_low(sim, x, low, i, 5, (n, n), (n, n), w, ld)
        assert r.level == 5
        acc = r if acc is None else sim.add(acc, r)
    XA = sum(Xs[i][0] @ A[(2 * i) * n:(2 * i + 1) * n] + Xs[i][1] @ A[(2 * i + 1) * n:(2 * i + 2) * n]
             for i in range(m))
    one = R.repack_to_one_col(sim, acc, 0, n, n, w, ld)
    left, right = halves(one.z)
    assert np.abs(left[:, :ld] - XA).max() < 1e-12 and np.abs(right[:, :ld] - XA).max() < 1e-12
    assert np.abs(left[:, ld:]).max() == 0 and np.abs(right[:, ld:]).max() == 0
    one = sim.encrypt(one.z)                       # the reference bootstraps here
    B = rng.normal(size=(ld, 2 * m * n))
    V0, V1 = rng.normal(size=(n, n)), rng.normal(size=(n, n))
    for i in range(m):
        V0[i * ld:(i + 1) * ld] = B[:, (2 * i) * n:(2 * i + 1) * n]
        V1[i * ld:(i + 1) * ld] = B[:, (2 * i + 1) * n:(2 * i + 2) * n]
    wb = sim.encrypt(tile2(sim, V0, V1))
    want = XA @ B
    for i in range(m):
        o = R.mult_mat_mat_low_low(sim, one, R.get_low_row_block(sim, wb, i, n, w, ld), 0, i, 4, (n, n), (n, n), w, ld)
        left, right = halves(o.z)
        assert o.level == 4
        assert np.abs(left - want[:, (2 * i) * n:(2 * i + 1) * n]).max() < 1e-12
        assert np.abs(right - want[:, (2 * i + 1) * n:(2 * i + 2) * n]).max() < 1e-12


@pytest.mark.parametrize("blk", [0, 1, 2, 3])
def test_lora_gradient_products(sim, blk):
    n, w, ld = N_TILE, W, LD
    rng = np.random.default_rng(10 + blk)
    Lw = rng.normal(size=(ld, n))                  # thin left operand in row block 0 of both tiles
    T0 = np.zeros((n, n))
    T0[:ld] = Lw
    G0, G1 = rng.normal(size=(n, n)), rng.normal(size=(n, n))
    a, g = sim.encrypt(tile2(sim, T0, T0)), sim.encrypt(tile2(sim, G0, G1))
    prod = R.mult_mat_mat_low_high(sim, a, g, 0, 5, (n, n), (n, n), w, ld)
    left, right = halves(R.repack_to_multi_row(sim, prod, blk, n, w, ld).z)
    want0, want1 = np.zeros((n, n)), np.zeros((n, n))
    want0[blk * ld:(blk + 1) * ld], want1[blk * ld:(blk + 1) * ld] = Lw @ G0, Lw @ G1
    assert np.abs(left - want0).max() < 1e-12 and np.abs(right - want1).max() < 1e-12
    left, right = halves(R.repack_to_one_row(sim, prod, blk, n, n, w, ld).z)
    want = np.zeros((n, n))
    want[blk * ld:(blk + 1) * ld] = Lw @ G0 + Lw @ G1
    assert np.abs(left - want).max() < 1e-12 and np.abs(right - want).max() < 1e-12
    # thin right operand in column block 0, result moved to column block blk
    X0, X1 = rng.normal(size=(n, n)), rng.normal(size=(n, n))
    gb = rng.normal(size=(n, ld))
    Gt = np.zeros((n, n))
    Gt[:, :ld] = gb
    prod = R.mult_mat_mat_high_low(sim, sim.encrypt(tile2(sim, X0, X1)), sim.encrypt(tile2(sim, Gt, Gt)), 0, 5,
                                   (n, n), (n, n), w, ld)
    left, right = halves(R.repack_to_multi_col(sim, prod, blk, n, n, w, ld).z)
    want0, want1 = np.zeros((n, n)), np.zeros((n, n))
    want0[:, blk * ld:(blk + 1) * ld], want1[:, blk * ld:(blk + 1) * ld] = X0 @ gb, X1 @ gb
    assert np.abs(left - want0).max() < 1e-12 and np.abs(right - want1).max() < 1e-12


def test_repack_lora_opti_closed_form(sim):
    """With s1 = 2 Re(t1), s2 = 2 Re(t2) and L/R the left/right tiles: the left tile of the result is
    s1_L + s1_R and the right tile s2_R + 0.5 s2_L + 0.5 i s1_L (worked out by hand from HEMMer.cpp:1055-1091)."""
    n = N_TILE
    rng = np.random.default_rng(5)
    t = [rng.normal(size=(4, n, n)) + 1j * rng.normal(size=(4, n, n)) for _ in range(2)]
    t1 = R.SimCt(tile2(sim, t[0][0], t[0][1]), 5, rc=1)
    t2 = R.SimCt(tile2(sim, t[1][0], t[1][1]), 5, rc=1)
    out = R.repack_lora_opti(sim, t1, t2, n).z.reshape(n, W)
    s1L, s1R, s2L, s2R = 2 * t[0][0].real, 2 * t[0][1].real, 2 * t[1][0].real, 2 * t[1][1].real
    assert np.abs(out[:, :n] - (s1L + s1R)).max() < 1e-12
    assert np.abs(out[:, n:] - (s2R + 0.5 * s2L + 0.5j * s1L)).max() < 1e-12


def test_repack_not_bts_and_split_in_two_closed_forms(sim):
    """repack_notBTS (HEMMer.cpp:1025-1053): with o = 2 Re(t1) + 2i Re(t2) and L / R its left and right tiles the result
    is [o_L + o_R | o_R]; splitInTwo (HEMMer.cpp:819-831): [A | B] -> [A | A] and [B | B].  Worked out by hand from the
    reference's rotations and masks."""
    n = N_TILE
    rng = np.random.default_rng(6)
    t = [rng.normal(size=(2, n, n)) + 1j * rng.normal(size=(2, n, n)) for _ in range(2)]
    t1 = R.SimCt(tile2(sim, t[0][0], t[0][1]), 5, rc=1)
    t2 = R.SimCt(tile2(sim, t[1][0], t[1][1]), 5, rc=1)
    out = R.repack_not_bts(sim, t1, t2, n).z.reshape(n, W)
    oL, oR = 2 * t[0][0].real + 2j * t[1][0].real, 2 * t[0][1].real + 2j * t[1][1].real
    assert np.abs(out[:, :n] - (oL + oR)).max() < 1e-12 and np.abs(out[:, n:] - oR).max() < 1e-12
    A, B = rng.normal(size=(n, n)), rng.normal(size=(n, n))
    a, b = R.split_in_two(sim, sim.encrypt(tile2(sim, A, B)), n)
    for got, want in ((a, A), (b, B)):
        left, right = halves(got.z)
        assert np.abs(left - want).max() < 1e-12 and np.abs(right - want).max() < 1e-12


@pytest.mark.parametrize("hoisted", [False, True], ids=["log-steps", "hoisted-sums"])
def test_lora_rank2_elementwise_path(sim, hoisted):
    """The production rank-2 form (element-wise products and rotate-and-sum, TransformerBlock.cpp:2199-2365):
    X (n x 6n, three pair-layout tiles) times A (6n x 2) gives two column ciphertexts, then times B (2 x 6n)."""
    n, w, m = N_TILE, W, 3
    rng = np.random.default_rng(31)
    X = rng.normal(size=(n, 2 * n * m))
    A = rng.normal(size=(2 * n * m, 2))
    B = rng.normal(size=(2, 2 * n * m))
    wa, wb = rng.normal(size=(n, w)), rng.normal(size=(n, w))     # unused rows hold other data
    for i in range(m):
        for j in range(2):
            wa[2 * i + j] = A[2 * n * i:2 * n * (i + 1), j]
            wb[2 * i + j] = B[j, 2 * n * i:2 * n * (i + 1)]
    cur = [sim.encrypt(X[:, 2 * n * i:2 * n * (i + 1)].reshape(-1)) for i in range(m)]
    xa = R.lora_rank2_down(sim, cur, sim.encrypt(wa.reshape(-1)), n, w, 9, hoisted)
    for j in range(2):
        z = xa[j].z.real.reshape(n, w)
        assert np.abs(z[:, 0] - X @ A[:, j]).max() < 1e-12 and np.abs(z[:, 1:]).max() == 0
        assert xa[j].level == 6                    # 9 -> mask 8 -> product 7 -> mask 6
    out = R.lora_rank2_up(sim, xa, sim.encrypt(wb.reshape(-1)), m, n, w, 6, hoisted)
    want = X @ A @ B
    for i in range(m):
        assert np.abs(out[i].z.real.reshape(n, w) - want[:, 2 * n * i:2 * n * (i + 1)]).max() < 1e-12
        assert out[i].level == 4
