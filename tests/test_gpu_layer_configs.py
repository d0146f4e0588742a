"""End-to-end compositions of the hot path at the shapes of the reference's layer-level workloads, full ring
(N = 2^16, 128 x 128 tiles), checked against float64 algebra:

  * LoRA forward projection: X (128 x 768, six activation tiles) times a plaintext 768 x 768 weight through
    the hoisted PCMM path (matMulPre once per activation tile pair, matMulReUse per weight tile group), plus
    the rank-8 update X A B with A (768 x 8) and B (8 x 768) zero-padded to 128-wide encrypted tiles
    (two chained CCMMs);
  * the same rank-2 update through the low-rank path the reference's LoRA layers use (matMulHighLow per
    activation pair, repackToOneCol, matMulLowLow per output pair; src/TransformerBlock.cpp:1785-1835);
  * attention heads with the Gaussian-kernel score of the reference's layer: norms by squaring and rotate-and-sum,
    -2 Q K^T + |q|^2 + |k|^2 (CCMM), a degree-15 Chebyshev table of exp(-x / 16), then scores x V (CCMM).
"""
import numpy as np
import pytest

from __graft_entry__ import load_package

pytestmark = pytest.mark.gpu
TOL = 2.0 ** -10


@pytest.fixture(scope="module")
def H():
    load_package()
    from efla_amd import hellm
    return hellm.HEMMer(preset=True, seed=3)


def test_lora_forward_projection(H):
    rng = np.random.default_rng(11)
    n, tiles, rank = 128, 6, 8
    X = 0.1 * rng.normal(size=(n, n * tiles))
    W = 0.02 * rng.normal(size=(n * tiles, n * tiles))
    A = 0.02 * rng.normal(size=(n * tiles, rank))
    B = 0.02 * rng.normal(size=(rank, n * tiles))
    xt = [X[:, i * n:(i + 1) * n] for i in range(tiles)]
    # --- frozen weight: complex-packed pairs of activation tiles, hoisted shifts reused over all weight columns
    T = 4
    pre = []
    for i in range(0, tiles, 2):
        x = H.complex_packing(H.encrypt2(xt[i], xt[i]), H.encrypt2(xt[i + 1], xt[i + 1]))
        pre.append(H.matmul_pre(x, T))
    Y = np.zeros((n, n * tiles))
    for j in range(0, 2, 2):               # two of the six output tile columns (the others repeat the same calls)
        acc = None
        for p, i in enumerate(range(0, tiles, 2)):
            w = [W[r * n:(r + 1) * n, c * n:(c + 1) * n] for r in (i, i + 1) for c in (j, j + 1)]
            # msgDiagonalToRow4 takes (W1, W2, W3, W4) with result columns X0 W1 + X1 W3 | X0 W2 + X1 W4
            wp = H.encode_diagonal_to_row4(w[0], w[1], w[2], w[3], level=T + 1)
            y = H.matmul_reuse(pre[p], wp, T)
            acc = y if acc is None else H.add(acc, y)
        z = H.decrypt2(H.repack_cc(acc))
        want = X @ W[:, j * n:(j + 2) * n]
        assert np.abs(z[0] - want[:, :n]).max() < TOL
        assert np.abs(z[1] - want[:, n:]).max() < TOL
    # --- low-rank update with zero-padded encrypted factors: (X A) at level 7, then (X A) B at level 4
    xa = None
    cx = [H.encrypt(t) for t in xt]
    for i in range(tiles):
        Ai = np.zeros((n, n))
        Ai[:, :rank] = A[i * n:(i + 1) * n]
        t = H.single_cc_matmul(cx[i], H.encrypt(Ai), 7)
        xa = t if xa is None else H.add(xa, t)
    assert xa.info()["level"] == 7
    Bj = np.zeros((n, n))
    Bj[:rank] = B[:, :n]
    xab = H.single_cc_matmul(xa, H.encrypt(Bj), 4)
    assert np.abs(H.decrypt(xab) - (X @ A @ B)[:, :n]).max() < TOL


def test_lora_low_rank_path(H):
    """X (128 x 768 as three pair-layout ciphertexts) times A (768 x 2) times B (2 x 768), both factors encrypted
    in the block layout of the LoRA weights: tile t of A sits in column block t // 2 of the left (even t) or
    right (odd t) half, tile t of B likewise in row block t // 2.  The reference refreshes X A by bootstrapping
    between the two products; here the second product simply runs at the levels that are left."""
    rng = np.random.default_rng(13)
    n, tiles, rank = 128, 6, 2
    X = 0.1 * rng.normal(size=(n, n * tiles))
    A = 0.1 * rng.normal(size=(n * tiles, rank))
    B = 0.1 * rng.normal(size=(rank, n * tiles))
    wa = [np.zeros((n, n)), np.zeros((n, n))]
    wb = [np.zeros((n, n)), np.zeros((n, n))]
    for t in range(tiles):
        wa[t % 2][:, (t // 2) * rank:(t // 2 + 1) * rank] = A[t * n:(t + 1) * n]
        wb[t % 2][(t // 2) * rank:(t // 2 + 1) * rank] = B[:, t * n:(t + 1) * n]
    cwa, cwb = H.encrypt2(*wa), H.encrypt2(*wb)
    xa = None
    for i in range(tiles // 2):
        cx = H.encrypt2(X[:, 2 * i * n:(2 * i + 1) * n], X[:, (2 * i + 1) * n:(2 * i + 2) * n])
        t = H.matmul_high_low(cx, H.get_low_col_block(cwa, i), i, 5)
        xa = t if xa is None else H.add(xa, t)
    xa = H.repack_to_one_col(xa, 0)
    assert xa.info()["level"] == 4
    d = H.decrypt2(xa)
    assert np.abs(d[0][:, :rank] - X @ A).max() < TOL and np.abs(d[1][:, :rank] - X @ A).max() < TOL
    want = X @ A @ B
    for i in range(tiles // 2):
        y = H.matmul_low_low(xa, H.get_low_row_block(cwb, i), 0, i, 1)
        d = H.decrypt2(y)
        assert np.abs(d[0] - want[:, 2 * i * n:(2 * i + 1) * n]).max() < TOL
        assert np.abs(d[1] - want[:, (2 * i + 1) * n:(2 * i + 2) * n]).max() < TOL


def test_attention_heads_gaussian_kernel():
    """Four heads (one pair-layout ciphertext of Q, K, V) through the score of the reference's attention layer:
    maskRightLeft, squares, oneMatRotSumInplace, transposed key norms, -2 Q K^T + |q|^2 + |k|^2, the degree-15
    table of exp(-x / 16), scores x V; every stage against float64.  12 levels hold masks (1) + scores (3) +
    polynomial (4) + scores x V (3) only if the products may run down to level 1: the preset keeps the reference's
    rule "bootstrap below level 4 + 3", so this uses the same primes with the minimum bootstrap level set to 0."""
    load_package()
    import bench
    from efla_amd import hellm
    from oracle import oracle as O
    qs, ps = O.ckks_chain(16, 13, 4)
    H = hellm.HEMMer(16, qs, ps, dnum=3, min_bootstrap_level=0, seed=3)
    rng = np.random.default_rng(12)
    n, d = 128, 64
    Q, K, V = (0.1 * rng.normal(size=(n, 12 * d)) for _ in range(3))
    (q, k, kt, v), = bench.gk_attention_inputs(H, Q, K, V, [1])
    # the stages of the first half (heads 8 and 10: left halves of tiles 2 and 3)
    mq, mk = H.mask_right_left(q), H.mask_right_left(k)
    sq, sk = [H.mult(x, x) for x in mq], [H.mult(x, x) for x in mk]
    H.one_mat_rot_sum_inplace(sq[0], sq[1])
    H.one_mat_rot_sum_inplace(sk[0], sk[1])
    H.transpose_inplace(sk[0], 8)
    s = H.single_cc_matmul(mq[0], kt, 8)
    x = H.add(H.add(H.mult_const(s, -2.0), H.level_down(sq[0], 8)), sk[0])
    assert x.info()["level"] == 8 == s.info()["level"]          # the integer constant took no level
    zx, zn = H.decrypt2(x), H.decrypt2(sq[1])
    for t in (0, 1):
        h = 2 * (2 + t)
        qh, kh = Q[:, h * d:(h + 1) * d], K[:, h * d:(h + 1) * d]
        dist = (qh * qh).sum(1)[:, None] + (kh * kh).sum(1)[None, :] - 2.0 * qh @ kh.T
        assert bench.GK_INTERVAL[0] < dist.min() and dist.max() < bench.GK_INTERVAL[1] + 0.25
        assert np.abs(zx[t] - dist).max() < TOL
        qr = Q[:, (h + 1) * d:(h + 2) * d]                       # the right half's norms, spread over the tile row
        assert np.abs(zn[t] - (qr * qr).sum(1)[:, None]).max() < TOL
    p = H.eval_chebyshev(H.linear_transform(x, *bench.GK_INTERVAL), bench.gk_table(), 4)
    assert p.info()["level"] == 4                                # the interval map is a subtraction; level_cost = 2 + 2
    # all four heads end to end
    outs = bench.gk_attention(H, [(q, k, kt, v)])
    assert all(o.info()["level"] == 1 for o in outs)
    assert bench.gk_attention_error(H, outs, Q, K, V, [1]) < 2.0 ** -12


def test_whole_layer_workloads(H):
    """Both layer-level workloads at their full extent -- every output column group of the LoRA projection (36 weight
    tile products, 12 CCMMs) and all 12 attention heads (24 CCMMs + 12 polynomial evaluations) -- exactly as the
    benchmark runs them, every decrypted output against float64 algebra."""
    import bench
    out = {}
    bench.gpu_layer_configs(None, out, H)
    assert out["config4_max_abs_err"] < 2.0 ** -12
    assert out["config5_max_abs_err"] < 2.0 ** -12
