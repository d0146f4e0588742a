"""A product recorded into a HIP graph (hellm_graph_*) and replayed: every replay against the eager result, with
eager work and synchronisations between the replays and the operands rewritten in place (hellm_ct_assign)."""
import numpy as np
import pytest

from __graft_entry__ import load_package
from oracle import oracle as O

pytestmark = pytest.mark.gpu


def run(H, n, T, replays):
    rng = np.random.default_rng(5)
    mats = [rng.uniform(-1, 1, (n, n)) for _ in range(4)]
    ca, cb, ca2, cb2 = (H.encrypt(m) for m in mats)
    keep_a, keep_b = ca.clone(), cb.clone()
    want = [H.single_cc_matmul(ca, cb, T).residues(), H.single_cc_matmul(ca2, cb2, T).residues()]   # also warms every cache
    assert not np.array_equal(want[0], want[1])
    H.sync()
    graph, res = H.record(lambda: H.single_cc_matmul(ca, cb, T))
    assert graph.nodes() > 10
    for r in range(replays):
        graph.launch()
        graph.sync()
        assert np.array_equal(res.residues(), want[r % 2]), r
        # eager work between the replays, then the other operand pair written where the graph reads
        other = H.single_cc_matmul(ca2, cb2, T)
        assert np.array_equal(other.residues(), want[1])
        src = (ca2, cb2) if r % 2 == 0 else (keep_a, keep_b)
        H.assign(ca, src[0])
        H.assign(cb, src[1])
        H.sync()
    graph.free()
    # the context is back on its own stream and the pool is whole: one more eager product
    H.assign(ca, keep_a)
    H.assign(cb, keep_b)
    assert np.array_equal(H.single_cc_matmul(ca, cb, T).residues(), want[0])
    assert np.abs(H.decrypt(res) - (mats[0] @ mats[1] if replays % 2 == 1 else mats[2] @ mats[3])).max() < 2.0 ** -12


def test_recorded_product_small_ring():
    load_package()
    from efla_amd import hellm
    qs, ps = O.ckks_chain(10, 8, 3)
    H = hellm.HEMMer(10, qs, ps, dnum=3, min_bootstrap_level=0, seed=7)
    run(H, 16, 2, 4)


def test_recorded_product_full_ring():
    load_package()
    from efla_amd import hellm
    H = hellm.HEMMer(preset=True, seed=3)
    run(H, 128, 4, 3)


def test_two_contexts_replay_side_by_side():
    """Two HEMMers of one process (same seed, so the same keys; nothing is shared between their contexts) replay their
    recorded products at the same time on their own streams: each replay gives the residues of its eager product."""
    load_package()
    from efla_amd import hellm
    qs, ps = O.ckks_chain(10, 8, 3)
    rng = np.random.default_rng(9)
    lanes = []
    for k in range(2):
        H = hellm.HEMMer(10, qs, ps, dnum=3, min_bootstrap_level=0, seed=7)
        a, b = rng.uniform(-1, 1, (16, 16)), rng.uniform(-1, 1, (16, 16))
        ca, cb = H.encrypt(a), H.encrypt(b)
        want = H.single_cc_matmul(ca, cb, 2).residues()
        H.sync()
        graph, res = H.record(lambda: H.single_cc_matmul(ca, cb, 2))
        lanes.append((H, graph, res, want, a @ b, (ca, cb)))
    assert not np.array_equal(lanes[0][3], lanes[1][3])
    for _ in range(3):
        for _, graph, _, _, _, _ in lanes:
            graph.launch()
            graph.launch()      # two replays in a row on each stream, the two streams side by side
        for H, graph, res, want, prod, _ in lanes:
            graph.sync()
            assert np.array_equal(res.residues(), want)
            assert np.abs(H.decrypt(res) - prod).max() < 2.0 ** -12
    for _, graph, _, _, _, _ in lanes:
        graph.free()
