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
