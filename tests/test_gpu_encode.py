"""GPU parity of the device-side encode / decode (the canonical embedding on the orbit zeta^(5^j) and its inverse,
EnDecoder.hpp:51,66) against the CPU oracle: identical residues after encode, identical doubles after decode."""
import numpy as np
import pytest

from __graft_entry__ import load_package
from oracle import oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=[(9, 3, 1, 1), (10, 6, 2, 3), (13, 4, 2, 2), (16, 5, 3, 2)],
                ids=["N512", "N1024", "N8192", "N65536"])
def S(request):
    log_n, n_q, n_p, dnum = request.param
    pkg = load_package()
    qs, ps = O.ckks_chain(log_n, n_q, n_p)
    return pkg, O.Oracle(log_n, qs, ps, dnum), pkg.Context(log_n, qs, ps, dnum)


def messages(orc, rng, count):
    z = rng.uniform(-1, 1, (count, orc.slots)) + 1j * rng.uniform(-1, 1, (count, orc.slots))
    z[0, orc.slots // 3:] = 0          # a message with empty slots
    if count > 1:
        z[1] = 0.37 - 0.25j            # a constant
    return z


def test_encode_residues_match_the_oracle(S):
    import torch
    pkg, orc, ctx = S
    rng = np.random.default_rng(5)
    z = messages(orc, rng, 3)
    for level in (orc.nQ - 1, 1):
        got = ctx.encode(torch.from_numpy(z).cuda(), orc.delta[level], level + 1).cpu().numpy().view(np.uint64)
        for m in range(z.shape[0]):
            assert np.array_equal(got[m], orc.encode(z[m], level).data), (level, m)
    # over the extended basis, at a scale of the caller's choosing
    scale = orc.delta[1] * 0.75
    got = ctx.encode(torch.from_numpy(z[2]).cuda(), scale, 2, with_p=True).cpu().numpy().view(np.uint64)
    assert np.array_equal(got[0], orc.encode_ext(z[2], 1, scale).data)


def test_encode_rounds_halves_away_from_zero(S):
    """Slots chosen so that scaled coefficients land exactly on halves: a constant c encodes to the single coefficient
    c * scale, and scale = 1 with c = k + 1/2 puts it on a tie."""
    import torch
    pkg, orc, ctx = S
    for c in (2.5, -2.5, 0.5, -0.5, 7.0):
        z = np.full(orc.slots, c, dtype=np.complex128)
        got = ctx.encode(torch.from_numpy(z).cuda(), 1.0, 1).cpu().numpy().view(np.uint64)[0]
        assert np.array_equal(got, orc.encode(z, 0, 1.0).data), c
        want = int(np.floor(abs(c) + 0.5)) * (1 if c > 0 else -1)
        assert np.all(got[0] == np.uint64(want % int(orc.q[0])))      # a constant polynomial: every NTT slot holds it


def test_decode_matches_the_oracle(S):
    import torch
    pkg, orc, ctx = S
    rng = np.random.default_rng(6)
    z = messages(orc, rng, 1)[0]
    for level in (orc.nQ - 1, 0):
        pt = orc.encode(z, level)
        d = torch.from_numpy(pt.data.view(np.int64)).cuda()
        got = ctx.decode(d, pt.scale, n_limbs=min(2, level + 1)).cpu().numpy()
        want = orc.decode(pt)
        assert np.array_equal(got.view(np.float64), want.view(np.float64)), level
        assert np.abs(got - z).max() < 1e-6
