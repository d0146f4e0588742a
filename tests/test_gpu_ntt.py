"""GPU parity: batched negacyclic NTT/INTT through the C ABI vs the CPU oracle (bit-exact)."""
import numpy as np
import pytest

from __graft_entry__ import load_package
from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _to_dev(a):
    import torch
    return torch.from_numpy(a.view(np.int64)).cuda()


def _to_host(t):
    return t.cpu().numpy().view(np.uint64)


@pytest.mark.parametrize("log_n", [6, 8, 10, 12, 13, 14, 15, 16])
def test_ntt_matches_oracle(log_n):
    pkg = load_package()
    qs = O.primes_below(60, log_n, 2) + [O.nearest_prime(2**42, log_n)]
    ps = O.primes_below(59, log_n, 1)
    ctx = pkg.Context(log_n, qs, ps, 1)
    orc = O.Oracle(log_n, qs, ps, 1)
    rng = np.random.default_rng(log_n)
    mods = qs + ps
    idx = [3, 0, 2, 1, 0]                      # arbitrary limb -> prime map, with a repeat
    a = np.stack([[rng.integers(0, mods[i], 1 << log_n, dtype=np.uint64) for i in idx] for _ in range(3)])
    a[0, 0, :4] = [mods[3] - 1, 0, 1, mods[3] - 1]
    for i in range(len(mods)):
        assert ctx.psi(i) == orc.L.orc_psi(orc.h, i)
    d = _to_dev(a)
    ctx.ntt(d, idx)
    want = a.copy()
    orc.ntt(want, idx)
    assert np.array_equal(_to_host(d), want)
    ctx.ntt(d, idx, inverse=True)
    assert np.array_equal(_to_host(d), a)
    # inverse alone on arbitrary residues
    ctx.ntt(d, idx, inverse=True)
    want = a.copy()
    orc.ntt(want, idx, inverse=True)
    assert np.array_equal(_to_host(d), want)


@pytest.mark.parametrize("log_n", [10, 16])
def test_ntt_extreme_residues(log_n):
    """Inputs that push the lazy butterflies towards the top of their ranges (values stay below 8q forward and 4q
    inverse between corrections): all q-1, alternating 0 / q-1, q-1 in one half; the largest primes below 2^61,
    below 2^60 and a small one."""
    pkg = load_package()
    qs = [O.nearest_prime(2**61 - 2**20, log_n), O.primes_below(60, log_n, 1)[0], O.nearest_prime(2**42, log_n)]
    assert qs[0] < 2**61
    ctx = pkg.Context(log_n, qs, [], 1)
    orc = O.Oracle(log_n, qs, [], 1)
    N = 1 << log_n
    pats = []
    for q in qs:
        top = np.uint64(q - 1)
        alt = np.zeros(N, dtype=np.uint64)
        alt[::2] = top
        half = np.zeros(N, dtype=np.uint64)
        half[N // 2:] = top
        pats.append([np.full(N, top, dtype=np.uint64), alt, half])
    a = np.ascontiguousarray(np.array(pats).transpose(1, 0, 2))    # [pattern][limb][N]
    idx = [0, 1, 2]
    for inverse in (False, True):
        d = _to_dev(a.copy())
        ctx.ntt(d, idx, inverse=inverse)
        want = a.copy()
        orc.ntt(want, idx, inverse=inverse)
        assert np.array_equal(_to_host(d), want)


def test_ntt_config2_roundtrip_full_batch():
    """32 polys x 24 limbs x 2^16 with the 24 largest 60-bit NTT primes: bit-exact round trip on
    the whole batch, forward output of every polynomial checked against the oracle."""
    import torch
    pkg = load_package()
    qs = O.primes_below(60, 16, 24)
    assert qs == pkg.primes_below(60, 16, 24)
    ctx = pkg.Context(16, qs, [], 1)
    orc = O.Oracle(16, qs, [], 1, threads=8)
    g = torch.Generator(device="cuda").manual_seed(7)
    q_t = torch.tensor(qs, dtype=torch.int64, device="cuda").view(1, 24, 1)
    d = torch.randint(0, 2**62, (32, 24, 1 << 16), dtype=torch.int64, device="cuda", generator=g) % q_t
    a = d.clone()
    ctx.ntt(d, list(range(24)))
    for p in range(32):
        sl = _to_host(a[p]).copy()
        orc.ntt(sl, list(range(24)))
        assert np.array_equal(_to_host(d[p]), sl), p
    assert bool((d >= 0).all()) and bool((d < q_t).all())
    # linearity: NTT(a + b) = NTT(a) + NTT(b) mod q on two polys of the batch
    s = (a[0] + a[1]) % q_t[0]
    ctx.ntt(s.unsqueeze(0).contiguous(), list(range(24)))
    ctx.ntt(d, list(range(24)), inverse=True)
    assert torch.equal(d, a)


def test_bad_arguments():
    pkg = load_package()
    with pytest.raises(ValueError):
        pkg.Context(16, [2**60 - 1], [], 1)          # not prime / not NTT friendly
    with pytest.raises(ValueError):
        pkg.Context(16, O.primes_below(60, 16, 2), [], 3)   # dnum > n_q
