"""hemm_rescale_static, the rescale for callers that cannot allocate device memory, against hemm_rescale (same
arguments, context-owned scratch) and the CPU oracle: bit-exact, on two calls in a row that share the static
scratch, the second on a smaller input; sizes beyond the static scratch are refused."""
import numpy as np
import pytest

from __graft_entry__ import load_package
from oracle import oracle as O

pytestmark = pytest.mark.gpu


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int64)).cuda()


def host(t):
    return t.cpu().numpy().view(np.uint64)


def rand_ct(rng, mods, n_polys, N):
    out = np.empty((n_polys, len(mods), N), dtype=np.uint64)
    for j, q in enumerate(mods):
        out[:, j, :] = rng.integers(0, q, (n_polys, N), dtype=np.uint64)
    return out


@pytest.mark.parametrize("log_n", [16, 12], ids=["N65536", "N4096"])
def test_rescale_static_matches_rescale(log_n):
    import torch
    pkg = load_package()
    qs, ps = O.ckks_chain(log_n, 7, 4)
    ctx = pkg.Context(log_n, qs, ps, 3)
    orc = O.Oracle(log_n, qs, ps, 3)
    N = 1 << log_n
    rng = np.random.default_rng(100 + log_n)
    # first call: two polynomials at the top level; second call: three polynomials (a tensor product) four limbs
    # lower, which reuses the front of the same scratch
    for n_polys, nq in ((2, 7), (3, 3)):
        a = rand_ct(rng, qs[:nq], n_polys, N)
        a[0, nq - 1, :4] = [0, 1, qs[nq - 1] - 1, qs[nq - 1] // 2]
        d = dev(a)
        want = host(ctx.rescale(d, nq))
        out = torch.full((n_polys, nq - 1, N), -1, dtype=torch.int64, device="cuda")
        torch.cuda.synchronize()
        got = host(ctx.rescale_static(d, nq, out))
        assert np.array_equal(got, want)
        assert np.array_equal(host(d), a), "the input is left as it was"
        assert np.array_equal(got, orc.rescale(O.Ct(a, 1.0)).data)


def test_rescale_static_allocates_nothing_on_a_fresh_context():
    """The first call on a context that has done nothing else: device memory in use is the same before and after
    (hipMemGetInfo through torch), and the result is the oracle's."""
    import torch
    pkg = load_package()
    qs, ps = O.ckks_chain(16, 7, 4)
    orc = O.Oracle(16, qs, ps, 3)
    rng = np.random.default_rng(321)
    a = rand_ct(rng, qs[:5], 2, 1 << 16)
    d = dev(a)
    out = torch.empty((2, 4, 1 << 16), dtype=torch.int64, device="cuda")
    # a first call on another context takes what the runtime allocates once per process (the library's code object,
    # its kernel-argument pools), so that what is measured below is the entry point and the fresh context alone
    warm = pkg.Context(16, qs, ps, 3)
    warm.rescale_static(d, 5, out)
    ctx = pkg.Context(16, qs, ps, 3)          # tables and the scratch address are set up here
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    ctx.rescale_static(d, 5, out)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert np.array_equal(host(out), orc.rescale(O.Ct(a, 1.0)).data)


def test_rescale_layout_checks_and_in_place():
    """Strides shorter than a polynomial and partial overlaps of out with in are refused by both entry points; out == in
    with equal strides gives the out-of-place result."""
    import torch
    pkg = load_package()
    qs, ps = O.ckks_chain(16, 7, 4)
    ctx = pkg.Context(16, qs, ps, 3)
    N, nq = 1 << 16, 4
    rng = np.random.default_rng(322)
    a = rand_ct(rng, qs[:nq], 2, N)
    want = host(ctx.rescale(dev(a), nq))
    lib, vp = pkg.lib(), pkg.vp
    for fn in (lib.hemm_rescale, lib.hemm_rescale_static):
        buf = dev(a)
        assert fn(ctx.h, vp(buf.data_ptr()), nq * N, vp(buf.data_ptr()), nq * N, nq, 2, vp(0)) == 0    # in place
        torch.cuda.synchronize()
        assert np.array_equal(host(buf)[:, : nq - 1], want)
        buf = dev(a)
        other = torch.empty((2, nq, N), dtype=torch.int64, device="cuda")
        assert fn(ctx.h, vp(buf.data_ptr()), nq * N - 1, vp(other.data_ptr()), (nq - 1) * N, nq, 2, vp(0)) == 1
        assert fn(ctx.h, vp(buf.data_ptr()), nq * N, vp(other.data_ptr()), (nq - 1) * N - 1, nq, 2, vp(0)) == 1
        assert fn(ctx.h, vp(buf.data_ptr()), nq * N, vp(buf.data_ptr() + 8 * N), nq * N, nq, 1, vp(0)) == 1   # shifted by a limb
        assert fn(ctx.h, vp(buf.data_ptr()), nq * N, vp(buf.data_ptr()), (nq - 1) * N, nq, 2, vp(0)) == 1   # other stride


def test_rescale_static_refuses_inputs_beyond_its_scratch():
    import torch
    pkg = load_package()
    qs, ps = O.ckks_chain(16, 7, 4)
    ctx = pkg.Context(16, qs, ps, 3)
    limit = 32  # limbs of N = 2^16 the static scratch holds
    n_polys, nq = 5, 7
    assert n_polys * nq > limit
    d = torch.zeros((n_polys, nq, 1 << 16), dtype=torch.int64, device="cuda")
    out = torch.zeros((n_polys, nq - 1, 1 << 16), dtype=torch.int64, device="cuda")
    with pytest.raises(ValueError, match="HEMM_STATIC_SCRATCH_WORDS"):
        ctx.rescale_static(d, nq, out)
    with pytest.raises(ValueError):
        ctx.rescale_static(d[:1], 1, out[:1])
