"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the polynomial evaluation routines built on the evaluator:

  * exp_iter             reference ciphertext/src/Exp.cpp:41-52   ((1 + x / 2^k)^(2^k) by repeated squaring)
  * exp_iter_parallel    reference ciphertext/src/Exp.cpp:55-77   (the same on a list of tensors, pair by pair)
  * eval_odd_polynomial  reference ciphertext/src/ReLU.cpp:53-188 (Han-Ki baby-step / giant-step for odd
                         polynomials given by monomial coefficients; products stay un-relinearised until
                         a giant-step multiplication needs them)
  * eval_chebyshev       HEaaN::Math::evaluateChebyshevExpansion is closed (PolynomialEvaluator.hpp:49-63 is
                         only a declaration).  Its coefficient convention -- the baby-step / giant-step product
                         basis the header comment spells out -- is followed; the order of operations is this
                         build's and is mirrored operation by operation by the product.  Pins: the reference's
                         own EXP_15_4 table (include/HELLM/LossRemezCoeff.hpp:18-35) evaluates to exp on
                         [-2, 2] (src/Loss.cpp:41-56) to 1e-10; plain Chebyshev series converted to the product
                         basis agree with numpy's chebval; GPU == this restatement.  Parity with HEaaN's own
                         residues is unpinned.

Every function takes an evaluator `ev` with mult / tensor / rescale / relinearize / add / sub / mult_const /
add_const / level_of (hemmer_ref.SlotSim for exact slot arithmetic, hemmer_ref.OracleEval for the CKKS oracle).
"""
import math


def exp_iter(ev, x, num_iter):
    r = ev.mult_const(x, 1.0 / math.pow(2, num_iter))
    r = ev.add_const(r, 1.0)
    for _ in range(num_iter):
        r = ev.mult(r, r)
    return r


def exp_iter_parallel(ev, xs, num_iter):
    """reference ciphertext/src/Exp.cpp:55-77: every tensor scaled and shifted, then num_iter rounds in which the
    pairs (2j, 2j+1) are squared; a trailing tensor without a partner is never squared."""
    xs = [ev.add_const(ev.mult_const(x, 1.0 / math.pow(2, num_iter)), 1.0) for x in xs]
    for _ in range(num_iter):
        for j in range(len(xs) // 2):
            xs[2 * j] = ev.mult(xs[2 * j], xs[2 * j])
            xs[2 * j + 1] = ev.mult(xs[2 * j + 1], xs[2 * j + 1])
    return xs


# ---- odd polynomials, monomial basis (ReLU.cpp) ----------------------------------------------------
def _mult_without_relin(ev, a, b):
    """ReLU.cpp:29-49: tensor + rescale at the lower of the two levels."""
    return ev.rescale(ev.tensor(a, b))


def _odd_set_up(ev, x, k, l):
    odd, even = [x], [x]
    for i in range(1, int(math.log2(k)) + 1):
        even.append(ev.mult(even[i - 1], even[i - 1]))
    for i in range(1, k // 2):
        alpha = int(math.floor(math.log2(2 * i + 1)))
        ind = 2 ** (alpha - 1)
        odd.append(ev.mult(even[alpha], odd[i - ind]))
    giant = [even[int(math.log2(k))]]
    for j in range(1, l):
        giant.append(ev.mult(giant[j - 1], giant[j - 1]))
    return odd, giant


def _odd_baby_step(ev, odd, poly, k):
    r = ev.mult_const(odd[0], poly[1])
    for i in range(1, k // 2):
        if 2 * i + 1 < len(poly):
            r = ev.add(r, ev.mult_const(odd[i], poly[2 * i + 1]))
    return r


def _odd_giant_step(ev, odd, giant, poly, k, l):
    degree = len(poly) - 1
    a = int(math.floor(math.log2(degree / float(k)))) if degree > 0 else -1
    if a < 0:
        return _odd_baby_step(ev, odd, poly, k)
    deg_div = k * 2 ** a
    quotient, remainder = poly[deg_div:], poly[:deg_div]
    q = _odd_giant_step(ev, odd, giant, quotient, k, l)
    if len(quotient) > k:
        q = ev.relinearize(q)
    r = _odd_giant_step(ev, odd, giant, remainder, k, l)
    return ev.add(_mult_without_relin(ev, giant[a], q), r)


def eval_odd_polynomial(ev, x, poly, k, l):
    """poly[i] = coefficient of x^i (even entries ignored); k = baby-step count (power of two), l = number
    of giant-step powers x^k, x^2k, x^4k, ... kept."""
    odd, giant = _odd_set_up(ev, x, k, l)
    return ev.relinearize(_odd_giant_step(ev, odd, giant, list(poly), k, l))


# ---- Chebyshev expansions in the baby-step / giant-step product basis ---------------------------------
def cheb_product_value(d, bs, t):
    """Value of the expansion the reference's tables hold (PolynomialEvaluator.hpp:49-58), straight from its
    definition: sum_i (sum_j d[bs i + j] T_j(t)) * prod_k T_{2^k bs}(t)^{bit k of i}.  numpy, for the tests."""
    import numpy as np
    from numpy.polynomial import chebyshev as C
    t = np.asarray(t, dtype=np.float64)
    d = [float(x) for x in d]
    bs = bs if bs > 0 else len(d)
    gs = -(-len(d) // bs)
    total = np.zeros_like(t)
    for i in range(gs):
        block = d[bs * i: bs * (i + 1)]
        term = C.chebval(t, block)
        k = 0
        while (i >> k) != 0:
            if (i >> k) & 1:
                term = term * C.chebval(t, [0.0] * ((1 << k) * bs) + [1.0])
            k += 1
        total = total + term
    return total


def cheb_plain_to_product(c, bs):
    """Plain Chebyshev series c (coefficient of T_k) -> the product basis with bs baby steps (bs a power of two):
    c_k T_k = 2 c_k T_m T_{k-m} - c_k T_{2m-k} for m < k < 2m, applied from the top giant step down to m = bs."""
    c = [float(x) for x in c]
    size = bs
    while size < len(c):
        size *= 2
    c = c + [0.0] * (size - len(c))

    def split(c):
        if len(c) <= bs:
            return c
        m = len(c) // 2
        q, r = [0.0] * m, c[:m]
        q[0] = c[m]
        for k in range(m + 1, len(c)):
            q[k - m] = 2.0 * c[k]
            r[2 * m - k] -= c[k]
        return split(r) + split(q)

    return split(c)


def _to_binary_product_basis(c):
    """c[0 .. 2m) plain -> coefficients over products of T_1, T_2, T_4, ..., T_m (bit k of the index <-> T_{2^k})."""
    if len(c) == 1:
        return [c[0]]
    m = len(c) // 2
    q, r = [0.0] * m, list(c[:m])
    q[0] = c[m]
    for k in range(m + 1, len(c)):
        q[k - m] = 2.0 * c[k]
        r[2 * m - k] -= c[k]
    return _to_binary_product_basis(r) + _to_binary_product_basis(q)


def _product_tree(ev, pw, e):
    """(ciphertext or None, constant): sum_b e[b] prod_k T_{2^k}^{bit k of b}, pw[k] = T_{2^k}."""
    if len(e) == 1:
        return None, e[0]
    if len(e) == 2:
        if e[1] == 0.0:
            return None, e[0]
        v = ev.mult_const_rescale(pw[0], e[1])
        return (ev.add_const(v, e[0]) if e[0] != 0.0 else v), e[0]
    h = len(e) // 2
    k = h.bit_length() - 1
    lo, lo_c = _product_tree(ev, pw, e[:h])
    hi, hi_c = _product_tree(ev, pw, e[h:])
    if hi is not None:
        v = ev.mult(hi, pw[k])
    elif hi_c != 0.0:
        v = ev.mult_const_rescale(pw[k], hi_c)
    else:
        return lo, lo_c
    if lo is not None:
        return ev.add(v, lo), 0.0
    return (ev.add_const(v, lo_c) if lo_c != 0.0 else v), 0.0


def linear_transform(ev, x, left, right):
    """HEaaN::Math::linearTransform (PolynomialEvaluator.hpp:42-47): (2 / (right - left)) (x - (right + left) / 2)."""
    mid = 0.5 * (right + left)
    r = ev.add_const(x, -mid) if mid != 0.0 else x
    return ev.mult_const(r, 2.0 / (right - left))


def eval_chebyshev(ev, u, coeffs, baby, multiplier=1.0):
    """HEaaN::Math::evaluateChebyshevExpansion on ChebyshevCoefficients{coeffs, baby} (PolynomialEvaluator.hpp:
    19-63): multiplier * sum_i (sum_j coeffs[bs i + j] T_j(u)) prod_k T_{2^k bs}(u)^{bit k of i}, u in [-1, 1].
    The blocks are rewritten over products of T_1, T_2, T_4, ... so that constants only multiply T_1; the tree then
    uses ceil(log2 bs) + ceil(log2 gs) levels, the header's level_cost."""
    d = [float(x) for x in coeffs]
    bs = baby if baby > 0 else len(d)
    gs = -(-len(d) // bs)
    if gs > 1 and bs & (bs - 1):
        raise ValueError("the number of baby steps must be a power of two")
    B = 1 << max(0, (bs - 1).bit_length())
    G = 1 << max(0, (gs - 1).bit_length())
    e = []
    for i in range(G):
        block = [multiplier * x for x in d[bs * i: bs * (i + 1)]] if i < gs else []
        e += _to_binary_product_basis(block + [0.0] * (B - len(block)))
    top = len(e)
    while top > 1 and e[top - 1] == 0.0:
        top -= 1
    size = 2
    while size < top:
        size *= 2
    pw = [u]
    m = 2
    while m < size:
        p = ev.mult(pw[-1], pw[-1])
        pw.append(ev.add_const(ev.add(p, p), -1.0))
        m *= 2
    v, _ = _product_tree(ev, pw, e[:size])
    if v is None:
        raise ValueError("constant polynomial")
    return v
