"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the polynomial evaluation routines built on the evaluator:

  * exp_iter             reference ciphertext/src/Exp.cpp:41-52   ((1 + x / 2^k)^(2^k) by repeated squaring)
  * eval_odd_polynomial  reference ciphertext/src/ReLU.cpp:53-188 (Han-Ki baby-step / giant-step for odd
                         polynomials given by monomial coefficients; products stay un-relinearised until
                         a giant-step multiplication needs them)
  * eval_chebyshev       HEaaN::Math::evaluateChebyshevExpansion is closed (PolynomialEvaluator.hpp:49-63
                         is only a declaration); this is the textbook baby-step / giant-step evaluation in
                         the Chebyshev basis, stated here and mirrored operation by operation by the product.
                         Parity with HEaaN's own residues is unpinned; what is pinned is the value
                         (numpy.polynomial.chebyshev.chebval) and GPU == this restatement.

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


# ---- Chebyshev basis -------------------------------------------------------------------------------
def _cheb_basis(ev, u, baby, top):
    """T_1 .. T_baby and T_{2 baby}, T_{4 baby}, ... up to `top`, from T_2m = 2 T_m^2 - 1 and
    T_{m+n} = 2 T_m T_n - T_{m-n}."""
    t = {1: u}
    for i in range(2, baby + 1):
        hi, lo = (i + 1) // 2, i // 2
        p = ev.mult(t[hi], t[lo])
        p = ev.add(p, p)
        t[i] = ev.add_const(p, -1.0) if hi == lo else ev.sub(p, t[1])
    m = baby
    while 2 * m <= top:
        p = ev.mult(t[m], t[m])
        t[2 * m] = ev.add_const(ev.add(p, p), -1.0)
        m *= 2
    return t


def _cheb_combination(ev, t, c):
    """sum_k c[k] T_k for len(c) <= baby + 1, None when every coefficient is zero."""
    r = None
    for k in range(1, len(c)):
        if c[k] == 0.0:
            continue
        term = ev.mult_const(t[k], c[k])
        r = term if r is None else ev.add(r, term)
    if r is None:
        return None
    return ev.add_const(r, c[0]) if c[0] != 0.0 else r


def _cheb_recursive(ev, t, c, baby):
    deg = len(c) - 1
    while deg > 0 and c[deg] == 0.0:
        deg -= 1
    c = c[: deg + 1]
    if deg < baby:
        return _cheb_combination(ev, t, c), (c[0] if deg == 0 else None)
    m = baby
    while 2 * m <= deg:
        m *= 2
    # c_k T_k = 2 c_k T_m T_{k-m} - c_k T_{2m-k}  for m < k < 2m;  c_m T_m = c_m T_m T_0
    q = [0.0] * (deg - m + 1)
    r = list(c[:m])
    q[0] = c[m]
    for k in range(m + 1, deg + 1):
        q[k - m] = 2.0 * c[k]
        r[2 * m - k] -= c[k]
    qv, qconst = _cheb_recursive(ev, t, q, baby)
    rv, rconst = _cheb_recursive(ev, t, r, baby)
    # q(u) * T_m: a constant q multiplies T_m by a scalar
    if qv is None:
        prod = ev.mult_const(t[m], qconst) if qconst not in (None, 0.0) else None
    else:
        prod = ev.mult(qv, t[m])
    if rv is None:
        out = prod
        if rconst not in (None, 0.0):
            out = ev.add_const(out, rconst)
        return out, None
    return (ev.add(prod, rv) if prod is not None else rv), None


def eval_chebyshev(ev, u, coeffs, baby):
    """sum_k coeffs[k] T_k(u) for u with values in [-1, 1]; baby = number of baby steps (power of two)."""
    coeffs = [float(x) for x in coeffs]
    deg = len(coeffs) - 1
    t = _cheb_basis(ev, u, baby, max(deg, 1))
    v, const = _cheb_recursive(ev, t, coeffs, baby)
    if v is None:
        raise ValueError("constant polynomial")
    return v
