// Polynomial evaluation on ciphertexts (see HELLM/PolyEval.hpp for the reference lines each routine follows).
#include <cmath>
#include <map>

#include "HELLM/PolyEval.hpp"

namespace HELLM {
using namespace HEaaN;

namespace Exp {

void exp_iter(const HomEvaluator &eval, const Bootstrapper &btp, const Ciphertext &op, Ciphertext &res, int num_iter) {
    Ciphertext r(eval.getContext());
    eval.mult(op, Complex(1.0 / std::pow(2, num_iter), 0.0), r);
    eval.add(r, Complex(1.0, 0.0), r);
    for (int i = 0; i < num_iter; i++) {
        if (r.getLevel() == btp.getMinLevelForBootstrap()) btp.bootstrap(r, r);
        eval.square(r, r);
    }
    res = std::move(r);
}

}  // namespace Exp

namespace ReLU {
namespace {

// tensor + rescale at the lower of the two levels, no relinearisation (ReLU.cpp:29-49)
void multWithoutRelin(const HomEvaluator &eval, const Ciphertext &a, const Ciphertext &b, Ciphertext &res) {
    Ciphertext t(eval.getContext());
    eval.tensor(a, b, t);
    eval.rescale(t);
    res = std::move(t);
}

void oddSetUp(const HomEvaluator &eval, const Ciphertext &ctxt, std::vector<Ciphertext> &odd, std::vector<Ciphertext> &giant,
              int k, int l) {
    std::vector<Ciphertext> even;
    odd.push_back(ctxt);
    even.push_back(ctxt);
    Ciphertext t(eval.getContext());
    const int logk = (int)std::log2(k);
    for (int i = 1; i <= logk; i++) {
        eval.mult(even[(size_t)i - 1], even[(size_t)i - 1], t);
        even.push_back(t);
    }
    for (int i = 1; i < k / 2; i++) {
        const int alpha = (int)std::floor(std::log2(2 * i + 1));
        const int ind = 1 << (alpha - 1);
        eval.mult(even[(size_t)alpha], odd[(size_t)(i - ind)], t);
        odd.push_back(t);
    }
    giant.push_back(even[(size_t)logk]);
    for (int j = 1; j < l; j++) {
        eval.mult(giant[(size_t)j - 1], giant[(size_t)j - 1], t);
        giant.push_back(t);
    }
}

void oddBabyStep(const HomEvaluator &eval, const std::vector<Ciphertext> &odd, const std::vector<double> &poly,
                 Ciphertext &res, int k) {
    Ciphertext r(eval.getContext()), t(eval.getContext());
    eval.mult(odd[0], Complex(poly[1], 0.0), r);
    for (int i = 1; i < k / 2; i++) {
        if ((size_t)(2 * i + 1) >= poly.size()) continue;
        eval.mult(odd[(size_t)i], Complex(poly[(size_t)(2 * i + 1)], 0.0), t);
        eval.add(r, t, r);
    }
    res = std::move(r);
}

void oddGiantStep(const HomEvaluator &eval, const std::vector<Ciphertext> &odd, const std::vector<Ciphertext> &giant,
                  const std::vector<double> &poly, Ciphertext &res, int k, int l) {
    const int degree = (int)poly.size() - 1;
    const int a = degree > 0 ? (int)std::floor(std::log2(degree / (double)k)) : -1;
    if (a < 0) {
        oddBabyStep(eval, odd, poly, res, k);
        return;
    }
    const int deg_div = k * (1 << a);
    const std::vector<double> quotient(poly.begin() + deg_div, poly.end()), remainder(poly.begin(), poly.begin() + deg_div);
    Ciphertext q(eval.getContext()), r(eval.getContext()), prod(eval.getContext());
    oddGiantStep(eval, odd, giant, quotient, q, k, l);
    if ((int)quotient.size() > k) eval.relinearize(q, q);
    oddGiantStep(eval, odd, giant, remainder, r, k, l);
    if ((size_t)a >= giant.size()) throw std::invalid_argument("[evalOddPolynomial] not enough giant-step powers (l)");
    multWithoutRelin(eval, giant[(size_t)a], q, prod);
    eval.add(prod, r, res);
}

}  // namespace

void evalOddPolynomial(const HomEvaluator &eval, Ciphertext &ctxt, Ciphertext &ctxt_poly,
                       const std::vector<double> &polynomial, int k, int l) {
    if (k < 2 || (k & (k - 1)) != 0 || l < 1 || polynomial.size() < 2)
        throw std::invalid_argument("[evalOddPolynomial] k must be a power of two >= 2, l >= 1, degree >= 1");
    std::vector<Ciphertext> odd, giant;
    oddSetUp(eval, ctxt, odd, giant, k, l);
    Ciphertext t(eval.getContext());
    oddGiantStep(eval, odd, giant, polynomial, t, k, l);
    if (t.getNumPoly() == 3)
        eval.relinearize(t, ctxt_poly);
    else
        ctxt_poly = std::move(t);
}

}  // namespace ReLU
}  // namespace HELLM

namespace HEaaN {
namespace Math {
namespace {

typedef std::map<u64, Ciphertext> Basis;

// T_1 .. T_baby and T_{2 baby}, T_{4 baby}, ... up to `top`
Basis chebBasis(const HomEvaluator &eval, const Ciphertext &u, u64 baby, u64 top) {
    Basis t;
    t.emplace(1, u);
    Ciphertext p(eval.getContext()), r(eval.getContext());
    for (u64 i = 2; i <= baby; i++) {
        const u64 hi = (i + 1) / 2, lo = i / 2;
        eval.mult(t.at(hi), t.at(lo), p);
        eval.add(p, p, p);
        if (hi == lo)
            eval.add(p, Complex(-1.0, 0.0), r);
        else
            eval.sub(p, t.at(1), r);
        t.emplace(i, r);
    }
    for (u64 m = baby; 2 * m <= top; m *= 2) {
        eval.mult(t.at(m), t.at(m), p);
        eval.add(p, p, p);
        eval.add(p, Complex(-1.0, 0.0), r);
        t.emplace(2 * m, r);
    }
    return t;
}

struct Value {
    bool has_ct = false;
    Ciphertext ct;
    bool has_const = false;
    Real cst = 0;
    explicit Value(const Context &c) : ct(c) {}
};

// sum_k c[k] T_k for len(c) <= baby + 1 (no ciphertext when every non-constant coefficient is zero)
Value chebCombination(const HomEvaluator &eval, const Basis &t, const std::vector<Real> &c) {
    Value v(eval.getContext());
    Ciphertext term(eval.getContext());
    for (size_t k = 1; k < c.size(); k++) {
        if (c[k] == 0.0) continue;
        eval.mult(t.at(k), Complex(c[k], 0.0), term);
        if (!v.has_ct) {
            v.ct = term;
            v.has_ct = true;
        } else {
            eval.add(v.ct, term, v.ct);
        }
    }
    if (v.has_ct && c[0] != 0.0) eval.add(v.ct, Complex(c[0], 0.0), v.ct);
    return v;
}

Value chebRecursive(const HomEvaluator &eval, const Basis &t, std::vector<Real> c, u64 baby) {
    size_t deg = c.size() - 1;
    while (deg > 0 && c[deg] == 0.0) deg--;
    c.resize(deg + 1);
    if (deg < baby) {
        Value v = chebCombination(eval, t, c);
        if (!v.has_ct && deg == 0) {
            v.has_const = true;
            v.cst = c[0];
        }
        return v;
    }
    u64 m = baby;
    while (2 * m <= deg) m *= 2;
    // c_k T_k = 2 c_k T_m T_{k-m} - c_k T_{2m-k} for m < k < 2m;  c_m T_m = c_m T_m T_0
    std::vector<Real> q(deg - m + 1, 0.0), r(c.begin(), c.begin() + (long)m);
    q[0] = c[m];
    for (size_t k = m + 1; k <= deg; k++) {
        q[k - m] = 2.0 * c[k];
        r[2 * m - k] -= c[k];
    }
    Value qv = chebRecursive(eval, t, q, baby), rv = chebRecursive(eval, t, r, baby);
    Value out(eval.getContext());
    if (!qv.has_ct) {
        if (qv.has_const && qv.cst != 0.0) {
            eval.mult(t.at(m), Complex(qv.cst, 0.0), out.ct);
            out.has_ct = true;
        }
    } else {
        eval.mult(qv.ct, t.at(m), out.ct);
        out.has_ct = true;
    }
    if (!rv.has_ct) {
        if (out.has_ct && rv.has_const && rv.cst != 0.0) eval.add(out.ct, Complex(rv.cst, 0.0), out.ct);
        return out;
    }
    if (out.has_ct)
        eval.add(out.ct, rv.ct, out.ct);
    else
        out = rv;
    return out;
}

}  // namespace

Ciphertext evaluateChebyshevExpansion(const HomEvaluator &eval, const Bootstrapper &, const Ciphertext &ctxt,
                                      const ChebyshevCoefficients &cc, Real multiplier) {
    const u64 baby = cc.num_baby_step;
    if (baby < 2 || (baby & (baby - 1)) != 0 || cc.coeffs.size() < 2)
        throw std::invalid_argument("[evaluateChebyshevExpansion] baby steps must be a power of two >= 2, degree >= 1");
    std::vector<Real> c(cc.coeffs);
    if (multiplier != 1.0)
        for (auto &x : c) x *= multiplier;
    const Basis t = chebBasis(eval, ctxt, baby, std::max<u64>(c.size() - 1, 1));
    Value v = chebRecursive(eval, t, c, baby);
    if (!v.has_ct) throw std::invalid_argument("[evaluateChebyshevExpansion] constant polynomial");
    return v.ct;
}

}  // namespace Math
}  // namespace HEaaN
