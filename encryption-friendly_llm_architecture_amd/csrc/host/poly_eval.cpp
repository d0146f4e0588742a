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

void exp_iter_Parallel(const HomEvaluator &eval, const Bootstrapper &btp, std::vector<HELLM::CtxtTensor> &op, int num_iter) {
    for (auto &t : op) {
        eval.mult(t.get(), Complex(1.0 / std::pow(2, num_iter), 0.0), t.get());
        eval.add(t.get(), Complex(1.0, 0.0), t.get());
    }
    for (int i = 0; i < num_iter; i++)
        for (size_t j = 0; j < op.size() / 2; j++) {
            Ciphertext &a = op[2 * j].get(), &b = op[2 * j + 1].get();
            if (a.getLevel() == btp.getMinLevelForBootstrap()) {
                eval.multImagUnit(b, b);
                eval.add(a, b, a);
                btp.bootstrap(a, a, b);
            }
            eval.square(a, a);
            eval.square(b, b);
        }
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

// A block of plain Chebyshev coefficients c[0 .. 2m) (coefficient of T_j) rewritten over products of T_1, T_2, T_4,
// ..., T_m: out[b] multiplies prod_k T_{2^k}^{bit k of b}.  One step: c_k T_k = 2 c_k T_m T_{k-m} - c_k T_{2m-k} for
// m < k < 2m and c_m T_m = c_m T_m T_0, i.e. c = r + T_m q with q[0] = c_m, q[k-m] = 2 c_k, r[2m-k] -= c_k.
void toBinaryProductBasis(std::vector<Real> c, Real *out) {
    const size_t len = c.size();
    if (len == 1) {
        out[0] = c[0];
        return;
    }
    const size_t m = len / 2;
    std::vector<Real> q(m, 0.0), r(c.begin(), c.begin() + (long)m);
    q[0] = c[m];
    for (size_t k = m + 1; k < len; k++) {
        q[k - m] = 2.0 * c[k];
        r[2 * m - k] -= c[k];
    }
    toBinaryProductBasis(std::move(r), out);
    toBinaryProductBasis(std::move(q), out + m);
}

struct Value {
    bool has_ct = false;
    Ciphertext ct;
    Real cst = 0;     // the value when !has_ct
    explicit Value(const Context &c) : ct(c) {}
};

// sum over b in [lo, lo + len) of e[b] prod_k T_{2^k}^{bit k of (b - lo)}; pw[k] = T_{2^k}.  A node of 2^k
// coefficients sits k levels below the input: leaves e0 + e1 T_1 take one level (the constant is multiplied at the
// scale of the level and rescaled, however small it is), each product with T_{len/2} one more.
Value productTree(const HomEvaluator &eval, const std::vector<Ciphertext> &pw, const Real *e, size_t len) {
    Value v(eval.getContext());
    if (len == 1) {
        v.cst = e[0];
        return v;
    }
    if (len == 2) {
        v.cst = e[0];
        if (e[1] != 0.0) {
            eval.multWithoutRescale(pw[0], Complex(e[1], 0.0), v.ct);
            eval.rescale(v.ct);
            if (e[0] != 0.0) eval.add(v.ct, Complex(e[0], 0.0), v.ct);
            v.has_ct = true;
        }
        return v;
    }
    const size_t h = len / 2;
    size_t k = 0;
    while (((size_t)1 << k) < h) k++;
    Value lo = productTree(eval, pw, e, h), hi = productTree(eval, pw, e + h, h);
    if (hi.has_ct) {
        eval.mult(hi.ct, pw[k], v.ct);
        v.has_ct = true;
    } else if (hi.cst != 0.0) {
        eval.multWithoutRescale(pw[k], Complex(hi.cst, 0.0), v.ct);
        eval.rescale(v.ct);
        v.has_ct = true;
    }
    if (!v.has_ct) return lo;
    if (lo.has_ct)
        eval.add(v.ct, lo.ct, v.ct);
    else if (lo.cst != 0.0)
        eval.add(v.ct, Complex(lo.cst, 0.0), v.ct);
    return v;
}

}  // namespace

Ciphertext linearTransform(const HomEvaluator &eval, const Bootstrapper &, const Ciphertext &ctxt,
                           const InputInterval &iv) {
    if (!(iv.right_end > iv.left_end)) throw std::invalid_argument("[linearTransform] empty interval");
    Ciphertext r(eval.getContext());
    const Real mid = 0.5 * (iv.right_end + iv.left_end);
    if (mid != 0.0)
        eval.add(ctxt, Complex(-mid, 0.0), r);
    else
        r = ctxt;
    eval.mult(r, Complex(2.0 / (iv.right_end - iv.left_end), 0.0), r);
    return r;
}

Ciphertext evaluateChebyshevExpansion(const HomEvaluator &eval, const Bootstrapper &, const Ciphertext &ctxt,
                                      const ChebyshevCoefficients &cc, const Real multiplier) {
    if (cc.basis != PolynomialBasis::basic)
        throw std::invalid_argument("[evaluateChebyshevExpansion] only the basic polynomial basis is built");
    if (cc.coeffs.size() < 2) throw std::invalid_argument("[evaluateChebyshevExpansion] constant polynomial");
    u64 bs = cc.num_bs, gs = cc.num_gs;
    if (gs > 1 && (bs & (bs - 1)) != 0)
        throw std::invalid_argument("[evaluateChebyshevExpansion] the number of baby steps must be a power of two");
    const u64 B = (u64)1 << cc.log_bs, G = (u64)1 << cc.log_gs;
    // every block of bs plain coefficients over products of T_1 .. T_{B/2}; block i then multiplies the product of
    // T_{2^k bs} over the bits of i: one coefficient vector over products of T_1, T_2, T_4, ..., T_{B G / 2}
    std::vector<Real> e(B * G, 0.0);
    for (u64 i = 0; i < gs; i++) {
        std::vector<Real> block(B, 0.0);
        for (u64 j = 0; j < bs && i * bs + j < cc.coeffs.size(); j++) block[j] = multiplier * cc.coeffs[i * bs + j];
        toBinaryProductBasis(std::move(block), e.data() + i * B);
    }
    size_t top = e.size();
    while (top > 1 && e[top - 1] == 0.0) top--;
    size_t len = 2;
    while (len < top) len *= 2;
    std::vector<Ciphertext> pw;      // T_1, T_2, T_4, ... as far as the tree multiplies by them
    pw.push_back(ctxt);
    Ciphertext p(eval.getContext());
    for (size_t m = 2; m < len; m *= 2) {
        eval.mult(pw.back(), pw.back(), p);
        eval.add(p, p, p);
        eval.add(p, Complex(-1.0, 0.0), p);
        pw.push_back(p);
    }
    Value v = productTree(eval, pw, e.data(), len);
    if (!v.has_ct) throw std::invalid_argument("[evaluateChebyshevExpansion] constant polynomial");
    return v.ct;
}

}  // namespace Math
}  // namespace HEaaN
