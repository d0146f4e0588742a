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
    for (int i = 0; i < num_iter; i++) {
        for (size_t j = 0; j < op.size() / 2; j++) {
            Ciphertext &a = op[2 * j].get(), &b = op[2 * j + 1].get();
            if (a.getLevel() == btp.getMinLevelForBootstrap()) {
                eval.multImagUnit(b, b);
                eval.add(a, b, a);
                btp.bootstrap(a, a, b);
            }
        }
        // the squares of a round do not depend on one another: one launch chain for all of them (same residues)
        std::vector<const Ciphertext *> xs;
        for (size_t j = 0; j < 2 * (op.size() / 2); j++) xs.push_back(&op[j].get());
        if (xs.empty()) continue;
        std::vector<Ciphertext> sq;
        eval.multBatch(xs, xs, sq);
        for (size_t j = 0; j < sq.size(); j++) op[j].get() = std::move(sq[j]);
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

// sum over b in [0, len) of e[b] prod_k T_{2^k}^{bit k of b}, pw[k] = T_{2^k}, as a binary tree: a node of 2^(k+1)
// coefficients is lo + hi T_{2^k} with lo, hi its halves and sits k + 1 levels below the input: leaves e0 + e1 T_1 take
// one level (the constant is multiplied at the scale of the level and rescaled, however small it is), each product
// with T_{2^k} one more.  The tree is taken level by level: the products of one level do not depend on one another and
// go through HomEvaluator::multBatch together with the square that makes T_{2^(k+1)} for the next level (same residues
// as one product after the other).  pw holds T_1 on entry and is extended as far as the tree multiplies.
Value productTree(const HomEvaluator &eval, std::vector<Ciphertext> &pw, const Real *e, size_t len) {
    const Context &ctx = eval.getContext();
    if (len == 1) {
        Value v(ctx);
        v.cst = e[0];
        return v;
    }
    std::vector<Value> cur;
    {   // leaves e0 + e1 T_1: the products by the constants through one rescale
        std::vector<Real> csts;
        for (size_t j = 0; j < len / 2; j++)
            if (e[2 * j + 1] != 0.0) csts.push_back(e[2 * j + 1]);
        std::vector<Ciphertext> scaled;
        eval.multRealBatch(pw[0], csts, scaled);
        size_t taken = 0;
        for (size_t j = 0; j < len / 2; j++) {
            Value v(ctx);
            v.cst = e[2 * j];
            if (e[2 * j + 1] != 0.0) {
                v.ct = std::move(scaled[taken++]);
                if (e[2 * j] != 0.0) eval.add(v.ct, Complex(e[2 * j], 0.0), v.ct);
                v.has_ct = true;
            }
            cur.push_back(std::move(v));
        }
    }
    auto next_power = [&](const Ciphertext &square) {   // T_{2m} = 2 T_m^2 - 1
        Ciphertext p(square);
        eval.add(p, p, p);
        eval.add(p, Complex(-1.0, 0.0), p);
        pw.push_back(std::move(p));
    };
    if (cur.size() > 1) {   // T_2, which the first level of products multiplies by
        Ciphertext sq(ctx);
        eval.mult(pw[0], pw[0], sq);
        next_power(sq);
    }
    for (size_t k = 1; cur.size() > 1; k++) {
        const size_t n_nodes = cur.size() / 2;
        const bool more = n_nodes > 1;   // the next level multiplies by T_{2^(k+1)}
        std::vector<const Ciphertext *> fa, fb;
        for (size_t j = 0; j < n_nodes; j++)
            if (cur[2 * j + 1].has_ct) {
                fa.push_back(&cur[2 * j + 1].ct);
                fb.push_back(&pw[k]);
            }
        if (more) {
            fa.push_back(&pw[k]);
            fb.push_back(&pw[k]);
        }
        std::vector<Ciphertext> prod;
        if (!fa.empty()) eval.multBatch(fa, fb, prod);
        std::vector<Value> next;
        size_t taken = 0;
        for (size_t j = 0; j < n_nodes; j++) {
            Value &lo = cur[2 * j], &hi = cur[2 * j + 1];
            Value v(ctx);
            if (hi.has_ct) {
                v.ct = std::move(prod[taken++]);
                v.has_ct = true;
            } else if (hi.cst != 0.0) {
                eval.multWithoutRescale(pw[k], Complex(hi.cst, 0.0), v.ct);
                eval.rescale(v.ct);
                v.has_ct = true;
            }
            if (!v.has_ct) {
                next.push_back(std::move(lo));
                continue;
            }
            if (lo.has_ct)
                eval.add(v.ct, lo.ct, v.ct);
            else if (lo.cst != 0.0)
                eval.add(v.ct, Complex(lo.cst, 0.0), v.ct);
            next.push_back(std::move(v));
        }
        if (more) next_power(prod[taken]);
        cur = std::move(next);
    }
    return std::move(cur[0]);
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
    std::vector<Ciphertext> pw;      // T_1; the tree adds T_2, T_4, ... as far as it multiplies by them
    pw.push_back(ctxt);
    Value v = productTree(eval, pw, e.data(), len);
    if (!v.has_ct) throw std::invalid_argument("[evaluateChebyshevExpansion] constant polynomial");
    return v.ct;
}

}  // namespace Math
}  // namespace HEaaN
