// Polynomial evaluation on ciphertexts.
//   HELLM::Exp::exp_iter            reference ciphertext/src/Exp.cpp:41-52, include/HELLM/Exp.hpp
//   HELLM::ReLU::evalOddPolynomial  reference ciphertext/src/ReLU.cpp:53-188 (Han-Ki baby-step / giant-step)
//   HEaaN::Math::ChebyshevCoefficients / linearTransform / evaluateChebyshevExpansion
//                                   declared by the closed HEaaN-math (PolynomialEvaluator.hpp:19-63, used as
//                                   in include/HELLM/LossRemezCoeff.hpp:18-35 and src/Loss.cpp:41-56): the
//                                   coefficient convention (baby-step / giant-step product basis) is the
//                                   header's; the order of operations is this build's.
// Every routine needs enough levels for its depth: bootstrapping is not part of this build, so the
// places where the reference would bootstrap raise HEaaN::RuntimeException instead.
#pragma once
#include <cmath>
#include <vector>

#include "HEaaN/HEaaN.hpp"

namespace HEaaN {
namespace Math {

// HEaaN-math/tools/Intervals.hpp:16-27
struct Interval {
    Interval(const Real left, const Real right) : left_end{left}, right_end{right} {}
    Real left_end;
    Real right_end;
};
using InputInterval = Interval;
using DiffInterval = Interval;

// HEaaN-math/tools/PolynomialEvaluator.hpp:19-40: same members, same constructor arithmetic.  The coefficients are
// NOT a plain Chebyshev series: entry bs * i + j multiplies T_j times the product of T_{2^k bs} over the set bits k
// of i (the tables of include/HELLM/*RemezCoeff.hpp are stored that way).
enum PolynomialBasis { basic, odd };
struct ChebyshevCoefficients {
    ChebyshevCoefficients(std::vector<Real> coefficient, u64 num_baby_step, PolynomialBasis base = PolynomialBasis::basic)
        : coeffs{std::move(coefficient)}, basis{base} {
        num_bs = (num_baby_step > 0) ? num_baby_step : coeffs.size();
        num_gs = static_cast<u64>(std::ceil(static_cast<Real>(coeffs.size()) / static_cast<Real>(num_bs)));
        log_bs = static_cast<u64>(std::ceil(std::log2(num_bs)));
        log_gs = static_cast<u64>(std::ceil(std::log2(num_gs)));
        level_cost = log_bs + log_gs;
    }
    std::vector<Real> coeffs;
    u64 num_bs;
    u64 num_gs;
    u64 log_bs;
    u64 log_gs;
    u64 level_cost;
    PolynomialBasis basis;
};

// (2 / (right - left)) * (ctxt - (right + left) / 2): [left, right] -> [-1, 1] (PolynomialEvaluator.hpp:42-47);
// one level unless 2 / (right - left) is an integer
Ciphertext linearTransform(const HomEvaluator &eval, const Bootstrapper &btp, const Ciphertext &ctxt,
                           const InputInterval &input_interval);

// multiplier * sum_i (sum_j coeffs[bs i + j] T_j(ctxt)) * prod_k T_{2^k bs}(ctxt)^{bit k of i} for slot values in
// [-1, 1] (PolynomialEvaluator.hpp:49-63).  Uses level_cost = log_bs + log_gs levels: the blocks are rewritten over
// products of T_1, T_2, T_4, ... on the host, so that constants only ever multiply T_1.  PolynomialBasis::odd is not
// built (the reference's tables all use the basic one).
Ciphertext evaluateChebyshevExpansion(const HomEvaluator &eval, const Bootstrapper &btp, const Ciphertext &ctxt,
                                      const ChebyshevCoefficients &cheby_coeffs, const Real multiplier = 1.0);

}  // namespace Math
}  // namespace HEaaN

namespace HELLM {
namespace Exp {
// (1 + op / 2^num_iter)^(2^num_iter): num_iter + 1 levels
void exp_iter(const HEaaN::HomEvaluator &eval, const HEaaN::Bootstrapper &btp, const HEaaN::Ciphertext &op,
              HEaaN::Ciphertext &res, int num_iter);
}  // namespace Exp
namespace ReLU {
// sum over odd i of polynomial[i] ctxt^i; k baby steps (power of two), l giant-step powers ctxt^k, ctxt^2k, ...
void evalOddPolynomial(const HEaaN::HomEvaluator &eval, HEaaN::Ciphertext &ctxt, HEaaN::Ciphertext &ctxt_poly,
                       const std::vector<double> &polynomial, int k, int l);
}  // namespace ReLU
}  // namespace HELLM
