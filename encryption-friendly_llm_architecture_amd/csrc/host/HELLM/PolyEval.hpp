// Polynomial evaluation on ciphertexts.
//   HELLM::Exp::exp_iter            reference ciphertext/src/Exp.cpp:41-52, include/HELLM/Exp.hpp
//   HELLM::Exp::exp_iter_Parallel   reference ciphertext/src/Exp.cpp:55-77 (called by HEMMer::expParallelInplace,
//                                   src/HEMMer.cpp:1416, with 14 iterations on the six score tensors of a layer)
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
#include "HELLM/HETensor.hpp"

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

// The coefficient holder HEaaN-math declares (tools/PolynomialEvaluator.hpp:19-40): member names and constructor
// arguments are that interface, so callers written against it compile.  The coefficients are NOT a plain Chebyshev
// series: entry bs * i + j multiplies T_j times the product of T_{2^k bs} over the set bits k of i (the tables of
// include/HELLM/*RemezCoeff.hpp are stored that way).  Derived sizes: the table is cut into blocks of num_bs entries
// (all of it when no block size is given), num_gs blocks in all; a block needs ceil(log2 num_bs) levels, combining
// the blocks ceil(log2 num_gs) more.
enum PolynomialBasis { basic, odd };
struct ChebyshevCoefficients {
    static u64 ceilLog2(u64 v) {
        u64 bits = 0;
        while ((u64(1) << bits) < v) bits++;
        return bits;
    }
    ChebyshevCoefficients(std::vector<Real> coefficient, u64 num_baby_step, PolynomialBasis base = PolynomialBasis::basic)
        : coeffs{std::move(coefficient)}, basis{base} {
        const u64 n = coeffs.size();
        num_bs = num_baby_step != 0 ? num_baby_step : n;
        num_gs = num_bs != 0 ? (n + num_bs - 1) / num_bs : 0;
        log_bs = ceilLog2(num_bs);
        log_gs = ceilLog2(num_gs);
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
// The same on every tensor of op, in place, the squarings interleaved pair by pair: tensors 2j and 2j+1 are squared
// together in each of the num_iter rounds, and a pair that has reached the bootstrap level is first merged into one
// complex ciphertext and bootstrapped as one (here: raises).  As in the reference, a trailing tensor without a partner
// is scaled and shifted but never squared.
void exp_iter_Parallel(const HEaaN::HomEvaluator &eval, const HEaaN::Bootstrapper &btp, std::vector<HELLM::CtxtTensor> &op,
                       int num_iter);
}  // namespace Exp
namespace ReLU {
// sum over odd i of polynomial[i] ctxt^i; k baby steps (power of two), l giant-step powers ctxt^k, ctxt^2k, ...
void evalOddPolynomial(const HEaaN::HomEvaluator &eval, HEaaN::Ciphertext &ctxt, HEaaN::Ciphertext &ctxt_poly,
                       const std::vector<double> &polynomial, int k, int l);
}  // namespace ReLU
}  // namespace HELLM
