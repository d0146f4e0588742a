// Polynomial evaluation on ciphertexts.
//   HELLM::Exp::exp_iter            reference ciphertext/src/Exp.cpp:41-52, include/HELLM/Exp.hpp
//   HELLM::ReLU::evalOddPolynomial  reference ciphertext/src/ReLU.cpp:53-188 (Han-Ki baby-step / giant-step)
//   HEaaN::Math::ChebyshevCoefficients / evaluateChebyshevExpansion
//                                   declared by the closed HEaaN-math (PolynomialEvaluator.hpp:49-63, used as
//                                   in include/HELLM/LossRemezCoeff.hpp:18-35); the algorithm here is the
//                                   textbook baby-step / giant-step evaluation in the Chebyshev basis.
// Every routine needs enough levels for its depth: bootstrapping is not part of this build, so the
// places where the reference would bootstrap raise HEaaN::RuntimeException instead.
#pragma once
#include <vector>

#include "HEaaN/HEaaN.hpp"

namespace HEaaN {
namespace Math {

struct ChebyshevCoefficients {
    std::vector<Real> coeffs;  // coefficient of T_k, k = 0 .. degree
    u64 num_baby_step;         // power of two
    ChebyshevCoefficients(std::vector<Real> c, u64 baby) : coeffs(std::move(c)), num_baby_step(baby) {}
};

// multiplier * sum_k coeffs[k] T_k(ctxt) for slot values in [-1, 1]
Ciphertext evaluateChebyshevExpansion(const HomEvaluator &eval, const Bootstrapper &btp, const Ciphertext &ctxt,
                                      const ChebyshevCoefficients &cheby_coeffs, Real multiplier = 1.0);

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
