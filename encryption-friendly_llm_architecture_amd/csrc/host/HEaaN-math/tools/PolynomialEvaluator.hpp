// HEaaN-math/tools/PolynomialEvaluator.hpp of the reference resolves here.
#pragma once
#include "HELLM/PolyEval.hpp"
