// HEaaN-math/HEaaN-math.hpp of the reference resolves here.
#pragma once
#include "HELLM/PolyEval.hpp"
