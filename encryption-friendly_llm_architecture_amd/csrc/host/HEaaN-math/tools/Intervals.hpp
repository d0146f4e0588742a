// HEaaN-math/tools/Intervals.hpp of the reference resolves here.
#pragma once
#include "HELLM/PolyEval.hpp"
