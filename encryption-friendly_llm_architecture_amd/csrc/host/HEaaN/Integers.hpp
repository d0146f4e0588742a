// Forwarding header: the whole HEaaN-compatible surface is declared in HEaaN/HEaaN.hpp.
#pragma once
#include "HEaaN/HEaaN.hpp"
