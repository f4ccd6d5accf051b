// Same include path as the reference's src/benchmark/competitor.hpp.
#pragma once
#include "../../sddmm_competitor.hpp"
