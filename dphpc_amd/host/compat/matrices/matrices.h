// Same include path as the reference's src/matrices/matrices.h.
#pragma once
#include "../../sddmm_containers.hpp"
