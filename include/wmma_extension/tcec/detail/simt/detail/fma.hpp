// One header serves the fp32 fragments here (reference:
// include/wmma_extension/tcec/detail/simt/detail/fma.hpp); see ../mma_simt.hpp.
#pragma once
#include "../mma_simt.hpp"
