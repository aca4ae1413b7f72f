// correction_scale_0 / correction_scale_1: the scale applied to the residual
// term before it is rounded, and removed when the error accumulator is folded
// back (reference: include/wmma_extension/tcec/detail/scale.hpp:8-20).  They
// are defined with the splits they belong to.
#pragma once
#include "split.hpp"
