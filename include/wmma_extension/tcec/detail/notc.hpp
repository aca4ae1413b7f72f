// The fp32 policy op_simt (reference: include/wmma_extension/tcec/detail/notc.hpp:12-779,
// a third copy of every TCEC function for fp32 fragments on the SIMT cores).
// Here the generic templates in tcec.hpp cover it through split_traits<float>
// and the fp32 matrix instruction, so this header only brings that in.
#pragma once
#include "../tcec.hpp"
