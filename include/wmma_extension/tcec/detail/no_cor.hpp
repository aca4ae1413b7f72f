// The without_ec policy (reference: include/wmma_extension/tcec/detail/no_cor.hpp:13-897,
// a second copy of every TCEC function for fragments without the residual
// terms).  Here one policy-generic set of templates in tcec.hpp serves both
// policies, so this header only brings that in.
#pragma once
#include "../tcec.hpp"
