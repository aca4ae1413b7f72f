// Fragment operators (reference: include/wmma_extension/detail/operators.hpp,
// the per-type helpers behind operators.hpp) are written once, in
// operators.hpp itself.
#pragma once
#include "../operators.hpp"
