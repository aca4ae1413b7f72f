// The function objects of the op_simt policy
// (reference: include/wmma_extension/tcec/detail/functions_simt.hpp:10-177):
// the templates in functions.hpp are generic in the policy and serve it too.
#pragma once
#include "functions.hpp"
