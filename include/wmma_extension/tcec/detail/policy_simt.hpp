// op_simt and default_policy<float, without_ec, op_simt>
// (reference: include/wmma_extension/tcec/detail/policy_simt.hpp:14-27) are
// defined with the other policies.
#pragma once
#include "policy.hpp"
