// tcec::print_fragment (reference: include/wmma_extension/tcec/detail/print.hpp:11-55)
// is defined in tcec.hpp beside the fragment it prints.
#pragma once
#include "../tcec.hpp"
