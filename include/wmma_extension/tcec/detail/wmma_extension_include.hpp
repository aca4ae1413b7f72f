// The primitive layer the TCEC headers stand on
// (reference: include/wmma_extension/tcec/detail/wmma_extension_include.hpp:3-4).
#pragma once
#include "../../wmma_extension.hpp"
#include "../../wmma_mma.hpp"
