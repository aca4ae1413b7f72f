// (reference: include/wmma_extension/tcec/detail/wmma_extension_simt_include.hpp:1-4)
#pragma once
#include "simt/mma_simt.hpp"
