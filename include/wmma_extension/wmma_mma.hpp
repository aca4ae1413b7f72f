// mtk::wmma::mma — the second fragment namespace of the reference.
//
// On NVIDIA the reference keeps two register layouts apart: the CUDA WMMA
// fragments (mtk::wmma::*) and the PTX mma.sync fragments (mtk::wmma::mma::*,
// reference: include/wmma_extension/wmma_mma.hpp:12-231).  gfx950 has one
// matrix instruction family and one layout, so this namespace re-exports the
// same types and functions; code written against either spelling compiles.
#pragma once
#include "wmma_extension.hpp"

namespace mtk {
namespace wmma {
namespace mma {
template <class Use, int M, int N, int K, class T, class Layout = void>
using fragment = mtk::wmma::fragment<Use, M, N, K, T, Layout>;

using mtk::wmma::fill_fragment;
using mtk::wmma::fill_zero;
using mtk::wmma::foreach;
using mtk::wmma::foreach_ij;
using mtk::wmma::foreach_v;
using mtk::wmma::load_matrix_sync;
using mtk::wmma::load_vector;
using mtk::wmma::map;
using mtk::wmma::mma_sync;
using mtk::wmma::print_fragment;
using mtk::wmma::store_matrix_sync;
using mtk::wmma::store_vector;
} // namespace mma
} // namespace wmma
} // namespace mtk
