// mtk::wmma::mma_simt - the fragment namespace behind the reference's op_simt
// policy (reference: include/wmma_extension/tcec/detail/simt/mma_simt.hpp:9-262,
// simt/detail/m16n16k16.hpp:50-356: 16x16x16 fragments of fp32 values held by
// the lanes of a warp and multiplied with fused multiply-adds on the SIMT
// cores, 15 shuffle rounds per product).
//
// gfx950 multiplies fp32 fragments on the matrix core itself
// (v_mfma_f32_16x16x4_f32, four chained per 16x16x16 product: detail/mfma.hpp),
// in the one register layout all fragments of this library share.  So this
// namespace re-exports the plain fragment types and primitives, the way
// mtk::wmma::mma does (wmma_mma.hpp); code written against
// mtk::wmma::mma_simt::fragment<Use, 16, 16, 16, float, Layout> and its
// foreach / load / store / mma functions compiles and runs on the matrix core.
#pragma once
#include "../../../wmma_extension.hpp"

namespace mtk {
namespace wmma {
namespace mma_simt {
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

namespace detail {
// c + a * b on values of any of the fragment element types, in fp32 (double
// stays double), fused: the scalar the reference builds its products from
// (simt/detail/fma.hpp:10-24).
template <class A_T, class B_T, class C_T> struct fma {
  WMMAE_D C_T operator()(const A_T a, const B_T b, const C_T c) const {
    return mtk::wmma::detail::common::cast<C_T>(
        __builtin_fmaf(mtk::wmma::detail::common::cast<float>(a),
                       mtk::wmma::detail::common::cast<float>(b),
                       mtk::wmma::detail::common::cast<float>(c)));
  }
};
template <> struct fma<double, double, double> {
  WMMAE_D double operator()(const double a, const double b,
                            const double c) const {
    return __builtin_fma(a, b, c);
  }
};
} // namespace detail
} // namespace mma_simt
} // namespace wmma
} // namespace mtk
