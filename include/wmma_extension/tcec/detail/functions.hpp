// Policy-dispatched function objects over the sub-fragment primitives
// (reference: include/wmma_extension/tcec/detail/functions.hpp:10-348, where
// every functor has one specialisation per instruction family, op_wmma and
// op_mma).  gfx950 has one matrix instruction family, so each functor is a
// single template: the policy only selects the sub-fragment type
// (default_fragment: element type T for op_mfma, float for op_simt) and its
// m, n, k.  Code that reached into tcec::detail for these names keeps
// compiling; tcec.hpp itself calls the primitives directly.
#pragma once
#include "policy.hpp"

namespace mtk {
namespace wmma {
namespace tcec {
namespace detail {

template <class Use, class T, class Layout, class Policy>
using policy_fragment_t =
    typename default_fragment<Use, T, Layout, Policy>::type;

template <class Use, class T, class Layout, class Policy>
struct foreach_wrapper {
  using frag_t = policy_fragment_t<Use, T, Layout, Policy>;
  template <class Func> WMMAE_D void operator()(Func func) {
    mtk::wmma::foreach<frag_t>(func);
  }
  template <class Func>
  WMMAE_D void operator()(const layout_t layout, Func func) {
    mtk::wmma::foreach<frag_t>(layout, func);
  }
};

template <class Use, class T, class Layout, class Policy>
struct foreach_ij_wrapper {
  using frag_t = policy_fragment_t<Use, T, Layout, Policy>;
  template <class Func> WMMAE_D void operator()(Func func) {
    mtk::wmma::foreach_ij<frag_t>(func);
  }
  template <class Func>
  WMMAE_D void operator()(const layout_t layout, Func func) {
    mtk::wmma::foreach_ij<frag_t>(layout, func);
  }
};

template <class Use, class T, class Layout, class Policy>
struct foreach_v_wrapper {
  using frag_t = policy_fragment_t<Use, T, Layout, Policy>;
  template <class Func> WMMAE_D void operator()(Func func) {
    mtk::wmma::foreach_v<frag_t>(func);
  }
  template <class Func>
  WMMAE_D void operator()(const layout_t layout, Func func) {
    mtk::wmma::foreach_v<frag_t>(layout, func);
  }
};

template <class Use, class T, class Layout, class Policy>
struct fill_zero_wrapper {
  WMMAE_D void operator()(policy_fragment_t<Use, T, Layout, Policy> &frag) {
    mtk::wmma::fill_zero(frag);
  }
};

template <class Use, class T, class Layout, class Policy, class VT>
struct fill_fragment_wrapper {
  WMMAE_D void operator()(policy_fragment_t<Use, T, Layout, Policy> &frag,
                          const VT v) {
    mtk::wmma::fill_fragment(frag, v);
  }
};

template <class Use, class T, class Layout, class Policy>
struct load_matrix_sync_wrapper {
  using frag_t = policy_fragment_t<Use, T, Layout, Policy>;
  WMMAE_D void operator()(frag_t &frag, const float *const ptr,
                          const unsigned ldm, const layout_t layout) {
    mtk::wmma::load_matrix_sync(frag, ptr, ldm, layout);
  }
  WMMAE_D void operator()(frag_t &frag, const float *const ptr,
                          const unsigned ldm) {
    mtk::wmma::load_matrix_sync(frag, ptr, ldm);
  }
};

template <class T, class Policy> struct store_matrix_sync_wrapper {
  WMMAE_D void
  operator()(float *const ptr,
             policy_fragment_t<accumulator, float, void, Policy> &frag,
             const unsigned ldm, const layout_t layout) {
    mtk::wmma::store_matrix_sync(ptr, frag, ldm, layout);
  }
};

template <class Use, class T, class Layout, class Policy>
struct load_vector_wrapper {
  using frag_t = policy_fragment_t<Use, T, Layout, Policy>;
  WMMAE_D void operator()(frag_t &frag, const float *const ptr,
                          const layout_t layout) {
    mtk::wmma::load_vector(frag, ptr, layout);
  }
  WMMAE_D void operator()(frag_t &frag, const float *const ptr) {
    mtk::wmma::load_vector(frag, ptr);
  }
};

template <class Use, class T, class Layout, class Policy>
struct store_vector_wrapper {
  WMMAE_D void operator()(float *const ptr,
                          policy_fragment_t<Use, T, Layout, Policy> &frag,
                          const layout_t layout) {
    mtk::wmma::store_vector(ptr, frag, layout);
  }
};

template <class AB_T, class A_Layout, class B_Layout, class CD_T, class Policy>
struct mma_sync_wrapper {
  using Fragment_A = policy_fragment_t<matrix_a, AB_T, A_Layout, Policy>;
  using Fragment_B = policy_fragment_t<matrix_b, AB_T, B_Layout, Policy>;
  using Fragment_C = policy_fragment_t<accumulator, CD_T, void, Policy>;
  WMMAE_D void operator()(Fragment_C &d, const Fragment_A &a,
                          const Fragment_B &b, const Fragment_C &c) {
    mtk::wmma::mma_sync(d, a, b, c);
  }
};

} // namespace detail
} // namespace tcec
} // namespace wmma
} // namespace mtk
