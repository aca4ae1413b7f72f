// Elementwise arithmetic on fragments (reference:
// include/wmma_extension/operators.hpp:6-58, detail/operators.hpp,
// docs/ops.md): a + b, a - b, a * s, a / s, fma(s, a, b) = s*a + b and
// fma(a, s, b) = a + s*b, where s has the fragment's storage element type.
//
// Every result element is the correctly rounded result in the fragment's
// element type: half uses native fp16 arithmetic (fp16 fused multiply-add for
// fma), float uses fp32, bfloat16 goes through fp32 and is rounded once at
// the end (its fma is an fp32 fma followed by one rounding to bf16).  The
// operators live in mtk::wmma and are found by argument-dependent lookup.
#pragma once
#include "detail/common.hpp"

namespace mtk {
namespace wmma {
namespace ops {
// arithmetic type an element type computes in
template <class S> struct compute_type {
  using type = float;
};
template <> struct compute_type<_Float16> {
  using type = _Float16;
};
template <class S> WMMAE_HD S fma_elem(const S a, const S b, const S c) {
  using C = typename compute_type<S>::type;
  if constexpr (std::is_same<C, _Float16>::value)
    return __builtin_fmaf16(a, b, c);
  else
    return static_cast<S>(__builtin_fmaf(static_cast<float>(a),
                                         static_cast<float>(b),
                                         static_cast<float>(c)));
}
} // namespace ops

#define WMMAE_FRAG fragment<Use, M, N, K, Type, Layout>
#define WMMAE_FRAG_TPARAMS                                                     \
  class Use, int M, int N, int K, class Type, class Layout

template <WMMAE_FRAG_TPARAMS>
WMMAE_D WMMAE_FRAG operator+(const WMMAE_FRAG &a, const WMMAE_FRAG &b) {
  using S = typename WMMAE_FRAG::storage_element_type;
  using C = typename ops::compute_type<S>::type;
  WMMAE_FRAG res;
#pragma unroll
  for (unsigned i = 0; i < res.num_elements; i++)
    res.x[i] = static_cast<S>(static_cast<C>(a.x[i]) + static_cast<C>(b.x[i]));
  return res;
}
template <WMMAE_FRAG_TPARAMS>
WMMAE_D WMMAE_FRAG operator-(const WMMAE_FRAG &a, const WMMAE_FRAG &b) {
  using S = typename WMMAE_FRAG::storage_element_type;
  using C = typename ops::compute_type<S>::type;
  WMMAE_FRAG res;
#pragma unroll
  for (unsigned i = 0; i < res.num_elements; i++)
    res.x[i] = static_cast<S>(static_cast<C>(a.x[i]) - static_cast<C>(b.x[i]));
  return res;
}
template <WMMAE_FRAG_TPARAMS>
WMMAE_D WMMAE_FRAG
operator*(const WMMAE_FRAG &a,
          const typename WMMAE_FRAG::storage_element_type b) {
  using S = typename WMMAE_FRAG::storage_element_type;
  using C = typename ops::compute_type<S>::type;
  WMMAE_FRAG res;
#pragma unroll
  for (unsigned i = 0; i < res.num_elements; i++)
    res.x[i] = static_cast<S>(static_cast<C>(a.x[i]) * static_cast<C>(b));
  return res;
}
template <WMMAE_FRAG_TPARAMS>
WMMAE_D WMMAE_FRAG
operator/(const WMMAE_FRAG &a,
          const typename WMMAE_FRAG::storage_element_type b) {
  using S = typename WMMAE_FRAG::storage_element_type;
  using C = typename ops::compute_type<S>::type;
  WMMAE_FRAG res;
#pragma unroll
  for (unsigned i = 0; i < res.num_elements; i++)
    res.x[i] = static_cast<S>(static_cast<C>(a.x[i]) / static_cast<C>(b));
  return res;
}

// alpha * a + b
template <WMMAE_FRAG_TPARAMS>
WMMAE_D WMMAE_FRAG fma(const typename WMMAE_FRAG::storage_element_type alpha,
                       const WMMAE_FRAG &a, const WMMAE_FRAG &b) {
  WMMAE_FRAG res;
#pragma unroll
  for (unsigned i = 0; i < res.num_elements; i++)
    res.x[i] = ops::fma_elem(alpha, a.x[i], b.x[i]);
  return res;
}
// a + alpha * b (reference: operators.hpp:50-58 forwards (alpha, b, a); its
// test labels the overload "fma(A+a*B)", test/primitive/operators.cu:211-225)
template <WMMAE_FRAG_TPARAMS>
WMMAE_D WMMAE_FRAG fma(const WMMAE_FRAG &a,
                       const typename WMMAE_FRAG::storage_element_type alpha,
                       const WMMAE_FRAG &b) {
  return fma(alpha, b, a);
}

#undef WMMAE_FRAG
#undef WMMAE_FRAG_TPARAMS
} // namespace wmma
} // namespace mtk
