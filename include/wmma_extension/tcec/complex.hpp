// Complex TCEC: a complex matrix fragment is a pair of real TCEC fragments and a
// complex product is four real ones (reference:
// include/wmma_extension/tcec/complex.hpp:9-17 fragment_complex, :19-36 fills,
// :136-390 loads, :393-602 stores, :604-727 products; docs/mma_f32.md:154-160).
//
// Memory holds interleaved (re, im) pairs.  The reference spells the element
// type cuComplex; here every loader and store takes any type with float
// members .x (real) and .y (imaginary) - hipFloatComplex, float2, or
// tcec::complex_t below - so no vendor complex header is needed.
#pragma once
#include "tcec.hpp"

namespace mtk {
namespace wmma {
namespace tcec {

// Plain interleaved single-precision complex number.
struct complex_t {
  float x, y;
};

template <class Use, int m, int n, int k, class T, class Layout = void,
          class Policy_ = typename detail::default_policy<T>::type>
struct fragment_complex {
  using frag_t = fragment<Use, m, n, k, T, Layout, Policy_>;
  static constexpr unsigned num_sub_frag_m = frag_t::num_sub_frag_m;
  static constexpr unsigned num_sub_frag_n = frag_t::num_sub_frag_n;
  frag_t real, imag;
};

#define WMMAE_TCEC_TPARAMS                                                     \
  int m, int n, int k, class T, class Op, class EC, int fm, int fn, int fk
#define WMMAE_TCEC_CFRAG(Use, Layout)                                          \
  fragment_complex<Use, m, n, k, T, Layout, Policy<Op, EC, fm, fn, fk>>

// ------------------------------------------------------------------- fills
template <class Use, WMMAE_TCEC_TPARAMS, class Layout>
WMMAE_D void fill_fragment(WMMAE_TCEC_CFRAG(Use, Layout) & frag,
                           const float real, const float imag = 0.f) {
  fill_fragment(frag.real, real);
  fill_fragment(frag.imag, imag);
}
template <class Use, WMMAE_TCEC_TPARAMS, class Layout>
WMMAE_D void fill_zero(WMMAE_TCEC_CFRAG(Use, Layout) & frag) {
  fill_zero(frag.real);
  fill_zero(frag.imag);
}

// ------------------------------------------------------------------- loads
// MatrixLayout is the layout of the memory being read.  Operands are split
// while loading, component by component; accumulators take the fp32 values
// and a zero error part.
template <class MatrixLayout, class Use, WMMAE_TCEC_TPARAMS, class Layout,
          class CPLX>
WMMAE_D void load_matrix_sync_with_mul(WMMAE_TCEC_CFRAG(Use, Layout) & frag,
                                       const CPLX *const ptr,
                                       const unsigned ldm, const float mul,
                                       const bool = true) {
  using F = typename WMMAE_TCEC_CFRAG(Use, Layout)::frag_t;
  constexpr unsigned bm_size = detail::select_value<Use, fm, fk, fm>::value;
  constexpr unsigned bn_size = detail::select_value<Use, fk, fn, fn>::value;
  mtk::wmma::foreach_ij<typename F::sub_frag_t>(
      [&](const unsigned *list, const unsigned, const unsigned i,
          const unsigned j) {
#pragma unroll
        for (unsigned bm = 0; bm < unsigned(F::num_sub_frag_m); bm++) {
#pragma unroll
          for (unsigned bn = 0; bn < unsigned(F::num_sub_frag_n); bn++) {
            const unsigned off = detail::mem_offset<MatrixLayout>(
                i, j, ldm, bm * bm_size, bn * bn_size);
            const unsigned block = bm + F::num_sub_frag_m * bn;
            const CPLX cv = ptr[off];
            const float re = static_cast<float>(cv.x) * mul;
            const float im = static_cast<float>(cv.y) * mul;
            if constexpr (F::is_acc) {
              frag.real.sub_frag[block].x[list[0]] = re;
              frag.imag.sub_frag[block].x[list[0]] = im;
              if constexpr (F::num_terms >= 2) {
                frag.real.sub_d_frag[block].x[list[0]] = 0.f;
                frag.imag.sub_d_frag[block].x[list[0]] = 0.f;
              }
            } else {
              detail::put_split(frag.real, block, list[0], re);
              detail::put_split(frag.imag, block, list[0], im);
            }
          }
        }
      });
}
template <class MatrixLayout, class Use, WMMAE_TCEC_TPARAMS, class Layout,
          class CPLX>
WMMAE_D void load_matrix_sync(WMMAE_TCEC_CFRAG(Use, Layout) & frag,
                              const CPLX *const ptr, const unsigned ldm,
                              const bool sync = true) {
  load_matrix_sync_with_mul<MatrixLayout>(frag, ptr, ldm, 1.f, sync);
}
// Memory layout = the fragment's own Layout (operands only).
template <class Use, WMMAE_TCEC_TPARAMS, class Layout, class CPLX>
WMMAE_D void load_matrix_sync(WMMAE_TCEC_CFRAG(Use, Layout) & frag,
                              const CPLX *const ptr, const unsigned ldm,
                              const bool sync = true) {
  static_assert(!std::is_same<Use, accumulator>::value,
                "accumulator loads need a layout");
  load_matrix_sync<Layout>(frag, ptr, ldm, sync);
}
template <class Use, WMMAE_TCEC_TPARAMS, class Layout, class CPLX>
WMMAE_D void load_matrix_sync_with_mul(WMMAE_TCEC_CFRAG(Use, Layout) & frag,
                                       const CPLX *const ptr,
                                       const unsigned ldm, const float mul,
                                       const bool sync = true) {
  static_assert(!std::is_same<Use, accumulator>::value,
                "accumulator loads need a layout");
  load_matrix_sync_with_mul<Layout>(frag, ptr, ldm, mul, sync);
}
// Accumulators with a run-time layout.
template <WMMAE_TCEC_TPARAMS, class CPLX>
WMMAE_D void load_matrix_sync(WMMAE_TCEC_CFRAG(accumulator, void) & frag,
                              const CPLX *const ptr, const unsigned ldm,
                              const layout_t layout, const bool sync = true) {
  if (layout == mem_col_major)
    load_matrix_sync<col_major>(frag, ptr, ldm, sync);
  else
    load_matrix_sync<row_major>(frag, ptr, ldm, sync);
}

// ------------------------------------------------------------------ stores
// ptr[off] = (main + err/scale) of each component, times mul.
template <class Layout, WMMAE_TCEC_TPARAMS, class CPLX>
WMMAE_D void
store_matrix_sync_with_mul(CPLX *const ptr,
                           const WMMAE_TCEC_CFRAG(accumulator, void) & frag,
                           const unsigned ldm, const float mul,
                           const bool = true) {
  using F = typename WMMAE_TCEC_CFRAG(accumulator, void)::frag_t;
  mtk::wmma::foreach_ij<typename F::sub_frag_t>(
      [&](const unsigned *list, const unsigned, const unsigned i,
          const unsigned j) {
#pragma unroll
        for (unsigned bm = 0; bm < unsigned(F::num_sub_frag_m); bm++) {
#pragma unroll
          for (unsigned bn = 0; bn < unsigned(F::num_sub_frag_n); bn++) {
            const unsigned off =
                detail::mem_offset<Layout>(i, j, ldm, bm * fm, bn * fn);
            const unsigned block = bm + F::num_sub_frag_m * bn;
            CPLX c;
            c.x = detail::combined(frag.real, block, list[0]) * mul;
            c.y = detail::combined(frag.imag, block, list[0]) * mul;
            ptr[off] = c;
          }
        }
      });
}
template <class Layout, WMMAE_TCEC_TPARAMS, class CPLX>
WMMAE_D void store_matrix_sync(CPLX *const ptr,
                               const WMMAE_TCEC_CFRAG(accumulator, void) & frag,
                               const unsigned ldm, const bool sync = true) {
  store_matrix_sync_with_mul<Layout>(ptr, frag, ldm, 1.f, sync);
}
// The reference spells the scaled store as an overload of store_matrix_sync
// (complex.hpp:501-602); both spellings are provided.
template <class Layout, WMMAE_TCEC_TPARAMS, class CPLX>
WMMAE_D void store_matrix_sync(CPLX *const ptr,
                               const WMMAE_TCEC_CFRAG(accumulator, void) & frag,
                               const unsigned ldm, const float mul,
                               const bool sync = true) {
  store_matrix_sync_with_mul<Layout>(ptr, frag, ldm, mul, sync);
}
template <WMMAE_TCEC_TPARAMS, class CPLX>
WMMAE_D void store_matrix_sync(CPLX *const ptr,
                               const WMMAE_TCEC_CFRAG(accumulator, void) & frag,
                               const unsigned ldm, const layout_t layout,
                               const bool sync = true) {
  if (layout == mem_col_major)
    store_matrix_sync<col_major>(ptr, frag, ldm, sync);
  else
    store_matrix_sync<row_major>(ptr, frag, ldm, sync);
}
template <WMMAE_TCEC_TPARAMS, class CPLX>
WMMAE_D void store_matrix_sync(CPLX *const ptr,
                               const WMMAE_TCEC_CFRAG(accumulator, void) & frag,
                               const unsigned ldm, const float mul,
                               const layout_t layout, const bool sync = true) {
  if (layout == mem_col_major)
    store_matrix_sync_with_mul<col_major>(ptr, frag, ldm, mul, sync);
  else
    store_matrix_sync_with_mul<row_major>(ptr, frag, ldm, mul, sync);
}

// ---------------------------------------------------------------- products
// (a.re + i a.im)(b.re + i b.im) + c, as four real TCEC products in the
// reference's order (complex.hpp:609-641): re = a.re b.re + c.re, im = a.im
// b.re + c.im, im += a.re b.im, re += a.im (-b.im).
namespace detail {
enum class rounding { standard, rn, rz };
template <rounding R, class D, class A, class B, class C>
WMMAE_D void real_mma(D &d, const A &a, const B &b, const C &c) {
  if constexpr (R == rounding::rn)
    mma_rn_sync(d, a, b, c);
  else if constexpr (R == rounding::rz)
    mma_rz_sync(d, a, b, c);
  else
    mma_sync(d, a, b, c);
}
template <rounding R, class D, class A, class B>
WMMAE_D void real_mma(D &d, const A &a, const B &b) {
  if constexpr (R == rounding::rn)
    mma_rn_sync(d, a, b);
  else if constexpr (R == rounding::rz)
    mma_rz_sync(d, a, b);
  else
    mma_sync(d, a, b);
}
template <rounding R, class D, class A, class B, class C>
WMMAE_D void complex_mma(D &d, const A &a, const B &b, const C &c) {
  real_mma<R>(d.real, a.real, b.real, c.real);
  real_mma<R>(d.imag, a.imag, b.real, c.imag);
  real_mma<R>(d.imag, a.real, b.imag, d.imag);
  real_mma<R>(d.real, a.imag, neg(b.imag), d.real);
}
template <rounding R, class D, class A, class B>
WMMAE_D void complex_mma(D &d, const A &a, const B &b) {
  real_mma<R>(d.imag, a.imag, b.real);
  real_mma<R>(d.imag, a.real, b.imag, d.imag);
  real_mma<R>(d.real, a.real, b.real);
  real_mma<R>(d.real, a.imag, neg(b.imag), d.real);
}
} // namespace detail

#define WMMAE_TCEC_COMPLEX_MMA(NAME, R)                                        \
  template <WMMAE_TCEC_TPARAMS, class LA, class LB>                            \
  WMMAE_D void NAME(WMMAE_TCEC_CFRAG(accumulator, void) & d,                   \
                    const WMMAE_TCEC_CFRAG(matrix_a, LA) & a,                  \
                    const WMMAE_TCEC_CFRAG(matrix_b, LB) & b,                  \
                    const WMMAE_TCEC_CFRAG(accumulator, void) & c) {           \
    detail::complex_mma<detail::rounding::R>(d, a, b, c);                      \
  }                                                                            \
  template <WMMAE_TCEC_TPARAMS, class LA, class LB>                            \
  WMMAE_D void NAME(WMMAE_TCEC_CFRAG(accumulator, void) & d,                   \
                    const WMMAE_TCEC_CFRAG(matrix_a, LA) & a,                  \
                    const WMMAE_TCEC_CFRAG(matrix_b, LB) & b) {                \
    detail::complex_mma<detail::rounding::R>(d, a, b);                         \
  }
WMMAE_TCEC_COMPLEX_MMA(mma_sync, standard)
WMMAE_TCEC_COMPLEX_MMA(mma_rn_sync, rn)
WMMAE_TCEC_COMPLEX_MMA(mma_rz_sync, rz)
#undef WMMAE_TCEC_COMPLEX_MMA

#undef WMMAE_TCEC_TPARAMS
#undef WMMAE_TCEC_CFRAG

} // namespace tcec
} // namespace wmma
} // namespace mtk
