// Operand splitting for TCEC on gfx950.
//
// An fp32 value v is represented by a short sum of 16-bit floats whose
// pairwise products are exact in fp32:
//   half        : v ~ hi + lo/2048,  hi = RN16(v), lo = RN16((v - hi) * 2048)
//                 (reference: tcec/tcec.hpp:219-223 with tcec/detail/scale.hpp:8-20)
//   bfloat16    : v ~ hi + lo            two bf16 terms, ~16 significand bits
//   precision::tf32 : v ~ hi + mid + lo  three bf16 terms, ~24 significand bits
//   float       : v itself (op_simt policy, fp32 MFMA)
// gfx950 has no xf32 MFMA; the reference's tf32 policy (two 11-bit terms,
// ~22 bits, no scaling) is replaced by the three-term bf16 split, which keeps
// fp32's exponent range and needs no scaling.
#pragma once
#include "../../detail/common.hpp"

namespace mtk {
namespace wmma {
namespace tcec {
namespace detail {

template <class T> struct split_traits;

template <> struct split_traits<mtk::wmma::half> {
  using mma_tag = mtk::wmma::half; // element tag of the MFMA operand
  using storage = _Float16;
  static constexpr int num_terms = 2;
  static constexpr float scale = 2048.f;
  static WMMAE_HD void split(const float v, storage &t0, storage &t1,
                             storage &) {
    t0 = static_cast<storage>(v);
    t1 = static_cast<storage>((v - static_cast<float>(t0)) * scale);
  }
};
#ifdef WMMAE_HAS_HIP_FP16
template <> struct split_traits<__half> : split_traits<mtk::wmma::half> {};
#endif

template <> struct split_traits<mtk::wmma::bfloat16> {
  using mma_tag = mtk::wmma::bfloat16;
  using storage = __bf16;
  static constexpr int num_terms = 2;
  static constexpr float scale = 1.f;
  static WMMAE_HD void split(const float v, storage &t0, storage &t1,
                             storage &) {
    t0 = static_cast<storage>(v);
    t1 = static_cast<storage>(v - static_cast<float>(t0));
  }
};

template <> struct split_traits<mtk::wmma::precision::tf32> {
  using mma_tag = mtk::wmma::bfloat16;
  using storage = __bf16;
  static constexpr int num_terms = 3;
  static constexpr float scale = 1.f;
  static WMMAE_HD void split(const float v, storage &t0, storage &t1,
                             storage &t2) {
    t0 = static_cast<storage>(v);
    const float r1 = v - static_cast<float>(t0);
    t1 = static_cast<storage>(r1);
    const float r2 = r1 - static_cast<float>(t1);
    t2 = static_cast<storage>(r2);
  }
};

// fp32 operands kept whole (the op_simt policy): one term, nothing to correct.
template <> struct split_traits<float> {
  using mma_tag = float;
  using storage = float;
  static constexpr int num_terms = 1;
  static constexpr float scale = 1.f;
  static WMMAE_HD void split(const float v, storage &t0, storage &,
                             storage &) {
    t0 = v;
  }
};

// split4: split() applied to four values at once (device code).  The
// arithmetic per element is that of split_traits<T>::split, arranged for the
// packed conversions of gfx950:
//   half : hi pair = v_cvt_pk_f16_f32; (v - hi) * 2048 is evaluated as
//          fma(hi, -2048, v * 2048) - v - hi and both scalings by a power of
//          two are exact, so this is the same number - by the mixed-precision
//          fma that reads hi as fp16 and writes its fp32 result rounded to one
//          half of a register (v_fma_mixlo_f16 / v_fma_mixhi_f16): five
//          instructions per two elements
//   bf16 : v_cvt_pk_bf16_f32 pairs, residuals by fp32 subtraction
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
// split2 in single instructions, for callers that place them themselves (the
// GEMM kernel that splits its own operands issues them one at a time between
// its matrix instructions):
//   split2_lead     : the leading terms                        (one instruction)
//   split2_prep<E>  : what the residual of element E is rounded from - half:
//                     the value times the scale (the mixed-precision fma
//                     subtracts); bf16: the fp32 residual, scaled (one / two)
//   split2_resid_lo : half: the residual term of element 0 into the low half
//                     of a register; bf16: nothing               (one / none)
//   split2_resid_hi : the finished pair of residual terms        (one)
template <class T, class S = typename split_traits<T>::storage,
          class S2 = S __attribute__((ext_vector_type(2)))>
WMMAE_D S2 split2_lead(const f32x2_t vv) {
  static_assert(!std::is_same<S, float>::value, "16-bit terms only");
  return __builtin_convertvector(vv, S2);
}
template <class T, int E, class S = typename split_traits<T>::storage,
          class S2 = S __attribute__((ext_vector_type(2)))>
WMMAE_D float split2_prep(const float v, const S2 h0) {
  using traits = split_traits<T>;
  if constexpr (std::is_same<S, _Float16>::value) {
    return v * traits::scale;
  } else {
    float r = v - static_cast<float>(h0[E]);
    if constexpr (traits::scale != 1.f)
      r *= traits::scale;
    return r;
  }
}
template <class T, class S = typename split_traits<T>::storage,
          class S2 = S __attribute__((ext_vector_type(2)))>
WMMAE_D S2 split2_resid_lo(const S2 h0, const float p0) {
  using traits = split_traits<T>;
  S2 h1 = {};
  if constexpr (std::is_same<S, _Float16>::value) {
    static_assert(traits::num_terms == 2, "two-term fp16 split");
    const float neg_scale = -traits::scale;
    asm("v_fma_mixlo_f16 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[1,0,0]"
        : "=v"(h1)
        : "v"(h0), "s"(neg_scale), "v"(p0));
  }
  return h1;
}
template <class T, class S = typename split_traits<T>::storage,
          class S2 = S __attribute__((ext_vector_type(2)))>
WMMAE_D S2 split2_resid_hi(S2 h1, const S2 h0, const float p0, const float p1) {
  using traits = split_traits<T>;
  if constexpr (std::is_same<S, _Float16>::value) {
    const float neg_scale = -traits::scale;
    asm("v_fma_mixhi_f16 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]"
        : "+v"(h1)
        : "v"(h0), "s"(neg_scale), "v"(p1));
    return h1;
  } else {
    return __builtin_convertvector(f32x2_t{p0, p1}, S2);
  }
}
// split2: two values -> pairs of terms (h0 leading, h1 residual, h2 second
// residual; the pairs beyond the split's number of terms are left alone)
template <class T, class S = typename split_traits<T>::storage,
          class S2 = S __attribute__((ext_vector_type(2)))>
WMMAE_D void split2(const f32x2_t vv, S2 &h0, S2 &h1, S2 &h2) {
  using traits = split_traits<T>;
  h0 = split2_lead<T>(vv);
  if constexpr (traits::num_terms >= 2) {
    const float p0 = split2_prep<T, 0>(vv[0], h0);
    const float p1 = split2_prep<T, 1>(vv[1], h0);
    h1 = split2_resid_hi<T>(split2_resid_lo<T>(h0, p0), h0, p0, p1);
    if constexpr (traits::num_terms >= 3)
      h2 = __builtin_convertvector(
          f32x2_t{p0, p1} - __builtin_convertvector(h1, f32x2_t), S2);
  }
}
template <class T, class S = typename split_traits<T>::storage>
WMMAE_D void split4(const f32x4_t v, S *const t0, S *const t1, S *const t2) {
  using traits = split_traits<T>;
  if constexpr (std::is_same<S, float>::value) {
#pragma unroll
    for (int e = 0; e < 4; e++)
      t0[e] = v[e];
  } else {
    typedef S s2_t __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int e = 0; e < 4; e += 2) {
      s2_t h0, h1, h2;
      split2<T>(f32x2_t{v[e], v[e + 1]}, h0, h1, h2);
      t0[e] = h0[0];
      t0[e + 1] = h0[1];
      if constexpr (traits::num_terms >= 2) {
        t1[e] = h1[0];
        t1[e + 1] = h1[1];
      }
      if constexpr (traits::num_terms >= 3) {
        t2[e] = h2[0];
        t2[e + 1] = h2[1];
      }
    }
  }
}

// Scale applied to the residual before rounding it (0) and removed when the
// error accumulator is folded back (1) (reference: tcec/detail/scale.hpp:8-20).
template <class T> WMMAE_HD float correction_scale_0(const float v) {
  return v * split_traits<T>::scale;
}
template <class T> WMMAE_HD float correction_scale_1(const float v) {
  return v / split_traits<T>::scale;
}

} // namespace detail
} // namespace tcec
} // namespace wmma
} // namespace mtk
