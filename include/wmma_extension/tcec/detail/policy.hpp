// TCEC policies for gfx950.
//
// Keeps the reference's compile-time configuration surface
// (reference: include/wmma_extension/tcec/detail/policy.hpp:12-125):
// Policy<Op, ErrorCorrection, m, n, k>, default_policy<T, EC, Op, Sm>,
// the with_ec / without_ec tags and their older spellings.  There is one
// matrix instruction family on gfx950, so op_mma and op_wmma both name the
// MFMA backend, and the default instruction shape is 16x16x32.
#pragma once
#include "../../wmma_extension.hpp"

namespace mtk {
namespace wmma {
namespace tcec {

// Instruction policy
struct op_mfma;
using op_mma = op_mfma;
using op_wmma = op_mfma;
// Plain fp32 operands, no split (reference: tcec/detail/policy_simt.hpp:14,
// docs/mma_f32.md:139-152, where this policy runs on the SIMT cores with
// warp shuffles).  On gfx950 the matrix core has an fp32 path
// (v_mfma_f32_16x16x4_f32) at the rate of the vector ALUs, so the policy keeps
// its name and its 16x16x16 shape but issues four fp32 MFMAs per sub-block.
struct op_simt;
using op_fp32 = op_simt;

// Error correction policy
struct with_ec;
struct without_ec;
using op_with_error_correction = with_ec;
using op_without_error_correction = without_ec;

// Architecture tag (the reference selects per-SM tables with it; one value here).
struct gfx950;
using sm_auto = gfx950;

template <class Op, class ErrorCorrection, int m_, int n_, int k_>
struct Policy {
  using op = Op;
  using error_correction = ErrorCorrection;
  static constexpr int m = m_;
  static constexpr int n = n_;
  static constexpr int k = k_;
};

namespace detail {
template <class T, class ErrorCorrection = with_ec, class Op = op_mfma,
          class Sm = sm_auto>
struct default_policy {
  using type = Policy<op_mfma, ErrorCorrection, 16, 16, 32>;
};

// default_policy<float, without_ec, op_simt>::type
// (reference: tcec/detail/policy_simt.hpp:21-27)
template <class T, class Sm>
struct default_policy<T, without_ec, op_simt, Sm> {
  using type = Policy<op_simt, without_ec, 16, 16, 16>;
};

template <class Use, class T, class Layout, class Policy>
struct default_fragment;
template <class Use, class T, class Layout, class ErrorCorrection, int fm,
          int fn, int fk>
struct default_fragment<Use, T, Layout,
                        Policy<op_simt, ErrorCorrection, fm, fn, fk>> {
  using type = mtk::wmma::fragment<Use, fm, fn, fk, float, Layout>;
};
template <class Use, class T, class Layout, class ErrorCorrection, int fm,
          int fn, int fk>
struct default_fragment<Use, T, Layout,
                        Policy<op_mfma, ErrorCorrection, fm, fn, fk>> {
  using type = mtk::wmma::fragment<Use, fm, fn, fk, T, Layout>;
};
} // namespace detail

template <class T, class ErrorCorrection = with_ec, class Op = op_mfma,
          class Sm = sm_auto>
using default_policy = detail::default_policy<T, ErrorCorrection, Op, Sm>;

} // namespace tcec
} // namespace wmma
} // namespace mtk
