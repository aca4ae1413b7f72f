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

template <class Use, class T, class Layout, class Policy>
struct default_fragment;
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
