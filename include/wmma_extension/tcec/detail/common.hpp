// Compile-time helpers of the TCEC layer
// (reference: include/wmma_extension/tcec/detail/common.hpp:12-82):
// select_value, get_fragment_k, compute_mem_offset, sub_frag_t, layout_switch.
#pragma once
#include "../../detail/common.hpp"
#include <type_traits>

namespace mtk {
namespace wmma {
namespace tcec {
namespace detail {

// select_value<Use, a, b, c>::value = a / b / c for matrix_a / matrix_b /
// accumulator (reference: tcec/detail/common.hpp:12-24)
using mtk::wmma::detail::common::select_value;

// k of the matrix instruction the default policy of element tag T uses
// (reference: tcec/detail/common.hpp:26-30, 16 for half and 8 for tf32 on the
// reference's hardware).  The fp16/bf16 default here is
// v_mfma_f32_16x16x32; fp32 operands (op_simt) take the 16x16x16 shape.
template <class T> WMMAE_HD constexpr int get_fragment_k() { return 32; }
template <> WMMAE_HD constexpr int get_fragment_k<float>() { return 16; }

template <class Layout, int a, int b> struct layout_switch;
template <int a, int b> struct layout_switch<col_major, a, b> {
  static constexpr int value = a;
};
template <int a, int b> struct layout_switch<row_major, a, b> {
  static constexpr int value = b;
};

// Memory offset of element (i,j) of the sub-block at (m_offset, n_offset)
// (reference: tcec/detail/common.hpp:32-63).
template <class Layout>
WMMAE_HD unsigned mem_offset(const unsigned i, const unsigned j,
                             const unsigned ldm, const unsigned m_offset,
                             const unsigned n_offset) {
  if constexpr (std::is_same<Layout, col_major>::value)
    return (i + m_offset) + (j + n_offset) * ldm;
  else
    return (j + n_offset) + (i + m_offset) * ldm;
}

// The same offsets as function objects under the reference's name
// (tcec/detail/common.hpp:32-63): from the mem_index a foreach callback
// receives for a frag_m x frag_n sub-block, or from a position (i, j).
template <int frag_m, int frag_n, class Layout> struct compute_mem_offset {
  WMMAE_HD unsigned operator()(const unsigned mem_index, const unsigned ldm,
                               const unsigned m_offset,
                               const unsigned n_offset) const {
    constexpr unsigned lead =
        std::is_same<Layout, col_major>::value ? frag_m : frag_n;
    const unsigned major = mem_index / lead, minor = mem_index % lead;
    if constexpr (std::is_same<Layout, col_major>::value)
      return mem_offset<Layout>(minor, major, ldm, m_offset, n_offset);
    else
      return mem_offset<Layout>(major, minor, ldm, m_offset, n_offset);
  }
  WMMAE_HD unsigned operator()(const unsigned i, const unsigned j,
                               const unsigned ldm, const unsigned m_offset,
                               const unsigned n_offset) const {
    return mem_offset<Layout>(i, j, ldm, m_offset, n_offset);
  }
};

// Element type of a sub-fragment: the operand tag itself for matrix_a and
// matrix_b, float for accumulators (reference: tcec/detail/common.hpp:65-74).
template <class Use, class T> struct sub_frag_t {
  using type = T;
};
template <class T> struct sub_frag_t<accumulator, T> {
  using type = float;
};

} // namespace detail
} // namespace tcec
} // namespace wmma
} // namespace mtk
