// Fragment-mapping primitives for gfx950 wave64 MFMA fragments.
//
// Same call surface as the reference's primitive layer
// (reference: include/wmma_extension/wmma_extension.hpp:27-228 and
// include/wmma_extension/wmma_mma.hpp:18-200), rebuilt on one closed-form
// layout model (detail/common.hpp, frag_layout) instead of per-architecture
// tables.  Every function is wave-collective: all 64 lanes of a wave call it
// with the same template arguments, each lane touches only its own registers.
// A wave64 runs in lock step, so no trailing wave barrier is needed.
//
// Callback contracts (unchanged from the reference):
//   foreach   : func(const unsigned *frag_index_list, unsigned count, unsigned mem_index)
//               mem_index addresses a densely packed tile,
//               i + j*rows (col_major) or i*cols + j (row_major)
//   foreach_ij: func(frag_index_list, count, i, j)
//   foreach_v : func(frag_index_list, count, mem_index) for the registers that
//               hold the first column (col_major) or first row (row_major)
// count is always 1 on gfx950 because no element is duplicated across lanes.
#pragma once
#include "detail/common.hpp"
#include "detail/mfma.hpp"
#include <stdio.h>

namespace mtk {
namespace wmma {

namespace detail {
template <class Frag_T>
using bare_frag_t = typename std::remove_const<
    typename std::remove_reference<Frag_T>::type>::type;

template <class Frag, class Func> WMMAE_D void foreach_ij_core(Func func) {
  using L = typename Frag::layout_model;
  const unsigned lane = common::get_lane_id();
#pragma unroll
  for (unsigned x = 0; x < L::num_elements; x++) {
    const unsigned frag_index_list[1] = {x};
    func(frag_index_list, 1u, L::row(lane, x), L::col(lane, x));
  }
}

template <class Frag, class Func>
WMMAE_D void foreach_core(const bool col, Func func) {
  using L = typename Frag::layout_model;
  foreach_ij_core<Frag>([&](const unsigned *list, const unsigned count,
                            const unsigned i, const unsigned j) {
    func(list, count, col ? (i + j * L::rows) : (i * L::cols + j));
  });
}

template <class Frag, class Func>
WMMAE_D void foreach_v_core(const bool col, Func func) {
  foreach_ij_core<Frag>([&](const unsigned *list, const unsigned count,
                            const unsigned i, const unsigned j) {
    if (col) {
      if (j == 0)
        func(list, count, i);
    } else {
      if (i == 0)
        func(list, count, j);
    }
  });
}

template <class Layout> struct is_col : std::is_same<Layout, col_major> {
  static_assert(std::is_same<Layout, col_major>::value ||
                    std::is_same<Layout, row_major>::value,
                "matrix_a / matrix_b fragments need row_major or col_major");
};
} // namespace detail

// ---------------------------------------------------------------- foreach
template <class Frag_T, class Func> WMMAE_D void foreach (Func func) {
  using F = detail::bare_frag_t<Frag_T>;
  detail::foreach_core<F>(detail::is_col<typename F::layout>::value, func);
}
template <class Frag_T, class Func>
WMMAE_D void foreach (const layout_t layout, Func func) {
  using F = detail::bare_frag_t<Frag_T>;
  detail::foreach_core<F>(layout == mem_col_major, func);
}
template <class Use, int M, int N, int K, class T, class Layout, class Func>
WMMAE_D void foreach (fragment<Use, M, N, K, T, Layout> &, Func func) {
  foreach
    <fragment<Use, M, N, K, T, Layout>>(func);
}
template <int M, int N, int K, class T, class Func>
WMMAE_D void foreach (fragment<accumulator, M, N, K, T> &,
                      const layout_t layout, Func func) {
  foreach
    <fragment<accumulator, M, N, K, T>>(layout, func);
}

// ------------------------------------------------------------- foreach_ij
template <class Frag_T, class Func> WMMAE_D void foreach_ij(Func func) {
  detail::foreach_ij_core<detail::bare_frag_t<Frag_T>>(func);
}
// The layout argument is kept for signature compatibility; (i,j) of an
// accumulator register does not depend on the memory layout.
template <class Frag_T, class Func>
WMMAE_D void foreach_ij(const layout_t, Func func) {
  detail::foreach_ij_core<detail::bare_frag_t<Frag_T>>(func);
}
template <class Use, int M, int N, int K, class T, class Layout, class Func>
WMMAE_D void foreach_ij(fragment<Use, M, N, K, T, Layout> &, Func func) {
  detail::foreach_ij_core<fragment<Use, M, N, K, T, Layout>>(func);
}
template <int M, int N, int K, class T, class Func>
WMMAE_D void foreach_ij(fragment<accumulator, M, N, K, T> &, const layout_t,
                        Func func) {
  detail::foreach_ij_core<fragment<accumulator, M, N, K, T>>(func);
}

// -------------------------------------------------------------- foreach_v
template <class Frag_T, class Func> WMMAE_D void foreach_v(Func func) {
  using F = detail::bare_frag_t<Frag_T>;
  detail::foreach_v_core<F>(detail::is_col<typename F::layout>::value, func);
}
template <class Frag_T, class Func>
WMMAE_D void foreach_v(const layout_t layout, Func func) {
  detail::foreach_v_core<detail::bare_frag_t<Frag_T>>(layout == mem_col_major,
                                                       func);
}
template <class Use, int M, int N, int K, class T, class Layout, class Func>
WMMAE_D void foreach_v(fragment<Use, M, N, K, T, Layout> &, Func func) {
  foreach_v<fragment<Use, M, N, K, T, Layout>>(func);
}
template <int M, int N, int K, class T, class Func>
WMMAE_D void foreach_v(fragment<accumulator, M, N, K, T> &,
                       const layout_t layout, Func func) {
  foreach_v<fragment<accumulator, M, N, K, T>>(layout, func);
}

// -------------------------------------------------------------------- map
// (i, j) -> (lane, register).  list_size is always 1 on gfx950; the [2]
// arrays keep the reference signature (wmma_extension.hpp:115-123).
template <class Frag_T>
WMMAE_HD void map(unsigned tid_list[2], unsigned fid_list[2],
                  unsigned &list_size, const unsigned i, const unsigned j) {
  using L = typename detail::bare_frag_t<Frag_T>::layout_model;
  list_size = 1;
  tid_list[0] = L::tid(i, j);
  fid_list[0] = L::fid(i, j);
}

// -------------------------------------------------------- fill functions
template <class Use, int M, int N, int K, class T, class Layout>
WMMAE_D void fill_zero(fragment<Use, M, N, K, T, Layout> &frag) {
#pragma unroll
  for (unsigned x = 0; x < frag.num_elements; x++)
    frag.x[x] = static_cast<typename fragment<Use, M, N, K, T,
                                              Layout>::storage_element_type>(0);
}
template <class Use, int M, int N, int K, class T, class Layout, class V>
WMMAE_D void fill_fragment(fragment<Use, M, N, K, T, Layout> &frag,
                           const V v) {
  const auto s = detail::common::cast<T>(v);
#pragma unroll
  for (unsigned x = 0; x < frag.num_elements; x++)
    frag.x[x] = s;
}

// ------------------------------------------------- matrix load / store
namespace detail {
// An fp32 accumulator holds rows r .. r+3 of one column in registers 4q .. 4q+3
// of a lane (the MFMA result layout), so a column-major tile whose base and
// leading dimension keep those four floats 16-byte aligned moves with one
// 16-byte access per four registers instead of four 4-byte ones.
typedef float f32_quad __attribute__((ext_vector_type(4)));
template <class L> constexpr bool rows_in_quads() {
  if (L::num_elements % 4 != 0)
    return false;
  for (unsigned lane = 0; lane < wave_size; lane++)
    for (unsigned x = 0; x < L::num_elements; x += 4)
      for (unsigned e = 0; e < 4; e++)
        if (L::row(lane, x) % 4 != 0 ||
            L::row(lane, x + e) != L::row(lane, x) + e ||
            L::col(lane, x + e) != L::col(lane, x))
          return false;
  return true;
}
template <int M, int N, int K, class T, class MEM_T> struct acc_quads {
  static constexpr bool value =
      std::is_same<T, float>::value &&
      std::is_same<typename std::remove_cv<MEM_T>::type, float>::value &&
      rows_in_quads<gfx950::frag_layout<accumulator, M, N, K>>();
};
template <class P>
WMMAE_D bool quad_aligned(const P *const ptr, const unsigned ldm) {
  return ldm % 4 == 0 && (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0;
}
} // namespace detail

// (reference: nvcuda::wmma::load_matrix_sync and wmma_mma.hpp:64-145; there
// the dense mem_index is re-strided to ldm, here (i,j) is used directly.)
template <class Use, int M, int N, int K, class T, class Layout, class MEM_T>
WMMAE_D void load_matrix_sync(fragment<Use, M, N, K, T, Layout> &frag,
                              const MEM_T *const ptr, const unsigned ldm,
                              const bool = true) {
  static_assert(!std::is_same<Use, accumulator>::value,
                "accumulator loads take a layout_t argument");
  constexpr bool col = detail::is_col<Layout>::value;
  foreach_ij<decltype(frag)>([&](const unsigned *list, const unsigned,
                                 const unsigned i, const unsigned j) {
    frag.x[list[0]] =
        detail::common::cast<T>(ptr[col ? (i + j * ldm) : (i * ldm + j)]);
  });
}
template <int M, int N, int K, class T, class MEM_T>
WMMAE_D void load_matrix_sync(fragment<accumulator, M, N, K, T> &frag,
                              const MEM_T *const ptr, const unsigned ldm,
                              const layout_t layout, const bool = true) {
  const bool col = layout == mem_col_major;
  if constexpr (detail::acc_quads<M, N, K, T, MEM_T>::value) {
    if (col && detail::quad_aligned(ptr, ldm)) {
      using L = typename fragment<accumulator, M, N, K, T>::layout_model;
      const unsigned lane = detail::common::get_lane_id();
#pragma unroll
      for (unsigned x = 0; x < frag.num_elements; x += 4) {
        const detail::f32_quad v = *reinterpret_cast<const detail::f32_quad *>(
            ptr + L::row(lane, x) + L::col(lane, x) * ldm);
#pragma unroll
        for (unsigned e = 0; e < 4; e++)
          frag.x[x + e] = v[e];
      }
      return;
    }
  }
  foreach_ij<decltype(frag)>([&](const unsigned *list, const unsigned,
                                 const unsigned i, const unsigned j) {
    frag.x[list[0]] =
        detail::common::cast<T>(ptr[col ? (i + j * ldm) : (i * ldm + j)]);
  });
}
template <int M, int N, int K, class T, class MEM_T>
WMMAE_D void store_matrix_sync(MEM_T *const ptr,
                               const fragment<accumulator, M, N, K, T> &frag,
                               const unsigned ldm, const layout_t layout,
                               const bool = true) {
  const bool col = layout == mem_col_major;
  if constexpr (detail::acc_quads<M, N, K, T, MEM_T>::value) {
    if (col && detail::quad_aligned(ptr, ldm)) {
      using L = typename fragment<accumulator, M, N, K, T>::layout_model;
      const unsigned lane = detail::common::get_lane_id();
#pragma unroll
      for (unsigned x = 0; x < frag.num_elements; x += 4) {
        const detail::f32_quad v = {frag.x[x], frag.x[x + 1], frag.x[x + 2],
                                    frag.x[x + 3]};
        *reinterpret_cast<detail::f32_quad *>(ptr + L::row(lane, x) +
                                              L::col(lane, x) * ldm) = v;
      }
      return;
    }
  }
  foreach_ij<decltype(frag)>([&](const unsigned *list, const unsigned,
                                 const unsigned i, const unsigned j) {
    ptr[col ? (i + j * ldm) : (i * ldm + j)] =
        detail::common::cast<MEM_T>(frag.x[list[0]]);
  });
}

// ------------------------------------------------- vector load / store
// load_vector puts a vector into the first column (col_major) or first row
// (row_major) of the fragment; with fill == true the rest is zeroed first
// (reference: wmma_extension.hpp:128-228).
template <class Use, int M, int N, int K, class FT, class Layout, class T>
WMMAE_D void load_vector(fragment<Use, M, N, K, FT, Layout> &frag,
                         const T *const ptr, const bool fill = true) {
  if (fill)
    fill_zero(frag);
  foreach_v<decltype(frag)>(
      [&](const unsigned *list, const unsigned, const unsigned mem_index) {
        frag.x[list[0]] = detail::common::cast<FT>(ptr[mem_index]);
      });
}
template <class Use, int M, int N, int K, class FT, class Layout, class T>
WMMAE_D void load_vector(fragment<Use, M, N, K, FT, Layout> &frag,
                         const T *const ptr, const T mul,
                         const bool fill = true) {
  if (fill)
    fill_zero(frag);
  foreach_v<decltype(frag)>(
      [&](const unsigned *list, const unsigned, const unsigned mem_index) {
        frag.x[list[0]] = detail::common::cast<FT>(ptr[mem_index] * mul);
      });
}
template <int M, int N, int K, class FT, class T>
WMMAE_D void load_vector(fragment<accumulator, M, N, K, FT> &frag,
                         const T *const ptr, const layout_t layout,
                         const bool fill = true) {
  if (fill)
    fill_zero(frag);
  foreach_v<decltype(frag)>(
      layout,
      [&](const unsigned *list, const unsigned, const unsigned mem_index) {
        frag.x[list[0]] = detail::common::cast<FT>(ptr[mem_index]);
      });
}
template <int M, int N, int K, class FT, class T>
WMMAE_D void load_vector(fragment<accumulator, M, N, K, FT> &frag,
                         const T *const ptr, const layout_t layout, const T mul,
                         const bool fill = true) {
  if (fill)
    fill_zero(frag);
  foreach_v<decltype(frag)>(
      layout,
      [&](const unsigned *list, const unsigned, const unsigned mem_index) {
        frag.x[list[0]] = detail::common::cast<FT>(ptr[mem_index] * mul);
      });
}
template <int M, int N, int K, class FT, class T>
WMMAE_D void store_vector(T *const ptr,
                          const fragment<accumulator, M, N, K, FT> &frag,
                          const layout_t layout) {
  foreach_v<decltype(frag)>(
      layout,
      [&](const unsigned *list, const unsigned, const unsigned mem_index) {
        ptr[mem_index] = detail::common::cast<T>(frag.x[list[0]]);
      });
}
template <int M, int N, int K, class FT, class T>
WMMAE_D void store_vector(T *const ptr,
                          const fragment<accumulator, M, N, K, FT> &frag,
                          const T mul, const layout_t layout) {
  foreach_v<decltype(frag)>(
      layout,
      [&](const unsigned *list, const unsigned, const unsigned mem_index) {
        ptr[mem_index] = detail::common::cast<T>(frag.x[list[0]]) * mul;
      });
}

// ---------------------------------------------------------- debug print
template <class Use, int M, int N, int K, class T, class Layout>
__device__ inline void
print_fragment(const fragment<Use, M, N, K, T, Layout> &frag,
               const char *name = "") {
  const unsigned lane = detail::common::get_lane_id();
  if (lane == 0 && name[0] != '\0')
    printf("%s = \n", name);
  for (unsigned l = 0; l < wave_size; l++) {
    if (l == lane) {
      for (unsigned x = 0; x < frag.num_elements; x++)
        printf("%+.3e ", static_cast<float>(frag.x[x]));
      printf("\n");
    }
  }
}

// ------------------------------------------------------- identity matrices
// frag += a * I (reference: wmma_extension.hpp:233-248; per-architecture
// register lists in detail/sm_80.hpp:404-415).  Here the diagonal is found
// through the layout model: the lane that owns (i, i) adds a.
template <int M, int N, int K, class T, class FT>
WMMAE_D void add_eye(fragment<accumulator, M, N, K, T> &frag, const FT a) {
  detail::foreach_ij_core<fragment<accumulator, M, N, K, T>>(
      [&](const unsigned *list, const unsigned, const unsigned i,
          const unsigned j) {
        if (i == j)
          frag.x[list[0]] += detail::common::cast<T>(a);
      });
}
template <int M, int N, int K, class T>
WMMAE_D void make_identity_matrix(fragment<accumulator, M, N, K, T> &frag) {
  fill_zero(frag);
  add_eye(frag, detail::common::cast<T>(1.0f));
}

// -------------------------------------------------- direct (outer) products
// Operand fragments whose single MMA gives the error-corrected outer product
// u v^T of two fp32 vectors held as x = leading 16-bit part, dx = residual
// (reference: wmma_extension.hpp:250-284, detail/sm_80.hpp:417-525,
// docs/make_direct_product_fragments-en.svg):
//   matrix_a: columns 0..3 = x, dx, x, dx      (column 3 only with 3 terms)
//   matrix_b: rows    0..3 = x, x, dx, dx      (row 3 only with 3 terms)
// so that A*B = x_a x_b^T + dx_a x_b^T + x_a dx_b^T (+ dx_a dx_b^T).  All other
// elements are zeroed when `fill` is set and left alone otherwise.
namespace detail {
template <unsigned CORRECTION_TERMS, class Use, int M, int N, int K, class FT,
          class Layout, class GetX, class GetDx>
WMMAE_D void direct_product_core(fragment<Use, M, N, K, FT, Layout> &frag,
                                 const bool fill, GetX x_of, GetDx dx_of) {
  static_assert(!std::is_same<Use, accumulator>::value,
                "direct products are operand fragments");
  static_assert(K >= 4, "four k positions are used");
  static_assert(CORRECTION_TERMS == 2 || CORRECTION_TERMS == 3,
                "2 or 3 correction terms");
  if (fill)
    fill_zero(frag);
  constexpr bool is_a = std::is_same<Use, matrix_a>::value;
  foreach_ij_core<fragment<Use, M, N, K, FT, Layout>>(
      [&](const unsigned *list, const unsigned, const unsigned i,
          const unsigned j) {
        const unsigned kk = is_a ? j : i; // position along k
        const unsigned e = is_a ? i : j;  // vector element
        if (kk >= 4 || (kk == 3 && CORRECTION_TERMS != 3))
          return;
        // matrix_a: x, dx, x, dx   matrix_b: x, x, dx, dx
        const bool residual = is_a ? (kk & 1u) != 0 : kk >= 2;
        frag.x[list[0]] = residual ? dx_of(e) : x_of(e);
      });
}
} // namespace detail

template <class MatrixType, int M, int N, int K, class MemMajor, class T,
          class S, class FT>
WMMAE_D void
make_direct_product_fragment(fragment<MatrixType, M, N, K, FT, MemMajor> &frag_x,
                             const T *const x, const S *const dx,
                             const bool fill = true) {
  detail::direct_product_core<2>(
      frag_x, fill,
      [&](const unsigned e) { return detail::common::cast<FT>(x[e]); },
      [&](const unsigned e) { return detail::common::cast<FT>(dx[e]); });
}
template <class MatrixType, int M, int N, int K, class MemMajor, class T,
          class S, class FT>
WMMAE_D void make_direct_product_fragment_c3(
    fragment<MatrixType, M, N, K, FT, MemMajor> &frag_x, const T *const x,
    const S *const dx, const bool fill = true) {
  detail::direct_product_core<3>(
      frag_x, fill,
      [&](const unsigned e) { return detail::common::cast<FT>(x[e]); },
      [&](const unsigned e) { return detail::common::cast<FT>(dx[e]); });
}
// From the fp32 vector itself: dx = x - float(cast(x)), computed on the fly.
template <class MatrixType, int M, int N, int K, class MemMajor, class FT>
WMMAE_D void
make_direct_product_fragment(fragment<MatrixType, M, N, K, FT, MemMajor> &frag_x,
                             const float *const x, const bool fill = true) {
  detail::direct_product_core<2>(
      frag_x, fill,
      [&](const unsigned e) { return detail::common::cast<FT>(x[e]); },
      [&](const unsigned e) {
        return detail::common::cast<FT>(
            x[e] - static_cast<float>(detail::common::cast<FT>(x[e])));
      });
}
template <class MatrixType, int M, int N, int K, class MemMajor, class FT>
WMMAE_D void make_direct_product_fragment_c3(
    fragment<MatrixType, M, N, K, FT, MemMajor> &frag_x, const float *const x,
    const bool fill = true) {
  detail::direct_product_core<3>(
      frag_x, fill,
      [&](const unsigned e) { return detail::common::cast<FT>(x[e]); },
      [&](const unsigned e) {
        return detail::common::cast<FT>(
            x[e] - static_cast<float>(detail::common::cast<FT>(x[e])));
      });
}

} // namespace wmma
} // namespace mtk
