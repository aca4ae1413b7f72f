// TCEC: error-corrected fp32 matrix multiply-accumulate on the gfx950 matrix
// cores, with the device-side API of the reference's mtk::wmma::tcec
// (reference: include/wmma_extension/tcec/tcec.hpp:13-927 for with_ec and
// tcec/detail/no_cor.hpp:13-897 for without_ec; docs/mma_f32.md:59-135).
//
// A tcec::fragment<Use,m,n,k,T,Layout,Policy> covers an m x n x k problem with
// a grid of MFMA sub-fragments of the policy's shape.  Sub-block (bm,bn) is
// stored at index bm + num_sub_frag_m*bn.  matrix_a / matrix_b fragments hold
// the split terms of their fp32 source (sub_frag = leading term, sub_d_frag =
// residual term, sub_d2_frag = second residual of the three-term split);
// accumulators hold an fp32 main part (sub_frag) and an fp32 error part
// (sub_d_frag, scaled by split_traits<T>::scale).  Everything is
// wave64-collective; `sync` arguments are accepted and ignored because a wave
// runs in lock step.
#pragma once
#include "detail/common.hpp"
#include "detail/functions.hpp"
#include "detail/policy.hpp"
#include "detail/scale.hpp"

namespace mtk {
namespace wmma {
namespace tcec {

template <class Use, int m, int n, int k, class T, class Layout = void,
          class Policy_ = typename detail::default_policy<T>::type>
struct fragment {
  using Policy = Policy_;
  using element_type = float;
  using split = detail::split_traits<T>;
  static constexpr int sub_frag_m = Policy::m;
  static constexpr int sub_frag_n = Policy::n;
  static constexpr int sub_frag_k = Policy::k;
  static constexpr bool is_acc = std::is_same<Use, accumulator>::value;
  static constexpr bool has_ec =
      std::is_same<typename Policy::error_correction, with_ec>::value;

  using sub_elem_t =
      typename detail::sub_frag_t<Use, typename split::mma_tag>::type;
  using sub_frag_t =
      typename detail::default_fragment<Use, sub_elem_t, Layout, Policy>::type;
  using storage_t = typename sub_frag_t::storage_element_type;

  static constexpr int num_sub_frag_m =
      detail::select_value<Use, m, k, m>::value /
      detail::select_value<Use, sub_frag_m, sub_frag_k, sub_frag_m>::value;
  static constexpr int num_sub_frag_n =
      detail::select_value<Use, k, n, n>::value /
      detail::select_value<Use, sub_frag_k, sub_frag_n, sub_frag_n>::value;
  static constexpr int num_sub_frags = num_sub_frag_m * num_sub_frag_n;
  static_assert(num_sub_frag_m * detail::select_value<Use, sub_frag_m,
                                                      sub_frag_k,
                                                      sub_frag_m>::value ==
                        detail::select_value<Use, m, k, m>::value &&
                    num_sub_frag_n * detail::select_value<Use, sub_frag_k,
                                                          sub_frag_n,
                                                          sub_frag_n>::value ==
                        detail::select_value<Use, k, n, n>::value,
                "m, n, k must be multiples of the policy's instruction shape");
  // number of stored parts: 1 without error correction; accumulators keep
  // main + error; operands keep as many terms as the split produces.
  static constexpr int num_terms =
      !has_ec ? 1 : (is_acc ? 2 : split::num_terms);
  // (the reference has no default_policy<float, with_ec, ...> either,
  // tcec/detail/policy.hpp:63-99)
  static_assert(!has_ec || split::num_terms >= 2,
                "error correction needs a split of at least two terms: fp32 "
                "operands (op_simt) go with without_ec");

  sub_frag_t sub_frag[num_sub_frags];
  sub_frag_t sub_d_frag[num_terms >= 2 ? num_sub_frags : 0];
  sub_frag_t sub_d2_frag[num_terms >= 3 ? num_sub_frags : 0];

  static constexpr unsigned num_elements =
      num_sub_frags * sub_frag_t::num_elements;

  WMMAE_D storage_t &x(const unsigned index) {
    return sub_frag[index / sub_frag_t::num_elements]
        .x[index % sub_frag_t::num_elements];
  }
  WMMAE_D storage_t x(const unsigned index) const {
    return sub_frag[index / sub_frag_t::num_elements]
        .x[index % sub_frag_t::num_elements];
  }
  WMMAE_D storage_t &dx(const unsigned index) {
    return sub_d_frag[index / sub_frag_t::num_elements]
        .x[index % sub_frag_t::num_elements];
  }
  WMMAE_D storage_t dx(const unsigned index) const {
    return sub_d_frag[index / sub_frag_t::num_elements]
        .x[index % sub_frag_t::num_elements];
  }

  // Fold the error part of an accumulator into its main part.
  WMMAE_D void integrate() {
    if constexpr (num_terms >= 2) {
#pragma unroll
      for (int f = 0; f < num_sub_frags; f++) {
#pragma unroll
        for (unsigned i = 0; i < sub_frag_t::num_elements; i++) {
          sub_frag[f].x[i] += detail::correction_scale_1<T>(
              static_cast<float>(sub_d_frag[f].x[i]));
          sub_d_frag[f].x[i] = static_cast<storage_t>(0);
        }
      }
    }
  }
};

#define WMMAE_TCEC_TPARAMS                                                     \
  int m, int n, int k, class T, class Op, class EC, int fm, int fn, int fk
#define WMMAE_TCEC_FRAG(Use, Layout)                                           \
  fragment<Use, m, n, k, T, Layout, Policy<Op, EC, fm, fn, fk>>

namespace detail {
// Write the split of v into every stored term of an operand fragment.
template <class Frag>
WMMAE_D void put_split(Frag &frag, const unsigned block,
                       const unsigned frag_index, const float v) {
  using split = typename Frag::split;
  typename split::storage t0, t1, t2;
  split::split(v, t0, t1, t2);
  frag.sub_frag[block].x[frag_index] = t0;
  if constexpr (Frag::num_terms >= 2)
    frag.sub_d_frag[block].x[frag_index] = t1;
  if constexpr (Frag::num_terms >= 3)
    frag.sub_d2_frag[block].x[frag_index] = t2;
}

// Operand sub-fragments keep runs of four consecutive k of one row (matrix_a)
// or one column (matrix_b) in registers 4q .. 4q+3 of a lane (a lane of the
// 16x16x32 instruction owns eight consecutive k).  When k is the contiguous
// direction of the memory being read - row-major memory for matrix_a,
// column-major for matrix_b: the layout of the reference's GEMM
// (test/tcec/batch_gemm.cu:259-260) - such a run is 16 contiguous bytes.
template <class L, bool is_a> constexpr bool k_runs_of_four() {
  if (L::num_elements % 4 != 0)
    return false;
  for (unsigned lane = 0; lane < wave_size; lane++)
    for (unsigned x = 0; x < L::num_elements; x += 4)
      for (unsigned e = 0; e < 4; e++) {
        const unsigned fixed0 = is_a ? L::row(lane, x) : L::col(lane, x);
        const unsigned fixed = is_a ? L::row(lane, x + e) : L::col(lane, x + e);
        const unsigned k0 = is_a ? L::col(lane, x) : L::row(lane, x);
        const unsigned kk = is_a ? L::col(lane, x + e) : L::row(lane, x + e);
        if (fixed != fixed0 || k0 % 4 != 0 || kk != k0 + e)
          return false;
      }
  return true;
}
template <class F, class MatrixLayout, class MEM_T> struct operand_quads {
  static constexpr bool is_a = std::is_same<typename F::sub_frag_t::use,
                                            matrix_a>::value;
  static constexpr bool value =
      !F::is_acc &&
      std::is_same<typename std::remove_cv<MEM_T>::type, float>::value &&
      std::is_same<MatrixLayout,
                   typename std::conditional<is_a, row_major,
                                             col_major>::type>::value &&
      k_runs_of_four<typename F::sub_frag_t::layout_model, is_a>();
};

// Swizzled staging tiles (additions; the reference pads the rows of its
// shared-memory tiles instead, test/tcec/batch_gemm.cu:11, a skew found with
// research/bank-conflict/main.cu:38-71).  On gfx950 no row padding makes the
// fragment read of a 16x16x32 operand from an fp32 tile conflict free: a
// 16-byte LDS read is served sixteen lanes at a time, and those sixteen are
// eight rows of one k group and eight rows of the next.  What does: rows of
// exactly 32 k (128 bytes, no padding) per k block, with the eight 16-byte
// pieces of row r stored at piece index p ^ swizzled_piece_mask(r).
WMMAE_HD constexpr unsigned swizzled_piece_mask(const unsigned row) {
  return (row >> 1) & 5u;
}
template <class MatrixLayout> struct is_swizzled : std::false_type {};

// Value an accumulator element stands for.
template <class Frag>
WMMAE_D float combined(const Frag &frag, const unsigned block,
                       const unsigned frag_index) {
  if constexpr (Frag::num_terms >= 2)
    return frag.sub_frag[block].x[frag_index] +
           frag.sub_d_frag[block].x[frag_index] / Frag::split::scale;
  else
    return frag.sub_frag[block].x[frag_index];
}
} // namespace detail

// Memory layout tags for load_matrix_sync<...>: an fp32 tile with k the
// contiguous direction (rows of matrix_a / columns of matrix_b, `ldm` floats
// apart, ldm a multiple of 32) whose 16-byte pieces are permuted inside every
// aligned block of 32 k: element (r, kk) of the tile is at
//   r * ldm + (kk & ~31) + 4 * (((kk & 31) / 4) ^ swizzled_piece(r)) + kk % 4
// with swizzled_piece(r) = (r / 2) & 5.  Fragment loads from such a tile are
// free of LDS bank conflicts with the policy shape 16x16x32 (other shapes read
// it correctly, with the conflicts a padded tile would have).  The pointer handed to
// load_matrix_sync must sit a multiple of 16 rows and of 32 k inside the tile.
// A writer fills the tile 16 bytes at a time: physical piece q of row r holds
// the logical piece q ^ swizzled_piece(r) - with utils::cp_async, whose lane l
// of a wave writes LDS piece base + l, lane l simply fetches that logical piece.
struct row_major_swizzled; // matrix_a: rows of k
struct col_major_swizzled; // matrix_b: columns of k
WMMAE_HD constexpr unsigned swizzled_piece(const unsigned row) {
  return detail::swizzled_piece_mask(row);
}
namespace detail {
template <> struct is_swizzled<row_major_swizzled> : std::true_type {};
template <> struct is_swizzled<col_major_swizzled> : std::true_type {};
} // namespace detail

// ------------------------------------------------------------ fill / neg
template <class Use, WMMAE_TCEC_TPARAMS, class Layout, class V>
WMMAE_D void fill_fragment(WMMAE_TCEC_FRAG(Use, Layout) & frag, const V v) {
  using F = WMMAE_TCEC_FRAG(Use, Layout);
#pragma unroll
  for (int b = 0; b < F::num_sub_frags; b++) {
    mtk::wmma::fill_fragment(frag.sub_frag[b], v);
    if constexpr (F::num_terms >= 2)
      mtk::wmma::fill_zero(frag.sub_d_frag[b]);
    if constexpr (F::num_terms >= 3)
      mtk::wmma::fill_zero(frag.sub_d2_frag[b]);
  }
}

template <class Use, WMMAE_TCEC_TPARAMS, class Layout>
WMMAE_D void fill_zero(WMMAE_TCEC_FRAG(Use, Layout) & frag) {
  using F = WMMAE_TCEC_FRAG(Use, Layout);
#pragma unroll
  for (int b = 0; b < F::num_sub_frags; b++) {
    mtk::wmma::fill_zero(frag.sub_frag[b]);
    if constexpr (F::num_terms >= 2)
      mtk::wmma::fill_zero(frag.sub_d_frag[b]);
    if constexpr (F::num_terms >= 3)
      mtk::wmma::fill_zero(frag.sub_d2_frag[b]);
  }
}

template <class Use, WMMAE_TCEC_TPARAMS, class Layout>
WMMAE_D WMMAE_TCEC_FRAG(Use, Layout)
    neg(const WMMAE_TCEC_FRAG(Use, Layout) & frag) {
  using F = WMMAE_TCEC_FRAG(Use, Layout);
  F res;
#pragma unroll
  for (int b = 0; b < F::num_sub_frags; b++) {
#pragma unroll
    for (unsigned i = 0; i < F::sub_frag_t::num_elements; i++) {
      res.sub_frag[b].x[i] = -frag.sub_frag[b].x[i];
      if constexpr (F::num_terms >= 2)
        res.sub_d_frag[b].x[i] = -frag.sub_d_frag[b].x[i];
      if constexpr (F::num_terms >= 3)
        res.sub_d2_frag[b].x[i] = -frag.sub_d2_frag[b].x[i];
    }
  }
  return res;
}

// ------------------------------------------------------------ load matrix
// MatrixLayout is the layout of the memory being read; it is independent of
// the fragment's own Layout argument (docs/mma_f32.md:114-123).  Operands are
// split while loading; accumulators are taken as fp32 with a zero error part.
template <class MatrixLayout, class Use, WMMAE_TCEC_TPARAMS, class Layout,
          class MEM_T>
WMMAE_D void load_matrix_sync_with_mul(WMMAE_TCEC_FRAG(Use, Layout) & frag,
                                       const MEM_T *const ptr,
                                       const unsigned ldm, const MEM_T mul,
                                       const bool = true) {
  using F = WMMAE_TCEC_FRAG(Use, Layout);
  constexpr unsigned bm_size =
      detail::select_value<Use, fm, fk, fm>::value; // rows of one sub-block
  constexpr unsigned bn_size = detail::select_value<Use, fk, fn, fn>::value;
  if constexpr (F::is_acc && std::is_same<MatrixLayout, col_major>::value &&
                mtk::wmma::detail::acc_quads<fm, fn, fk, float,
                                             MEM_T>::value) {
    // column-major fp32 memory, four consecutive rows per register quad
    if (mtk::wmma::detail::quad_aligned(ptr, ldm)) {
      using L = typename F::sub_frag_t::layout_model;
      const unsigned lane = mtk::wmma::detail::common::get_lane_id();
#pragma unroll
      for (unsigned bn = 0; bn < unsigned(F::num_sub_frag_n); bn++) {
#pragma unroll
        for (unsigned bm = 0; bm < unsigned(F::num_sub_frag_m); bm++) {
          const unsigned block = bm + F::num_sub_frag_m * bn;
#pragma unroll
          for (unsigned x = 0; x < L::num_elements; x += 4) {
            const detail::f32x4_t v =
                *reinterpret_cast<const detail::f32x4_t *>(
                    ptr + detail::mem_offset<col_major>(
                              L::row(lane, x), L::col(lane, x), ldm,
                              bm * bm_size, bn * bn_size)) *
                static_cast<float>(mul);
#pragma unroll
            for (unsigned e = 0; e < 4; e++) {
              frag.sub_frag[block].x[x + e] = v[e];
              if constexpr (F::num_terms >= 2)
                frag.sub_d_frag[block].x[x + e] = 0.f;
            }
          }
        }
      }
      return;
    }
  }
  if constexpr (detail::is_swizzled<MatrixLayout>::value) {
    // swizzled staging tile: 16-byte reads, conflict free in LDS
    constexpr bool is_a = std::is_same<Use, matrix_a>::value;
    using L = typename F::sub_frag_t::layout_model;
    static_assert(!F::is_acc &&
                      std::is_same<typename std::remove_cv<MEM_T>::type,
                                   float>::value &&
                      std::is_same<MatrixLayout,
                                   typename std::conditional<
                                       is_a, row_major_swizzled,
                                       col_major_swizzled>::type>::value &&
                      detail::k_runs_of_four<L, is_a>(),
                  "swizzled tiles: fp32 memory, matrix_a with "
                  "row_major_swizzled or matrix_b with col_major_swizzled, an "
                  "instruction shape whose lanes own runs of four k");
    const unsigned lane = mtk::wmma::detail::common::get_lane_id();
#pragma unroll
    for (unsigned bn = 0; bn < unsigned(F::num_sub_frag_n); bn++) {
#pragma unroll
      for (unsigned bm = 0; bm < unsigned(F::num_sub_frag_m); bm++) {
        const unsigned block = bm + F::num_sub_frag_m * bn;
#pragma unroll
        for (unsigned x = 0; x < L::num_elements; x += 4) {
          const unsigned i = L::row(lane, x) + bm * bm_size;
          const unsigned j = L::col(lane, x) + bn * bn_size;
          const unsigned line = is_a ? i : j, kk = is_a ? j : i;
          const unsigned off =
              line * ldm + (kk & ~31u) +
              4u * (((kk & 31u) >> 2) ^ detail::swizzled_piece_mask(line));
          const detail::f32x4_t v =
              *reinterpret_cast<const detail::f32x4_t *>(ptr + off) *
              static_cast<float>(mul);
          typename F::storage_t *d1 = nullptr, *d2 = nullptr;
          if constexpr (F::num_terms >= 2)
            d1 = &frag.sub_d_frag[block].x[x];
          if constexpr (F::num_terms >= 3)
            d2 = &frag.sub_d2_frag[block].x[x];
          if constexpr (F::num_terms == F::split::num_terms) {
            detail::split4<T>(v, &frag.sub_frag[block].x[x], d1, d2);
          } else { // without_ec: the leading term only
            typename F::storage_t t1[4], t2[4];
            detail::split4<T>(v, &frag.sub_frag[block].x[x], t1, t2);
          }
        }
      }
    }
    return;
  }
  if constexpr (detail::operand_quads<F, MatrixLayout, MEM_T>::value) {
    // k contiguous in memory, base and leading dimension keeping every run
    // of four k 16-byte aligned: one 16-byte read per four registers, split
    // two elements at a time (same arithmetic, same bits as the path below)
    if (mtk::wmma::detail::quad_aligned(ptr, ldm)) {
      using L = typename F::sub_frag_t::layout_model;
      const unsigned lane = mtk::wmma::detail::common::get_lane_id();
#pragma unroll
      for (unsigned bn = 0; bn < unsigned(F::num_sub_frag_n); bn++) {
#pragma unroll
        for (unsigned bm = 0; bm < unsigned(F::num_sub_frag_m); bm++) {
          const unsigned block = bm + F::num_sub_frag_m * bn;
#pragma unroll
          for (unsigned x = 0; x < L::num_elements; x += 4) {
            const unsigned off = detail::mem_offset<MatrixLayout>(
                L::row(lane, x), L::col(lane, x), ldm, bm * bm_size,
                bn * bn_size);
            const detail::f32x4_t v =
                *reinterpret_cast<const detail::f32x4_t *>(ptr + off) *
                static_cast<float>(mul);
            typename F::storage_t *d1 = nullptr, *d2 = nullptr;
            if constexpr (F::num_terms >= 2)
              d1 = &frag.sub_d_frag[block].x[x];
            if constexpr (F::num_terms >= 3)
              d2 = &frag.sub_d2_frag[block].x[x];
            if constexpr (F::num_terms == F::split::num_terms) {
              detail::split4<T>(v, &frag.sub_frag[block].x[x], d1, d2);
            } else { // without_ec: the leading term only
              typename F::storage_t t1[4], t2[4];
              detail::split4<T>(v, &frag.sub_frag[block].x[x], t1, t2);
            }
          }
        }
      }
      return;
    }
  }
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
            const float v = static_cast<float>(ptr[off]) *
                            static_cast<float>(mul);
            if constexpr (F::is_acc) {
              frag.sub_frag[block].x[list[0]] = v;
              if constexpr (F::num_terms >= 2)
                frag.sub_d_frag[block].x[list[0]] = 0.f;
            } else {
              detail::put_split(frag, block, list[0], v);
            }
          }
        }
      });
}

template <class MatrixLayout, class Use, WMMAE_TCEC_TPARAMS, class Layout,
          class MEM_T>
WMMAE_D void load_matrix_sync(WMMAE_TCEC_FRAG(Use, Layout) & frag,
                              const MEM_T *const ptr, const unsigned ldm,
                              const bool sync = true) {
  load_matrix_sync_with_mul<MatrixLayout>(frag, ptr, ldm,
                                          static_cast<MEM_T>(1), sync);
}

// Memory layout = the fragment's own Layout (operands only).
template <class Use, WMMAE_TCEC_TPARAMS, class Layout, class MEM_T>
WMMAE_D void load_matrix_sync(WMMAE_TCEC_FRAG(Use, Layout) & frag,
                              const MEM_T *const ptr, const unsigned ldm,
                              const bool sync = true) {
  static_assert(!std::is_same<Use, accumulator>::value,
                "accumulator loads need a layout");
  load_matrix_sync<Layout>(frag, ptr, ldm, sync);
}
template <class Use, WMMAE_TCEC_TPARAMS, class Layout, class MEM_T>
WMMAE_D void load_matrix_sync_with_mul(WMMAE_TCEC_FRAG(Use, Layout) & frag,
                                       const MEM_T *const ptr,
                                       const unsigned ldm, const MEM_T mul,
                                       const bool sync = true) {
  static_assert(!std::is_same<Use, accumulator>::value,
                "accumulator loads need a layout");
  load_matrix_sync_with_mul<Layout>(frag, ptr, ldm, mul, sync);
}

// Accumulators with a run-time layout.
template <WMMAE_TCEC_TPARAMS, class MEM_T>
WMMAE_D void load_matrix_sync(WMMAE_TCEC_FRAG(accumulator, void) & frag,
                              const MEM_T *const ptr, const unsigned ldm,
                              const layout_t layout, const bool sync = true) {
  if (layout == mem_col_major)
    load_matrix_sync<col_major>(frag, ptr, ldm, sync);
  else
    load_matrix_sync<row_major>(frag, ptr, ldm, sync);
}
template <WMMAE_TCEC_TPARAMS, class MEM_T>
WMMAE_D void load_matrix_sync_with_mul(WMMAE_TCEC_FRAG(accumulator, void) &
                                           frag,
                                       const MEM_T *const ptr,
                                       const unsigned ldm, const MEM_T mul,
                                       const layout_t layout,
                                       const bool sync = true) {
  if (layout == mem_col_major)
    load_matrix_sync_with_mul<col_major>(frag, ptr, ldm, mul, sync);
  else
    load_matrix_sync_with_mul<row_major>(frag, ptr, ldm, mul, sync);
}

// ----------------------------------------------------------- store matrix
template <class Layout, WMMAE_TCEC_TPARAMS, class MEM_T>
WMMAE_D void
store_matrix_sync_with_mul(MEM_T *const ptr,
                           const WMMAE_TCEC_FRAG(accumulator, void) & frag,
                           const unsigned ldm, const MEM_T mul,
                           const bool = true) {
  using F = WMMAE_TCEC_FRAG(accumulator, void);
  if constexpr (std::is_same<Layout, col_major>::value &&
                mtk::wmma::detail::acc_quads<fm, fn, fk, float,
                                             MEM_T>::value) {
    if (mtk::wmma::detail::quad_aligned(ptr, ldm)) {
      using L = typename F::sub_frag_t::layout_model;
      const unsigned lane = mtk::wmma::detail::common::get_lane_id();
#pragma unroll
      for (unsigned bn = 0; bn < unsigned(F::num_sub_frag_n); bn++) {
#pragma unroll
        for (unsigned bm = 0; bm < unsigned(F::num_sub_frag_m); bm++) {
          const unsigned block = bm + F::num_sub_frag_m * bn;
#pragma unroll
          for (unsigned x = 0; x < L::num_elements; x += 4) {
            detail::f32x4_t v;
#pragma unroll
            for (unsigned e = 0; e < 4; e++)
              v[e] = detail::combined(frag, block, x + e) *
                     static_cast<float>(mul);
            *reinterpret_cast<detail::f32x4_t *>(
                ptr + detail::mem_offset<col_major>(L::row(lane, x),
                                                    L::col(lane, x), ldm,
                                                    bm * fm, bn * fn)) = v;
          }
        }
      }
      return;
    }
  }
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
            ptr[off] = static_cast<MEM_T>(
                detail::combined(frag, block, list[0]) *
                static_cast<float>(mul));
          }
        }
      });
}
template <class Layout, WMMAE_TCEC_TPARAMS, class MEM_T>
WMMAE_D void store_matrix_sync(MEM_T *const ptr,
                               const WMMAE_TCEC_FRAG(accumulator, void) & frag,
                               const unsigned ldm, const bool sync = true) {
  store_matrix_sync_with_mul<Layout>(ptr, frag, ldm, static_cast<MEM_T>(1),
                                     sync);
}
template <WMMAE_TCEC_TPARAMS, class MEM_T>
WMMAE_D void store_matrix_sync(MEM_T *const ptr,
                               const WMMAE_TCEC_FRAG(accumulator, void) & frag,
                               const unsigned ldm, const layout_t layout,
                               const bool sync = true) {
  if (layout == mem_col_major)
    store_matrix_sync<col_major>(ptr, frag, ldm, sync);
  else
    store_matrix_sync<row_major>(ptr, frag, ldm, sync);
}
template <WMMAE_TCEC_TPARAMS, class MEM_T>
WMMAE_D void
store_matrix_sync_with_mul(MEM_T *const ptr,
                           const WMMAE_TCEC_FRAG(accumulator, void) & frag,
                           const unsigned ldm, const MEM_T mul,
                           const layout_t layout, const bool sync = true) {
  if (layout == mem_col_major)
    store_matrix_sync_with_mul<col_major>(ptr, frag, ldm, mul, sync);
  else
    store_matrix_sync_with_mul<row_major>(ptr, frag, ldm, mul, sync);
}

// ------------------------------------------------------------ load vector
// Operands: the vector goes into the first column (col_major fragment) or
// first row (row_major fragment) of the m x k / k x n tile; only the
// sub-blocks on that edge are written, the caller zero-fills first
// (reference: tcec/tcec.hpp:450-536; test/tcec/matvec.cu:41-42).
template <class Use, WMMAE_TCEC_TPARAMS, class Layout, class MEM_T>
WMMAE_D void load_vector(WMMAE_TCEC_FRAG(Use, Layout) & frag,
                         const MEM_T *const ptr, const MEM_T mul) {
  using F = WMMAE_TCEC_FRAG(Use, Layout);
  static_assert(!F::is_acc, "accumulator load_vector needs a layout_t");
  constexpr unsigned bm_size = detail::select_value<Use, fm, fk, fm>::value;
  constexpr unsigned bn_size = detail::select_value<Use, fk, fn, fn>::value;
  constexpr unsigned num_blocks =
      detail::layout_switch<Layout, F::num_sub_frag_m,
                            F::num_sub_frag_n>::value;
  constexpr unsigned block_ld =
      detail::layout_switch<Layout, 1, F::num_sub_frag_m>::value;
  constexpr unsigned vec_per_block =
      detail::layout_switch<Layout, bm_size, bn_size>::value;
  mtk::wmma::foreach_v<typename F::sub_frag_t>(
      [&](const unsigned *list, const unsigned, const unsigned mem_index) {
#pragma unroll
        for (unsigned b = 0; b < num_blocks; b++) {
          const float v =
              static_cast<float>(ptr[mem_index + b * vec_per_block]) *
              static_cast<float>(mul);
          detail::put_split(frag, b * block_ld, list[0], v);
        }
      });
}
template <class Use, WMMAE_TCEC_TPARAMS, class Layout, class MEM_T>
WMMAE_D void load_vector(WMMAE_TCEC_FRAG(Use, Layout) & frag,
                         const MEM_T *const ptr) {
  load_vector(frag, ptr, static_cast<MEM_T>(1));
}

// Accumulators: first column (mem_col_major) or first row (mem_row_major).
// The touched main sub-blocks are zeroed and then receive the vector; the
// error part is left as it is (reference: tcec/tcec.hpp:421-448, which
// forwards to the primitive load_vector with its default fill).
template <WMMAE_TCEC_TPARAMS, class MEM_T>
WMMAE_D void load_vector(WMMAE_TCEC_FRAG(accumulator, void) & frag,
                         const MEM_T *const ptr, const layout_t layout) {
  using F = WMMAE_TCEC_FRAG(accumulator, void);
  if (layout == mem_col_major) {
#pragma unroll
    for (unsigned bm = 0; bm < unsigned(F::num_sub_frag_m); bm++)
      mtk::wmma::load_vector(frag.sub_frag[bm], ptr + bm * fm, layout);
  } else {
#pragma unroll
    for (unsigned bn = 0; bn < unsigned(F::num_sub_frag_n); bn++)
      mtk::wmma::load_vector(frag.sub_frag[bn * F::num_sub_frag_m],
                             ptr + bn * fn, layout);
  }
}

// ----------------------------------------------------------- store vector
template <WMMAE_TCEC_TPARAMS, class MEM_T>
WMMAE_D void store_vector(MEM_T *const ptr,
                          const WMMAE_TCEC_FRAG(accumulator, void) & frag,
                          const MEM_T mul, const layout_t layout) {
  using F = WMMAE_TCEC_FRAG(accumulator, void);
  const bool col = layout == mem_col_major;
  mtk::wmma::foreach_v<typename F::sub_frag_t>(
      layout,
      [&](const unsigned *list, const unsigned, const unsigned mem_index) {
        if (col) {
#pragma unroll
          for (unsigned bm = 0; bm < unsigned(F::num_sub_frag_m); bm++)
            ptr[bm * fm + mem_index] = static_cast<MEM_T>(
                detail::combined(frag, bm, list[0]) * static_cast<float>(mul));
        } else {
#pragma unroll
          for (unsigned bn = 0; bn < unsigned(F::num_sub_frag_n); bn++)
            ptr[bn * fn + mem_index] = static_cast<MEM_T>(
                detail::combined(frag, bn * F::num_sub_frag_m, list[0]) *
                static_cast<float>(mul));
        }
      });
}
template <WMMAE_TCEC_TPARAMS, class MEM_T>
WMMAE_D void store_vector(MEM_T *const ptr,
                          const WMMAE_TCEC_FRAG(accumulator, void) & frag,
                          const layout_t layout) {
  store_vector(ptr, frag, static_cast<MEM_T>(1), layout);
}

// -------------------------------------------------------------------- mma
// d = a*b + c over the sub-block grid.  With error correction the products
//   main:  a0*b0
//   error: a1*b0 + a0*b1                      (two-term splits)
//          + a1*b1 + a2*b0 + a0*b2            (three-term split)
// are issued as separate MFMAs; a1*b1 of the two-term split and the
// higher-order products of the three-term split are below fp32 resolution
// and dropped (reference: tcec/tcec.hpp:640-706).
namespace detail {
template <bool main_outside, bool use_c, WMMAE_TCEC_TPARAMS, class LA, class LB>
WMMAE_D void mma_core(WMMAE_TCEC_FRAG(accumulator, void) & d,
                      const WMMAE_TCEC_FRAG(matrix_a, LA) & a,
                      const WMMAE_TCEC_FRAG(matrix_b, LB) & b,
                      const WMMAE_TCEC_FRAG(accumulator, void) * c) {
  using FD = WMMAE_TCEC_FRAG(accumulator, void);
  using FA = WMMAE_TCEC_FRAG(matrix_a, LA);
  constexpr unsigned nmb = FD::num_sub_frag_m;
  constexpr unsigned nnb = FD::num_sub_frag_n;
  constexpr unsigned nkb = FA::num_sub_frag_n;
  constexpr int terms = FA::num_terms;
#pragma unroll
  for (unsigned bm = 0; bm < nmb; bm++) {
#pragma unroll
    for (unsigned bn = 0; bn < nnb; bn++) {
      const unsigned cd = bm + bn * nmb;
      typename FD::sub_frag_t main_acc, err_acc;
      if constexpr (use_c) {
        main_acc = c->sub_frag[cd];
        if constexpr (terms >= 2)
          err_acc = c->sub_d_frag[cd];
      } else {
        mtk::wmma::fill_zero(main_acc);
        mtk::wmma::fill_zero(err_acc);
      }
#pragma unroll
      for (unsigned bk = 0; bk < nkb; bk++) {
        const unsigned ia = bm + bk * nmb;
        const unsigned ib = bk + bn * nkb;
        if constexpr (main_outside) {
          // round-to-nearest variant: the main product starts from a zero
          // accumulator and is added to the running sum with an fp32 add.
          typename FD::sub_frag_t tmp;
          mtk::wmma::fill_zero(tmp);
          mtk::wmma::mma_sync(tmp, a.sub_frag[ia], b.sub_frag[ib], tmp);
#pragma unroll
          for (unsigned i = 0; i < tmp.num_elements; i++)
            main_acc.x[i] += tmp.x[i];
        } else {
          mtk::wmma::mma_sync(main_acc, a.sub_frag[ia], b.sub_frag[ib],
                              main_acc);
        }
        if constexpr (terms >= 3) {
          mtk::wmma::mma_sync(err_acc, a.sub_d2_frag[ia], b.sub_frag[ib],
                              err_acc);
          mtk::wmma::mma_sync(err_acc, a.sub_frag[ia], b.sub_d2_frag[ib],
                              err_acc);
          mtk::wmma::mma_sync(err_acc, a.sub_d_frag[ia], b.sub_d_frag[ib],
                              err_acc);
        }
        if constexpr (terms >= 2) {
          mtk::wmma::mma_sync(err_acc, a.sub_d_frag[ia], b.sub_frag[ib],
                              err_acc);
          mtk::wmma::mma_sync(err_acc, a.sub_frag[ia], b.sub_d_frag[ib],
                              err_acc);
        }
      }
      d.sub_frag[cd] = main_acc;
      if constexpr (terms >= 2)
        d.sub_d_frag[cd] = err_acc;
    }
  }
}
} // namespace detail

// mma_rn_sync: main term accumulated with fp32 adds outside the matrix core.
template <WMMAE_TCEC_TPARAMS, class LA, class LB>
WMMAE_D void mma_rn_sync(WMMAE_TCEC_FRAG(accumulator, void) & d,
                         const WMMAE_TCEC_FRAG(matrix_a, LA) & a,
                         const WMMAE_TCEC_FRAG(matrix_b, LB) & b,
                         const WMMAE_TCEC_FRAG(accumulator, void) & c) {
  detail::mma_core<true, true>(d, a, b, &c);
}
template <WMMAE_TCEC_TPARAMS, class LA, class LB>
WMMAE_D void mma_rn_sync(WMMAE_TCEC_FRAG(accumulator, void) & d,
                         const WMMAE_TCEC_FRAG(matrix_a, LA) & a,
                         const WMMAE_TCEC_FRAG(matrix_b, LB) & b) {
  detail::mma_core<true, false>(
      d, a, b, static_cast<const WMMAE_TCEC_FRAG(accumulator, void) *>(nullptr));
}
// mma_rz_sync: main term chained through the matrix core's own accumulator
// (named after the truncating accumulate of the reference's hardware).
template <WMMAE_TCEC_TPARAMS, class LA, class LB>
WMMAE_D void mma_rz_sync(WMMAE_TCEC_FRAG(accumulator, void) & d,
                         const WMMAE_TCEC_FRAG(matrix_a, LA) & a,
                         const WMMAE_TCEC_FRAG(matrix_b, LB) & b,
                         const WMMAE_TCEC_FRAG(accumulator, void) & c) {
  detail::mma_core<false, true>(d, a, b, &c);
}
template <WMMAE_TCEC_TPARAMS, class LA, class LB>
WMMAE_D void mma_rz_sync(WMMAE_TCEC_FRAG(accumulator, void) & d,
                         const WMMAE_TCEC_FRAG(matrix_a, LA) & a,
                         const WMMAE_TCEC_FRAG(matrix_b, LB) & b) {
  detail::mma_core<false, false>(
      d, a, b, static_cast<const WMMAE_TCEC_FRAG(accumulator, void) *>(nullptr));
}

// Default: with_ec -> mma_rn_sync (tcec.hpp:896-927); without_ec ->
// mma_rz_sync (no_cor.hpp:858-897, docs/mma_f32.md:131-135).
template <WMMAE_TCEC_TPARAMS, class LA, class LB>
WMMAE_D void mma_sync(WMMAE_TCEC_FRAG(accumulator, void) & d,
                      const WMMAE_TCEC_FRAG(matrix_a, LA) & a,
                      const WMMAE_TCEC_FRAG(matrix_b, LB) & b,
                      const WMMAE_TCEC_FRAG(accumulator, void) & c) {
  if constexpr (std::is_same<EC, with_ec>::value)
    mma_rn_sync(d, a, b, c);
  else
    mma_rz_sync(d, a, b, c);
}
template <WMMAE_TCEC_TPARAMS, class LA, class LB>
WMMAE_D void mma_sync(WMMAE_TCEC_FRAG(accumulator, void) & d,
                      const WMMAE_TCEC_FRAG(matrix_a, LA) & a,
                      const WMMAE_TCEC_FRAG(matrix_b, LB) & b) {
  if constexpr (std::is_same<EC, with_ec>::value)
    mma_rn_sync(d, a, b);
  else
    mma_rz_sync(d, a, b);
}

// ------------------------------------------------------------ debug print
template <class Use, WMMAE_TCEC_TPARAMS, class Layout>
__device__ inline void print_fragment(const WMMAE_TCEC_FRAG(Use, Layout) & frag,
                                      const char *const name = "") {
  using F = WMMAE_TCEC_FRAG(Use, Layout);
  const unsigned lane = mtk::wmma::detail::common::get_lane_id();
  if (lane == 0 && name[0] != '\0')
    printf("%s = \n", name);
  for (unsigned l = 0; l < wave_size; l++) {
    if (l == lane) {
      for (unsigned i = 0; i < F::num_elements; i++) {
        if constexpr (F::num_terms >= 2)
          printf("(%+.3e)+(%+.3e) ", static_cast<float>(frag.x(i)),
                 detail::correction_scale_1<T>(static_cast<float>(frag.dx(i))));
        else
          printf("(%+.3e) ", static_cast<float>(frag.x(i)));
      }
      printf("\n");
    }
  }
}

#undef WMMAE_TCEC_TPARAMS
#undef WMMAE_TCEC_FRAG

} // namespace tcec

// Historic name of the same API.
namespace mma_f32 = tcec;

} // namespace wmma
} // namespace mtk
