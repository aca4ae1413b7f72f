// Vocabulary types, element traits and the gfx950 (wave64 MFMA) register
// layout model used by every other header of this library.
//
// The reference borrows its vocabulary (matrix_a, row_major, layout_t,
// precision::tf32, fragment<>) from CUDA's <mma.h> (reference:
// include/wmma_extension/detail/common.hpp:1-101).  gfx950 has no such vendor
// header, so the same names are defined natively here, in mtk::wmma.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <type_traits>
#if __has_include(<hip/hip_fp16.h>)
#include <hip/hip_fp16.h>
#define WMMAE_HAS_HIP_FP16 1
#endif

#define WMMAE_HD __host__ __device__ __forceinline__
#define WMMAE_D __device__ __forceinline__

namespace mtk {
namespace wmma {

// ---- fragment roles and layouts -------------------------------------------
struct matrix_a;
struct matrix_b;
struct accumulator;
struct row_major;
struct col_major;
enum layout_t { mem_row_major, mem_col_major };

// ---- element tags -----------------------------------------------------------
// half / bfloat16 are the compiler's native 16-bit types; the MFMA builtins
// take vectors of exactly these.
using half = _Float16;
using bfloat16 = __bf16;
namespace precision {
// gfx950 has no xf32 MFMA.  At the primitive level a tf32 fragment element is
// stored as fp32 rounded to 10 explicit mantissa bits; in TCEC the tf32 tag
// selects the three-term bf16 split (see tcec/detail/split.hpp).
struct tf32;
} // namespace precision

constexpr unsigned wave_size = 64;

namespace detail {
namespace common {

// storage_t: the register type behind an element tag
// (reference: detail/common.hpp:22-36).
template <class T> struct storage_t {
  using type = T;
};
template <> struct storage_t<precision::tf32> {
  using type = float;
};
#ifdef WMMAE_HAS_HIP_FP16
template <> struct storage_t<__half> {
  using type = _Float16;
};
#endif

// fp32 -> tf32 (10 explicit mantissa bits in an fp32 container), round to
// nearest with ties away from zero: the reference converts with PTX
// cvt.rna.tf32.f32 (detail/common.hpp:36-48).  On the sign-magnitude bit
// pattern that is "add half a unit of the kept precision, drop the low 13
// bits".  inf / nan pass through.
WMMAE_HD float to_tf32(const float a) {
  uint32_t u = __builtin_bit_cast(uint32_t, a);
  if ((u & 0x7f800000u) == 0x7f800000u)
    return a;
  u = (u + 0x00001000u) & 0xffffe000u;
  return __builtin_bit_cast(float, u);
}

// cast<T>(v): convert v to the storage type of tag T: round to nearest even
// for half and bfloat16, ties away from zero for precision::tf32, as in the
// reference (detail/common.hpp:25-61).
template <class T, class S>
WMMAE_HD typename storage_t<T>::type cast(const S v) {
  if constexpr (std::is_same<T, precision::tf32>::value) {
    return to_tf32(static_cast<float>(v));
  } else if constexpr (std::is_same<typename storage_t<T>::type,
                                    bfloat16>::value &&
                       !std::is_same<S, bfloat16>::value) {
    return static_cast<bfloat16>(static_cast<float>(v));
  } else if constexpr (std::is_same<S, bfloat16>::value &&
                       !std::is_same<typename storage_t<T>::type,
                                     bfloat16>::value) {
    return static_cast<typename storage_t<T>::type>(static_cast<float>(v));
  } else {
    return static_cast<typename storage_t<T>::type>(v);
  }
}

// Lane index inside the wave64 (reference: detail/common.hpp:63-67 reads
// %laneid of a 32-wide warp).
WMMAE_D unsigned get_lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

template <class Use, int a, int b, int c> struct select_value;
template <int a, int b, int c> struct select_value<matrix_a, a, b, c> {
  static constexpr int value = a;
};
template <int a, int b, int c> struct select_value<matrix_b, a, b, c> {
  static constexpr int value = b;
};
template <int a, int b, int c> struct select_value<accumulator, a, b, c> {
  static constexpr int value = c;
};

// Rows / columns of the tile a fragment of the given role covers
// (reference: detail/common.hpp:69-91).
template <class Use, int M, int N, int K> struct get_M {
  static constexpr int value = select_value<Use, M, K, M>::value;
};
template <class Use, int M, int N, int K> struct get_N {
  static constexpr int value = select_value<Use, K, N, N>::value;
};

template <class Layout, int col_value, int row_value> struct layout_switch;
template <int col_value, int row_value>
struct layout_switch<col_major, col_value, row_value> {
  static constexpr int value = col_value;
};
template <int col_value, int row_value>
struct layout_switch<row_major, col_value, row_value> {
  static constexpr int value = row_value;
};

} // namespace common

// ---------------------------------------------------------------------------
// gfx950 MFMA register layout model.
//
// For v_mfma_f32_{16x16x16,16x16x32,32x32x8,32x32x16}_{f16,bf16} and
// v_mfma_f32_{16x16x4,32x32x2}_f32 a wave64 holds
//   A (M x K): lane l, register x  ->  A[l % M][P*(l / M) + x],  P = K*M/64
//   B (K x N): lane l, register x  ->  B[P*(l / N) + x][l % N],  P = K*N/64
//   D (M x N): lane l, register x  ->  D[(256/N)*(x/4) + 4*(l / N) + x%4][l % N]
// Every (i,j) lives in exactly one (lane, register): unlike the NVIDIA tables
// of the reference (detail/sm_80.hpp:9-402) nothing is duplicated, and the
// register assignment does not depend on the Layout template argument.
// ---------------------------------------------------------------------------
namespace gfx950 {

template <class Use, int M, int N, int K> struct frag_layout;

template <int M, int N, int K> struct frag_layout<matrix_a, M, N, K> {
  static_assert(M == 16 || M == 32, "MFMA A tiles have 16 or 32 rows");
  static constexpr unsigned rows = M, cols = K;
  static constexpr unsigned groups = wave_size / M;
  static constexpr unsigned num_elements = K / groups;
  static_assert(num_elements * groups == unsigned(K), "K not divisible");
  static WMMAE_HD constexpr unsigned row(unsigned lane, unsigned) {
    return lane % M;
  }
  static WMMAE_HD constexpr unsigned col(unsigned lane, unsigned x) {
    return num_elements * (lane / M) + x;
  }
  static WMMAE_HD constexpr unsigned tid(unsigned i, unsigned j) {
    return i + M * (j / num_elements);
  }
  static WMMAE_HD constexpr unsigned fid(unsigned, unsigned j) {
    return j % num_elements;
  }
};

template <int M, int N, int K> struct frag_layout<matrix_b, M, N, K> {
  static_assert(N == 16 || N == 32, "MFMA B tiles have 16 or 32 columns");
  static constexpr unsigned rows = K, cols = N;
  static constexpr unsigned groups = wave_size / N;
  static constexpr unsigned num_elements = K / groups;
  static_assert(num_elements * groups == unsigned(K), "K not divisible");
  static WMMAE_HD constexpr unsigned row(unsigned lane, unsigned x) {
    return num_elements * (lane / N) + x;
  }
  static WMMAE_HD constexpr unsigned col(unsigned lane, unsigned) {
    return lane % N;
  }
  static WMMAE_HD constexpr unsigned tid(unsigned i, unsigned j) {
    return j + N * (i / num_elements);
  }
  static WMMAE_HD constexpr unsigned fid(unsigned i, unsigned) {
    return i % num_elements;
  }
};

template <int M, int N, int K> struct frag_layout<accumulator, M, N, K> {
  static_assert((M == 16 && N == 16) || (M == 32 && N == 32),
                "MFMA accumulators are 16x16 or 32x32");
  static constexpr unsigned rows = M, cols = N;
  static constexpr unsigned groups = wave_size / N;
  static constexpr unsigned num_elements = M * N / wave_size;
  static constexpr unsigned block_rows = 4 * groups; // rows covered per 4 regs
  static WMMAE_HD constexpr unsigned row(unsigned lane, unsigned x) {
    return block_rows * (x / 4) + 4 * (lane / N) + (x % 4);
  }
  static WMMAE_HD constexpr unsigned col(unsigned lane, unsigned) {
    return lane % N;
  }
  static WMMAE_HD constexpr unsigned tid(unsigned i, unsigned j) {
    return j + N * ((i % block_rows) / 4);
  }
  static WMMAE_HD constexpr unsigned fid(unsigned i, unsigned) {
    return 4 * (i / block_rows) + (i % 4);
  }
};

} // namespace gfx950
} // namespace detail

// ---------------------------------------------------------------------------
// fragment: the per-lane registers of one MFMA operand tile.  Same members as
// the CUDA fragment the reference builds on: x[], num_elements, element_type.
// ---------------------------------------------------------------------------
template <class T, int size> struct __frag_base {
  using element_type = T;
  using storage_element_type = typename detail::common::storage_t<T>::type;
  static constexpr unsigned num_elements = size;
  // 16-byte alignment lets mma_sync reinterpret x[] as the MFMA vector operand.
  alignas(size * sizeof(storage_element_type) >= 16
              ? 16
              : size * sizeof(storage_element_type)) storage_element_type
      x[size];
};

template <class Use, int M, int N, int K, class T, class Layout = void>
struct fragment
    : public __frag_base<
          T, detail::gfx950::frag_layout<Use, M, N, K>::num_elements> {
  using layout_model = detail::gfx950::frag_layout<Use, M, N, K>;
  using use = Use;
  using layout = Layout;
  static constexpr int m = M, n = N, k = K;
};

template <class Frag> struct is_fragment : std::false_type {};
template <class Use, int M, int N, int K, class T, class Layout>
struct is_fragment<fragment<Use, M, N, K, T, Layout>> : std::true_type {};

} // namespace wmma
} // namespace mtk
