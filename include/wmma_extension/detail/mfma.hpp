// Binding of fragment shapes to gfx950 MFMA instructions.
//
// This is the layer the reference gets from CUDA's nvcuda::wmma::mma_sync and
// from inline PTX mma.sync (reference: tcec/detail/functions.hpp:313-348,
// detail/m16n8k16.hpp:265-287, detail/m16n8k8_tf32.hpp:154-176).
#pragma once
#include "common.hpp"

namespace mtk {
namespace wmma {
namespace detail {
namespace gfx950 {

template <class T, int n> using vec_t = T __attribute__((ext_vector_type(n)));

// mfma_op<T,M,N,K>::run(a, b, c) returns a*b + c for one wave64.
template <class T, int M, int N, int K> struct mfma_op;

#define WMMAE_MFMA_OP(T_, M_, N_, K_, AB_T, AB_N, C_N, BUILTIN)                \
  template <> struct mfma_op<T_, M_, N_, K_> {                                 \
    using ab_vec = vec_t<AB_T, AB_N>;                                          \
    using c_vec = vec_t<float, C_N>;                                           \
    static WMMAE_D c_vec run(const ab_vec a, const ab_vec b, const c_vec c) {  \
      return BUILTIN(a, b, c, 0, 0, 0);                                        \
    }                                                                          \
  }

WMMAE_MFMA_OP(half, 16, 16, 16, _Float16, 4, 4,
              __builtin_amdgcn_mfma_f32_16x16x16f16);
WMMAE_MFMA_OP(half, 16, 16, 32, _Float16, 8, 4,
              __builtin_amdgcn_mfma_f32_16x16x32_f16);
WMMAE_MFMA_OP(half, 32, 32, 8, _Float16, 4, 16,
              __builtin_amdgcn_mfma_f32_32x32x8f16);
WMMAE_MFMA_OP(half, 32, 32, 16, _Float16, 8, 16,
              __builtin_amdgcn_mfma_f32_32x32x16_f16);
WMMAE_MFMA_OP(bfloat16, 16, 16, 32, __bf16, 8, 4,
              __builtin_amdgcn_mfma_f32_16x16x32_bf16);
WMMAE_MFMA_OP(bfloat16, 32, 32, 16, __bf16, 8, 16,
              __builtin_amdgcn_mfma_f32_32x32x16_bf16);
#undef WMMAE_MFMA_OP

// The K=16 / K=8 bf16 instructions (the "_1k" forms) take their operands as
// vectors of 16-bit integers.
template <> struct mfma_op<bfloat16, 16, 16, 16> {
  using ab_vec = vec_t<__bf16, 4>;
  using c_vec = vec_t<float, 4>;
  static WMMAE_D c_vec run(const ab_vec a, const ab_vec b, const c_vec c) {
    using s4 = vec_t<short, 4>;
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
        __builtin_bit_cast(s4, a), __builtin_bit_cast(s4, b), c, 0, 0, 0);
  }
};
template <> struct mfma_op<bfloat16, 32, 32, 8> {
  using ab_vec = vec_t<__bf16, 4>;
  using c_vec = vec_t<float, 16>;
  static WMMAE_D c_vec run(const ab_vec a, const ab_vec b, const c_vec c) {
    using s4 = vec_t<short, 4>;
    return __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(
        __builtin_bit_cast(s4, a), __builtin_bit_cast(s4, b), c, 0, 0, 0);
  }
};

// fp32 operands on the matrix core: one k per lane group.
template <> struct mfma_op<float, 16, 16, 4> {
  using ab_vec = float;
  using c_vec = vec_t<float, 4>;
  static WMMAE_D c_vec run(const ab_vec a, const ab_vec b, const c_vec c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
};
template <> struct mfma_op<float, 32, 32, 2> {
  using ab_vec = float;
  using c_vec = vec_t<float, 16>;
  static WMMAE_D c_vec run(const ab_vec a, const ab_vec b, const c_vec c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
};

// A 16x16x16 fp32 product as four chained 16x16x4 steps.  Register x of an
// operand fragment holds k = 4*(lane/16) + x, and step x of the chain consumes
// register x of both operands, so every k is used exactly once; inside a step
// the four lane groups supply k = x, 4+x, 8+x, 12+x.
template <> struct mfma_op<float, 16, 16, 16> {
  using ab_vec = vec_t<float, 4>;
  using c_vec = vec_t<float, 4>;
  static WMMAE_D c_vec run(const ab_vec a, const ab_vec b, c_vec c) {
#pragma unroll
    for (int x = 0; x < 4; x++)
      c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[x], b[x], c, 0, 0, 0);
    return c;
  }
};
// 32x32x8 fp32 as four chained 32x32x2 steps (k = 4*(lane/32) + x).
template <> struct mfma_op<float, 32, 32, 8> {
  using ab_vec = vec_t<float, 4>;
  using c_vec = vec_t<float, 16>;
  static WMMAE_D c_vec run(const ab_vec a, const ab_vec b, c_vec c) {
#pragma unroll
    for (int x = 0; x < 4; x++)
      c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[x], b[x], c, 0, 0, 0);
    return c;
  }
};

} // namespace gfx950
} // namespace detail

// d = a * b + c on the matrix core.  The fragment Layout arguments only record
// how the caller filled the fragment; the registers are layout independent.
template <int M, int N, int K, class T, class LA, class LB>
WMMAE_D void mma_sync(fragment<accumulator, M, N, K, float> &d,
                      const fragment<matrix_a, M, N, K, T, LA> &a,
                      const fragment<matrix_b, M, N, K, T, LB> &b,
                      const fragment<accumulator, M, N, K, float> &c) {
  using S = typename detail::common::storage_t<T>::type;
  using op = detail::gfx950::mfma_op<S, M, N, K>;
  typename op::ab_vec av, bv;
  typename op::c_vec cv;
  __builtin_memcpy(&av, a.x, sizeof(av));
  __builtin_memcpy(&bv, b.x, sizeof(bv));
  __builtin_memcpy(&cv, c.x, sizeof(cv));
  cv = op::run(av, bv, cv);
  __builtin_memcpy(d.x, &cv, sizeof(cv));
}

} // namespace wmma
} // namespace mtk
