// extern "C" boundary of libwmmae_tcec.so, device-API harness part: entry
// points that run the reference's one-wave test kernels, rebuilt on the
// gfx950 headers, on caller-provided device buffers.  Declarations and
// per-entry documentation live in include/wmmae_tcec.h.
#include "capi_common.hpp"
#include "harness_kernels.hpp"

using namespace wmmae_capi;

extern "C" {

// ------------------------------------------------------------ harness
int wmmae_primitive_tiles(const float *const tiles, const long long num_tiles,
                          void *const a_row, void *const a_col,
                          void *const b_row, void *const b_col,
                          float *const acc_out, float *const vec_out,
                          void *const stream) {
  if (num_tiles < 0)
    return WMMAE_STATUS_INVALID_VALUE;
  if (num_tiles == 0)
    return WMMAE_STATUS_SUCCESS;
  if (!tiles || !a_row || !a_col || !b_row || !b_col || !acc_out || !vec_out)
    return WMMAE_STATUS_NULL_POINTER;
  long long blocks = (num_tiles + 3) / 4; // 4 waves per block, one tile per wave
  if (blocks > (1 << 20))
    blocks = 1 << 20; // grid-stride beyond this
  hipLaunchKernelGGL(wmmae_harness::primitive_tiles_kernel,
                     dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), tiles, num_tiles,
                     static_cast<w::half *>(a_row), static_cast<w::half *>(a_col),
                     static_cast<w::half *>(b_row), static_cast<w::half *>(b_col),
                     acc_out, vec_out);
  return launch_status();
}

} // extern "C"

namespace {
template <class Frag>
int launch_layout_dump(const int col, int *ij, int *mem_index, int *v_index,
                       int *map_tid, int *map_fid, hipStream_t s) {
  hipLaunchKernelGGL((wmmae_harness::layout_dump_kernel<Frag>), dim3(1),
                     dim3(64), 0, s, col, ij, mem_index, v_index, map_tid,
                     map_fid);
  return launch_status();
}
template <int M, int N, int K>
int layout_dump_shape(const int use, const int col, int *ij, int *mem_index,
                      int *v_index, int *map_tid, int *map_fid,
                      hipStream_t s) {
  if (use == 0) {
    return col ? launch_layout_dump<
                     w::fragment<w::matrix_a, M, N, K, w::half, w::col_major>>(
                     col, ij, mem_index, v_index, map_tid, map_fid, s)
               : launch_layout_dump<
                     w::fragment<w::matrix_a, M, N, K, w::half, w::row_major>>(
                     col, ij, mem_index, v_index, map_tid, map_fid, s);
  }
  if (use == 1) {
    return col ? launch_layout_dump<
                     w::fragment<w::matrix_b, M, N, K, w::half, w::col_major>>(
                     col, ij, mem_index, v_index, map_tid, map_fid, s)
               : launch_layout_dump<
                     w::fragment<w::matrix_b, M, N, K, w::half, w::row_major>>(
                     col, ij, mem_index, v_index, map_tid, map_fid, s);
  }
  if (use == 2)
    return launch_layout_dump<w::fragment<w::accumulator, M, N, K, float>>(
        col, ij, mem_index, v_index, map_tid, map_fid, s);
  return WMMAE_STATUS_INVALID_VALUE;
}
} // namespace

extern "C" {

int wmmae_layout_dump(const int use, const int m, const int n, const int k,
                      const int col, int *const ij, int *const mem_index,
                      int *const v_index, int *const map_tid,
                      int *const map_fid, void *const stream) {
  if (!ij || !mem_index || !v_index || !map_tid || !map_fid)
    return WMMAE_STATUS_NULL_POINTER;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define WMMAE_SHAPE(M_, N_, K_)                                                \
  if (m == M_ && n == N_ && k == K_)                                           \
    return layout_dump_shape<M_, N_, K_>(use, col, ij, mem_index, v_index,     \
                                         map_tid, map_fid, s);
  WMMAE_SHAPE(16, 16, 16)
  WMMAE_SHAPE(16, 16, 32)
  WMMAE_SHAPE(32, 32, 8)
  WMMAE_SHAPE(32, 32, 16)
#undef WMMAE_SHAPE
  return WMMAE_STATUS_NOT_SUPPORTED;
}

} // extern "C"


extern "C" {

int wmmae_tcec_mma_tile(const int shape, const int type, const int ec,
                        const int inst, float *const d, const float *const a,
                        const float *const b, const float *const c,
                        const int a_col, const int b_col, const int c_col,
                        const int d_col, const int rounding,
                        void *const stream) {
  if (!d || !a || !b)
    return WMMAE_STATUS_NULL_POINTER;
  if (shape < 0 || shape > 1 || inst < 0 || inst > 2 || rounding < 0 ||
      rounding > 2)
    return WMMAE_STATUS_INVALID_VALUE;
  if (!type_ec_supported(type, ec))
    return WMMAE_STATUS_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return with_type(type, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_ec(ec, [&](auto te) {
      using EC = typename decltype(te)::type;
      auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(1), dim3(64), 0, s, d, a, b, c, a_col,
                           b_col, c_col, d_col, rounding);
        return launch_status();
      };
      using R = w::row_major;
      using Cm = w::col_major;
      if (inst == 0) {
        using P = typename harness_policy<T, EC, 16, 16, 32>::type;
        return shape == 0
                   ? go(wmmae_harness::tcec_mma_tile_kernel<32, 32, 32, T, P, R,
                                                            Cm>)
                   : go(wmmae_harness::tcec_mma_tile_kernel<16, 48, 64, T, P, R,
                                                            Cm>);
      }
      if (inst == 1) {
        using P = typename harness_policy<T, EC, 16, 16, 16>::type;
        return shape == 0
                   ? go(wmmae_harness::tcec_mma_tile_kernel<32, 32, 32, T, P, R,
                                                            Cm>)
                   : go(wmmae_harness::tcec_mma_tile_kernel<16, 48, 64, T, P, R,
                                                            Cm>);
      }
      using P = typename harness_policy<T, EC, 32, 32, 16>::type;
      return shape == 0
                 ? go(wmmae_harness::tcec_mma_tile_kernel<32, 32, 32, T, P, R,
                                                          Cm>)
                 : go(wmmae_harness::tcec_mma_tile_kernel<32, 64, 32, T, P, R,
                                                          Cm>);
    });
  });
}

int wmmae_tcec_mma_tile_native(const int type, const int ec,
                               const int a_frag_col, const int b_frag_col,
                               float *const d, const float *const a,
                               const float *const b, const int d_col,
                               void *const stream) {
  if (!d || !a || !b)
    return WMMAE_STATUS_NULL_POINTER;
  if (!type_ec_supported(type, ec))
    return WMMAE_STATUS_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return with_type(type, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_ec(ec, [&](auto te) {
      using EC = typename decltype(te)::type;
      using P = typename harness_policy<T, EC, 16, 16, 32>::type;
      return with_layout(a_frag_col, [&](auto la) {
        using AL = typename decltype(la)::type;
        return with_layout(b_frag_col, [&](auto lb) {
          using BL = typename decltype(lb)::type;
          hipLaunchKernelGGL(
              (wmmae_harness::tcec_mma_tile_native_kernel<32, 32, 32, T, P, AL,
                                                          BL>),
              dim3(1), dim3(64), 0, s, d, a, b, d_col);
          return launch_status();
        });
      });
    });
  });
}

int wmmae_tcec_matvec(const int type, const int ec, float *const y,
                      const float *const a, const float *const x,
                      const int a_col, const int left_vector,
                      void *const stream) {
  if (!y || !a || !x)
    return WMMAE_STATUS_NULL_POINTER;
  if (!type_ec_supported(type, ec))
    return WMMAE_STATUS_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return with_type(type, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_ec(ec, [&](auto te) {
      using EC = typename decltype(te)::type;
      using P = typename harness_policy<T, EC, 16, 16, 32>::type;
      hipLaunchKernelGGL((wmmae_harness::tcec_matvec_kernel<32, T, P>), dim3(1),
                         dim3(64), 0, s, y, a, x, a_col, left_vector);
      return launch_status();
    });
  });
}

int wmmae_tcec_frag_dump(const int use, const int type, const int ec,
                         const int frag_col, unsigned short *const terms,
                         const float *const src, const int from_vector,
                         const int mem_col, void *const stream) {
  if (!terms || !src)
    return WMMAE_STATUS_NULL_POINTER;
  if (use < 0 || use > 1 || mem_col < 0 || mem_col > 2)
    return WMMAE_STATUS_INVALID_VALUE;
  // (the swizzled tile is staged with 16-byte copies)
  if (mem_col == 2 && reinterpret_cast<uintptr_t>(src) % 16 != 0)
    return WMMAE_STATUS_MISALIGNED;
  if (type == 3) // fp32 fragments hold no 16-bit terms
    return WMMAE_STATUS_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return with_type(type, [&](auto tt) {
    using T = typename decltype(tt)::type;
    if constexpr (std::is_same<T, float>::value)
      return static_cast<int>(WMMAE_STATUS_NOT_SUPPORTED);
    else
    return with_ec(ec, [&](auto te) {
      using EC = typename decltype(te)::type;
      using P = typename harness_policy<T, EC, 16, 16, 32>::type;
      return with_layout(frag_col, [&](auto ll) {
        using L = typename decltype(ll)::type;
        if (use == 0)
          hipLaunchKernelGGL(
              (wmmae_harness::tcec_frag_dump_kernel<w::matrix_a, 32, T, P, L>),
              dim3(1), dim3(64), 0, s, terms, src, from_vector, mem_col);
        else
          hipLaunchKernelGGL(
              (wmmae_harness::tcec_frag_dump_kernel<w::matrix_b, 32, T, P, L>),
              dim3(1), dim3(64), 0, s, terms, src, from_vector, mem_col);
        return launch_status();
      });
    });
  });
}

int wmmae_tcec_elementwise(const int type, const int ec, const int inst,
                           float *const out, const float base,
                           const int do_neg, const int do_integrate,
                           void *const stream) {
  if (!out)
    return WMMAE_STATUS_NULL_POINTER;
  if (inst < 0 || inst > 2)
    return WMMAE_STATUS_INVALID_VALUE;
  if (!type_ec_supported(type, ec))
    return WMMAE_STATUS_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return with_type(type, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_ec(ec, [&](auto te) {
      using EC = typename decltype(te)::type;
      auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(1), dim3(64), 0, s, out, base, do_neg,
                           do_integrate);
        return launch_status();
      };
      if (inst == 0)
        return go(wmmae_harness::tcec_elementwise_kernel<
                  32, T, typename harness_policy<T, EC, 16, 16, 32>::type>);
      if (inst == 1)
        return go(wmmae_harness::tcec_elementwise_kernel<
                  32, T, typename harness_policy<T, EC, 16, 16, 16>::type>);
      return go(wmmae_harness::tcec_elementwise_kernel<
                32, T, typename harness_policy<T, EC, 32, 32, 16>::type>);
    });
  });
}
int wmmae_tcec_mma_complex(const int type, const int ec, float *const d,
                           const float *const a, const float *const b,
                           const float *const c, const int a_col,
                           const int b_col, const int c_col, const int d_col,
                           const int rounding, const float mul,
                           void *const stream) {
  if (!d || !a || !b)
    return WMMAE_STATUS_NULL_POINTER;
  if (rounding < 0 || rounding > 2 || mul == 0.f)
    return WMMAE_STATUS_INVALID_VALUE;
  if (!type_ec_supported(type, ec))
    return WMMAE_STATUS_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  using cplx = tcec::complex_t;
  return with_type(type, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_ec(ec, [&](auto te) {
      using EC = typename decltype(te)::type;
      using P = typename harness_policy<T, EC, 16, 16, 32>::type;
      hipLaunchKernelGGL(
          (wmmae_harness::tcec_mma_complex_kernel<32, T, P, w::row_major,
                                                  w::col_major>),
          dim3(1), dim3(64), 0, s, reinterpret_cast<cplx *>(d),
          reinterpret_cast<const cplx *>(a), reinterpret_cast<const cplx *>(b),
          reinterpret_cast<const cplx *>(c), a_col, b_col, c_col, d_col,
          rounding, mul);
      return launch_status();
    });
  });
}

int wmmae_primitive_mma(const int elem, const int shape_arg, float *const d,
                        const float *const a, const float *const b,
                        const float *const c, const int a_col, const int b_col,
                        const int c_col, const int d_col, void *const stream) {
  if (!d || !a || !b)
    return WMMAE_STATUS_NULL_POINTER;
  const bool wrappers = shape_arg >= 8; // + 8: tcec::detail function objects
  const int shape = wrappers ? shape_arg - 8 : shape_arg;
  if (elem < 0 || elem > 2 || shape < 0 || shape > 3)
    return WMMAE_STATUS_INVALID_VALUE;
  if (elem == 2 && shape != 0 && shape != 2)
    return WMMAE_STATUS_NOT_SUPPORTED; // fp32 operands: 16x16x16 and 32x32x8
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(1), dim3(64), 0, s, d, a, b, c, c_col,
                       d_col);
    return launch_status();
  };
  return with_layout(a_col, [&](auto la) {
    using AL = typename decltype(la)::type;
    return with_layout(b_col, [&](auto lb) {
      using BL = typename decltype(lb)::type;
      auto by_shape = [&](auto tt) {
        using T = typename decltype(tt)::type;
        switch (shape) {
        case 0:
          return wrappers ? go(wmmae_harness::wrapper_mma_kernel<T, 16, 16, 16, AL, BL>)
                          : go(wmmae_harness::primitive_mma_kernel<T, 16, 16, 16, AL, BL>);
        case 1:
          if constexpr (!std::is_same<T, float>::value)
            return wrappers ? go(wmmae_harness::wrapper_mma_kernel<T, 16, 16, 32, AL, BL>)
                          : go(wmmae_harness::primitive_mma_kernel<T, 16, 16, 32, AL, BL>);
          break;
        case 2:
          return wrappers ? go(wmmae_harness::wrapper_mma_kernel<T, 32, 32, 8, AL, BL>)
                          : go(wmmae_harness::primitive_mma_kernel<T, 32, 32, 8, AL, BL>);
        default:
          if constexpr (!std::is_same<T, float>::value)
            return wrappers ? go(wmmae_harness::wrapper_mma_kernel<T, 32, 32, 16, AL, BL>)
                          : go(wmmae_harness::primitive_mma_kernel<T, 32, 32, 16, AL, BL>);
          break;
        }
        return static_cast<int>(WMMAE_STATUS_NOT_SUPPORTED);
      };
      if (elem == 0)
        return by_shape(tag<w::half>{});
      if (elem == 1)
        return by_shape(tag<w::bfloat16>{});
      return by_shape(tag<float>{});
    });
  });
}

int wmmae_foreach_ec(float *const d, const float *const a, const float *const b,
                     void *const stream) {
  if (!d || !a || !b)
    return WMMAE_STATUS_NULL_POINTER;
  hipLaunchKernelGGL(wmmae_harness::foreach_ec_kernel, dim3(1), dim3(64), 0,
                     static_cast<hipStream_t>(stream), d, a, b);
  return launch_status();
}

int wmmae_gevm(float *const y, const float *const x, const float *const e,
               void *const stream) {
  if (!y || !x || !e)
    return WMMAE_STATUS_NULL_POINTER;
  hipLaunchKernelGGL(wmmae_harness::gevm_kernel, dim3(1), dim3(64), 0,
                     static_cast<hipStream_t>(stream), y, x, e);
  return launch_status();
}

int wmmae_fragment_ops(const int op, const int use, const int elem,
                       const float alpha, const float *const a,
                       const float *const b, float *const out,
                       void *const stream) {
  if (!a || !b || !out)
    return WMMAE_STATUS_NULL_POINTER;
  if (op < 0 || op > 5 || use < 0 || use > 2 || elem < 0 || elem > 2)
    return WMMAE_STATUS_INVALID_VALUE;
  if (use == 2 && elem != 2) // accumulators are fp32 on the matrix core
    return WMMAE_STATUS_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(1), dim3(64), 0, s, out, a, b, alpha, op);
    return launch_status();
  };
  using R = w::row_major;
  if (use == 2)
    return go(wmmae_harness::fragment_ops_kernel<w::accumulator, float, void>);
  if (use == 0) {
    if (elem == 0)
      return go(wmmae_harness::fragment_ops_kernel<w::matrix_a, w::half, R>);
    if (elem == 1)
      return go(wmmae_harness::fragment_ops_kernel<w::matrix_a, w::bfloat16, R>);
    return go(wmmae_harness::fragment_ops_kernel<w::matrix_a, float, R>);
  }
  if (elem == 0)
    return go(wmmae_harness::fragment_ops_kernel<w::matrix_b, w::half, R>);
  if (elem == 1)
    return go(wmmae_harness::fragment_ops_kernel<w::matrix_b, w::bfloat16, R>);
  return go(wmmae_harness::fragment_ops_kernel<w::matrix_b, float, R>);
}

int wmmae_fragment_eye(const int shape, const int identity, const float alpha,
                       float *const out, void *const stream) {
  if (!out)
    return WMMAE_STATUS_NULL_POINTER;
  if (shape < 0 || shape > 1)
    return WMMAE_STATUS_INVALID_VALUE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (shape == 0)
    hipLaunchKernelGGL((wmmae_harness::fragment_eye_kernel<16, 16, 16>),
                       dim3(1), dim3(64), 0, s, out, alpha, identity);
  else
    hipLaunchKernelGGL((wmmae_harness::fragment_eye_kernel<32, 32, 8>), dim3(1),
                       dim3(64), 0, s, out, alpha, identity);
  return launch_status();
}

int wmmae_direct_product(const int elem, const int terms, const int from_float,
                         const float *const u, const float *const v,
                         float *const h, void *const stream) {
  if (!u || !v || !h)
    return WMMAE_STATUS_NULL_POINTER;
  if (elem < 0 || elem > 1 || (terms != 2 && terms != 3))
    return WMMAE_STATUS_INVALID_VALUE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(1), dim3(64), 0, s, h, u, v, from_float);
    return launch_status();
  };
  if (elem == 0)
    return terms == 2 ? go(wmmae_harness::direct_product_kernel<w::half, 2>)
                      : go(wmmae_harness::direct_product_kernel<w::half, 3>);
  return terms == 2 ? go(wmmae_harness::direct_product_kernel<w::bfloat16, 2>)
                    : go(wmmae_harness::direct_product_kernel<w::bfloat16, 3>);
}

int wmmae_clock_samples(unsigned long long *const out, const int nsamples,
                        const long long period_ticks, void *const stream) {
  if (!out)
    return WMMAE_STATUS_NULL_POINTER;
  // at most 10 s of sampling: the kernel must end on its own
  if (nsamples < 1 || period_ticks < 0 ||
      static_cast<long long>(nsamples) * period_ticks > 1000000000ll)
    return WMMAE_STATUS_INVALID_VALUE;
  hipLaunchKernelGGL(wmmae_harness::clock_samples_kernel, dim3(1), dim3(64), 0,
                     static_cast<hipStream_t>(stream), out, nsamples,
                     static_cast<unsigned long long>(period_ticks));
  return launch_status();
}

int wmmae_utils_cp_async(const int size, const int mode, void *const dst,
                         const void *const src, void *const stream) {
  if (!dst || !src)
    return WMMAE_STATUS_NULL_POINTER;
  if (mode < 0 || mode > 5 || (size != 4 && size != 8 && size != 16))
    return WMMAE_STATUS_INVALID_VALUE;
  if (mode >= 4 && size == 8) // the direct load moves 4 or 16 bytes per lane
    return WMMAE_STATUS_NOT_SUPPORTED;
  if (reinterpret_cast<uintptr_t>(src) % size != 0 ||
      reinterpret_cast<uintptr_t>(dst) % 4 != 0)
    return WMMAE_STATUS_MISALIGNED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint32_t *const d = static_cast<uint32_t *>(dst);
  const uint32_t *const g = static_cast<const uint32_t *>(src);
  if (size == 4)
    hipLaunchKernelGGL(wmmae_harness::cp_async_kernel<4>, dim3(1), dim3(128), 0,
                       s, d, g, mode);
  else if (size == 8)
    hipLaunchKernelGGL(wmmae_harness::cp_async_kernel<8>, dim3(1), dim3(128), 0,
                       s, d, g, mode);
  else
    hipLaunchKernelGGL(wmmae_harness::cp_async_kernel<16>, dim3(1), dim3(128),
                       0, s, d, g, mode);
  return launch_status();
}

int wmmae_utils_cp_async_pipeline(const int size, const int copies,
                                  const int groups, void *const dst,
                                  const void *const src, int *const pending,
                                  void *const stream) {
  if (!dst || !src || !pending)
    return WMMAE_STATUS_NULL_POINTER;
  if ((size != 4 && size != 8 && size != 16) || copies < 1 || copies > 4 ||
      groups < 1 || groups > 8)
    return WMMAE_STATUS_INVALID_VALUE;
  if (reinterpret_cast<uintptr_t>(src) % size != 0 ||
      reinterpret_cast<uintptr_t>(dst) % 4 != 0 ||
      reinterpret_cast<uintptr_t>(pending) % 4 != 0)
    return WMMAE_STATUS_MISALIGNED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint32_t *const d = static_cast<uint32_t *>(dst);
  const uint32_t *const g = static_cast<const uint32_t *>(src);
  if (size == 4)
    hipLaunchKernelGGL(wmmae_harness::cp_async_pipeline_kernel<4>, dim3(1),
                       dim3(64), 0, s, d, g, groups, copies, pending);
  else if (size == 8)
    hipLaunchKernelGGL(wmmae_harness::cp_async_pipeline_kernel<8>, dim3(1),
                       dim3(64), 0, s, d, g, groups, copies, pending);
  else
    hipLaunchKernelGGL(wmmae_harness::cp_async_pipeline_kernel<16>, dim3(1),
                       dim3(64), 0, s, d, g, groups, copies, pending);
  return launch_status();
}

int wmmae_print_fragment(const int type, const int ec, const float *const src,
                         const float base, void *const stream) {
  if (!src)
    return WMMAE_STATUS_NULL_POINTER;
  if (type == 3 || !type_ec_supported(type, ec))
    return WMMAE_STATUS_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return with_type(type, [&](auto tt) -> int {
    using T = typename decltype(tt)::type;
    if constexpr (std::is_same<T, float>::value)
      return WMMAE_STATUS_NOT_SUPPORTED;
    else
      return with_ec(ec, [&](auto te) -> int {
        using EC = typename decltype(te)::type;
        using P = typename harness_policy<T, EC, 16, 16, 32>::type;
        hipLaunchKernelGGL((wmmae_harness::print_fragment_kernel<T, P>), dim3(1),
                           dim3(64), 0, s, src, base);
        return launch_status();
      });
  });
}

int wmmae_utils_cast(const int dst_type, const float *const in, void *const out,
                     const long long n, void *const stream) {
  if (!in || !out)
    return WMMAE_STATUS_NULL_POINTER;
  if (n < 0 || n > (1ll << 38))
    return WMMAE_STATUS_INVALID_VALUE;
  if (n == 0)
    return WMMAE_STATUS_SUCCESS;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(ceil_div(n, 256)));
  return with_type(dst_type, [&](auto tt) {
    using T = typename decltype(tt)::type;
    hipLaunchKernelGGL(wmmae_harness::cast_kernel<T>, grid, dim3(256), 0, s, in,
                       out, n);
    return launch_status();
  });
}

int wmmae_mfma_probe(const int type, const int m, const int n, const int k,
                     float *const d, const unsigned short *const a,
                     const unsigned short *const b, const float *const c,
                     void *const stream) {
  if (!d || !a || !b || !c)
    return WMMAE_STATUS_NULL_POINTER;
  if (type < 0 || type > 1)
    return WMMAE_STATUS_INVALID_VALUE;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define WMMAE_PROBE(M_, N_, K_)                                                \
  if (m == M_ && n == N_ && k == K_) {                                         \
    if (type == 0)                                                             \
      hipLaunchKernelGGL(                                                      \
          (wmmae_harness::mfma_probe_kernel<w::half, M_, N_, K_>), dim3(1),    \
          dim3(64), 0, s, d, a, b, c);                                         \
    else                                                                       \
      hipLaunchKernelGGL(                                                      \
          (wmmae_harness::mfma_probe_kernel<w::bfloat16, M_, N_, K_>),         \
          dim3(1), dim3(64), 0, s, d, a, b, c);                                \
    return launch_status();                                                    \
  }
  WMMAE_PROBE(16, 16, 16)
  WMMAE_PROBE(16, 16, 32)
  WMMAE_PROBE(32, 32, 8)
  WMMAE_PROBE(32, 32, 16)
#undef WMMAE_PROBE
  return WMMAE_STATUS_NOT_SUPPORTED;
}

int wmmae_mfma_source_hazard_probe(const int producer, const int gap,
                                   float *const d, void *const stream) {
  if (!d)
    return WMMAE_STATUS_NULL_POINTER;
  if (producer < 0 || producer > 1 || gap < 0 || gap > 3)
    return WMMAE_STATUS_INVALID_VALUE;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define WMMAE_HAZARD(P_, G_)                                                   \
  if (producer == P_ && gap == G_) {                                           \
    hipLaunchKernelGGL((wmmae_harness::mfma_source_hazard_kernel<P_, G_>),     \
                       dim3(1), dim3(64), 0, s, d);                            \
    return launch_status();                                                    \
  }
  WMMAE_HAZARD(0, 0)
  WMMAE_HAZARD(0, 1)
  WMMAE_HAZARD(0, 2)
  WMMAE_HAZARD(0, 3)
  WMMAE_HAZARD(1, 0)
  WMMAE_HAZARD(1, 1)
  WMMAE_HAZARD(1, 2)
  WMMAE_HAZARD(1, 3)
#undef WMMAE_HAZARD
  return WMMAE_STATUS_INVALID_VALUE;
}

} // extern "C"