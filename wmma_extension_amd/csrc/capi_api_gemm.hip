// extern "C" boundary of libwmmae_tcec.so: the tiled GEMM written against the
// public tcec:: device API.  Declarations and documentation:
// include/wmmae_tcec.h.
#include "capi_common.hpp"
#include "tcec_api_gemm_kernel.hpp"

using namespace wmmae_capi;

namespace {
int api_gemm_impl(const int type, const int ec, const int m, const int n,
                  const int k, const float *const alpha, const float *const A,
                  const float *const *const a_ptrs, const int lda,
                  const long long stride_a, const float *const B,
                  const float *const *const b_ptrs, const int ldb,
                  const long long stride_b, const float *const beta,
                  float *const C, float *const *const c_ptrs, const int ldc,
                  const long long stride_c, const int batch,
                  void *const stream, const int rounding = 0) {
  using S = wmmae_harness::ApiGemmShape;
  if (!alpha || !beta || (!A && !a_ptrs) || (!B && !b_ptrs) || (!C && !c_ptrs))
    return WMMAE_STATUS_NULL_POINTER;
  if (m <= 0 || n <= 0 || k <= 0 || batch < 0 || rounding < 0 || rounding > 2)
    return WMMAE_STATUS_INVALID_VALUE;
  if (lda < k || ldb < k || ldc < m)
    return WMMAE_STATUS_BAD_LEADING_DIM;
  // the staging copies move 16 bytes per lane (pointer-array entries are the
  // caller's to keep 16-byte aligned)
  if (m % S::BM != 0 || n % S::BN != 0 || k % S::SK != 0 || lda % 4 != 0 ||
      ldb % 4 != 0 ||
      (!a_ptrs &&
       (reinterpret_cast<uintptr_t>(A) % 16 != 0 || stride_a % 4 != 0)) ||
      (!b_ptrs &&
       (reinterpret_cast<uintptr_t>(B) % 16 != 0 || stride_b % 4 != 0)))
    return WMMAE_STATUS_NOT_SUPPORTED;
  if (!type_ec_supported(type, ec))
    return WMMAE_STATUS_NOT_SUPPORTED;
  if (batch == 0)
    return WMMAE_STATUS_SUCCESS;
  const long long blocks =
      static_cast<long long>(m / S::BM) * (n / S::BN) * batch;
  if (blocks > 0x7fffffffLL)
    return WMMAE_STATUS_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float al = *alpha, be = *beta;
  return with_type(type, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_ec(ec, [&](auto te) -> int {
      using EC = typename decltype(te)::type;
      using P = typename harness_policy<T, EC, 16, 16, 32>::type;
      const auto launch = [&](auto rr) -> int {
        auto kernel =
            wmmae_harness::tcec_api_gemm_kernel<T, P, 2, decltype(rr)::value>;
        static std::atomic<unsigned long long> lds_allowed{0};
        WMMAE_HIP_TRY(allow_dynamic_lds(reinterpret_cast<const void *>(kernel),
                                        S::LDS_BYTES, lds_allowed));
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(blocks)),
                           dim3(S::THREADS), S::LDS_BYTES, s, m, n, k, al, A,
                           a_ptrs, lda, stride_a, B, b_ptrs, ldb, stride_b, be,
                           C, c_ptrs, ldc, stride_c);
        return launch_status();
      };
      switch (rounding) {
      case 1:
        return launch(std::integral_constant<int, 1>{});
      case 2:
        return launch(std::integral_constant<int, 2>{});
      default:
        return launch(std::integral_constant<int, 0>{});
      }
    });
  });
}
} // namespace

extern "C" {

int wmmae_tcec_api_gemm(const int type, const int ec, const int m, const int n,
                        const int k, const float *const alpha,
                        const float *const A, const int lda,
                        const float *const B, const int ldb,
                        const float *const beta, float *const C, const int ldc,
                        void *const stream) {
  return api_gemm_impl(type, ec, m, n, k, alpha, A, nullptr, lda, 0, B, nullptr,
                       ldb, 0, beta, C, nullptr, ldc, 0, 1, stream);
}

int wmmae_tcec_api_gemm_rounding(const int type, const int ec,
                                 const int rounding, const int m, const int n,
                                 const int k, const float *const alpha,
                                 const float *const A, const int lda,
                                 const float *const B, const int ldb,
                                 const float *const beta, float *const C,
                                 const int ldc, void *const stream) {
  return api_gemm_impl(type, ec, m, n, k, alpha, A, nullptr, lda, 0, B, nullptr,
                       ldb, 0, beta, C, nullptr, ldc, 0, 1, stream, rounding);
}

int wmmae_tcec_api_gemm_batched(const int type, const int ec, const int m,
                                const int n, const int k,
                                const float *const alpha,
                                const float *const *const A_array,
                                const int lda,
                                const float *const *const B_array,
                                const int ldb, const float *const beta,
                                float *const *const C_array, const int ldc,
                                const int batch, void *const stream) {
  return api_gemm_impl(type, ec, m, n, k, alpha, nullptr, A_array, lda, 0,
                       nullptr, B_array, ldb, 0, beta, nullptr, C_array, ldc, 0,
                       batch, stream);
}

} // extern "C"
