// extern "C" boundary of libwmmae_tcec.so: the tiled GEMM written against the
// public tcec:: device API.  Declaration and documentation:
// include/wmmae_tcec.h.
#include "capi_common.hpp"
#include "tcec_api_gemm_kernel.hpp"

using namespace wmmae_capi;

extern "C" {

int wmmae_tcec_api_gemm(const int type, const int ec, const int m, const int n,
                        const int k, const float *const alpha,
                        const float *const A, const int lda,
                        const float *const B, const int ldb,
                        const float *const beta, float *const C, const int ldc,
                        void *const stream) {
  if (!alpha || !beta || !A || !B || !C)
    return WMMAE_STATUS_NULL_POINTER;
  if (m <= 0 || n <= 0 || k <= 0)
    return WMMAE_STATUS_INVALID_VALUE;
  if (lda < k || ldb < k || ldc < m)
    return WMMAE_STATUS_BAD_LEADING_DIM;
  if (m % 128 != 0 || n % 128 != 0 || k % 32 != 0 || lda % 4 != 0 ||
      ldb % 4 != 0 || reinterpret_cast<uintptr_t>(A) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(B) % 16 != 0)
    return WMMAE_STATUS_NOT_SUPPORTED;
  if (!type_ec_supported(type, ec))
    return WMMAE_STATUS_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float al = *alpha, be = *beta;
  return with_type(type, [&](auto tt) {
    using T = typename decltype(tt)::type;
    return with_ec(ec, [&](auto te) {
      using EC = typename decltype(te)::type;
      using P = typename harness_policy<T, EC, 16, 16, 32>::type;
      hipLaunchKernelGGL((wmmae_harness::tcec_api_gemm_kernel<T, P>),
                         dim3(m / 128, n / 128), dim3(256), 0, s, m, n, k, al,
                         A, lda, B, ldb, be, C, ldc);
      return launch_status();
    });
  });
}

} // extern "C"
