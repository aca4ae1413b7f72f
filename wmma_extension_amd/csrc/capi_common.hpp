// Helpers shared by the translation units behind the extern "C" boundary of
// libwmmae_tcec.so (declarations and per-entry documentation:
// include/wmmae_tcec.h).
#pragma once
#include <wmmae_tcec.h>
#include <wmmae_tcec_aux.h>

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <hip/hip_runtime.h>
#include <wmma_extension/tcec/tcec.hpp>

namespace wmmae_capi {
namespace w = mtk::wmma;
namespace tcec = mtk::wmma::tcec;

#define WMMAE_HIP_TRY(expr)                                                    \
  do {                                                                         \
    if ((expr) != hipSuccess)                                                  \
      return WMMAE_STATUS_RUNTIME_ERROR;                                       \
  } while (0)

inline int launch_status() {
  return hipGetLastError() == hipSuccess ? WMMAE_STATUS_SUCCESS
                                         : WMMAE_STATUS_RUNTIME_ERROR;
}

template <class T> struct tag {
  using type = T;
};

inline long long ceil_div(const long long a, const long long b) {
  return (a + b - 1) / b;
}

// A kernel that wants more dynamic LDS than the default limit has to be told
// so once per device; `done` is the calling site's own bit mask of devices
// (one static per kernel instantiation), so later launches skip the driver
// call.
inline hipError_t allow_dynamic_lds(const void *const kernel, const int bytes,
                                    std::atomic<unsigned long long> &done) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return e;
  const bool tracked = dev >= 0 && dev < 64;
  if (tracked && ((done.load(std::memory_order_relaxed) >> dev) & 1ull) != 0)
    return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                          bytes);
  if (e == hipSuccess && tracked)
    done.fetch_or(1ull << dev, std::memory_order_relaxed);
  return e;
}

// ---- type / policy dispatch of the device-API harness entry points
template <class F> int with_type(const int type, F f) {
  switch (type) {
  case 0:
    return f(tag<w::half>{});
  case 1:
    return f(tag<w::bfloat16>{});
  case 2:
    return f(tag<w::precision::tf32>{});
  case 3:
    return f(tag<float>{});
  default:
    return WMMAE_STATUS_INVALID_VALUE;
  }
}
// Policy a harness kernel is instantiated with: the MFMA policy of the asked
// instruction shape, or, for fp32 operands, the one op_simt policy.
template <class T, class EC, int fm, int fn, int fk> struct harness_policy {
  using type = tcec::Policy<tcec::op_mfma, EC, fm, fn, fk>;
};
template <class EC, int fm, int fn, int fk>
struct harness_policy<float, EC, fm, fn, fk> {
  using type = typename tcec::default_policy<float, tcec::without_ec,
                                             tcec::op_simt>::type;
};
// fp32 operands exist without error correction only
inline bool type_ec_supported(const int type, const int ec) {
  return !(type == 3 && ec != 0);
}
template <class F> int with_ec(const int ec, F f) {
  if (ec)
    return f(tag<tcec::with_ec>{});
  return f(tag<tcec::without_ec>{});
}
template <class F> int with_layout(const int col, F f) {
  if (col)
    return f(tag<w::col_major>{});
  return f(tag<w::row_major>{});
}
} // namespace wmmae_capi
