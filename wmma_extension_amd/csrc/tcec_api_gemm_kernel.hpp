// A tiled SGEMM written only against the public device API of this library
// (tcec::fragment, load_matrix_sync, mma_sync, store_matrix_sync,
// utils::cp_async), the way a user of the reference writes one.
#pragma once
#include <wmma_extension/tcec/tcec.hpp>
#include <wmma_extension/utils.hpp>

namespace wmmae_harness {
namespace w = mtk::wmma;
namespace tcec = mtk::wmma::tcec;

// --------------------------------------------------------------------------
// A tiled SGEMM written only against the public tcec:: API, the way a user of
// the reference writes one (reference: bgemm_kernel / mma_core,
// test/tcec/batch_gemm.cu:196-386): fp32 tiles are staged in LDS, every wave
// splits the elements it needs while loading its fragments
// (tcec::load_matrix_sync), multiplies with tcec::mma_sync and writes the
// result with the element accessors.  A is row-major m x k (lda), B is
// column-major k x n (ldb), C column-major (ldc); m, n multiples of 128, k of 32.
// It exists to show the drop-in at GEMM scale and as the comparator for the
// packed-operand driver, which does the split once per element instead.
// --------------------------------------------------------------------------
template <class T, class Policy>
__global__ void __launch_bounds__(256)
    tcec_api_gemm_kernel(const int m, const int n, const int k,
                         const float alpha, const float *__restrict__ A,
                         const int lda, const float *__restrict__ B,
                         const int ldb, const float beta,
                         float *__restrict__ C, const int ldc) {
  constexpr int BM = 128, BN = 128, BK = 32, LD = BK + 4; // +4 floats: skewed rows
  constexpr int WM = 64, WN = 64;
  __shared__ float sa[BM * LD];
  __shared__ float sb[BN * LD];
  const int wave = threadIdx.x / 64;
  const int wm = wave % 2, wn = wave / 2;
  const int m0 = blockIdx.x * BM, n0 = blockIdx.y * BN;

  tcec::fragment<w::matrix_a, WM, WN, BK, T, w::row_major, Policy> fa;
  tcec::fragment<w::matrix_b, WM, WN, BK, T, w::col_major, Policy> fb;
  tcec::fragment<w::accumulator, WM, WN, BK, T, void, Policy> fc;
  tcec::fill_zero(fc);

  for (int k0 = 0; k0 < k; k0 += BK) {
    // 128 rows x 32 floats per operand = 1024 float4, 4 per thread
    for (int f = threadIdx.x; f < BM * BK / 4; f += 256) {
      const int r = f / (BK / 4), c4 = f % (BK / 4);
      const float4 va = *reinterpret_cast<const float4 *>(
          A + static_cast<long long>(m0 + r) * lda + k0 + 4 * c4);
      const float4 vb = *reinterpret_cast<const float4 *>(
          B + static_cast<long long>(n0 + r) * ldb + k0 + 4 * c4);
      *reinterpret_cast<float4 *>(&sa[r * LD + 4 * c4]) = va;
      *reinterpret_cast<float4 *>(&sb[r * LD + 4 * c4]) = vb;
    }
    __syncthreads();
    tcec::load_matrix_sync(fa, sa + wm * WM * LD, LD);  // memory layout = row_major
    tcec::load_matrix_sync(fb, sb + wn * WN * LD, LD);  // memory layout = col_major
    tcec::mma_sync(fc, fa, fb, fc);
    __syncthreads();
  }

  float *const cw = C + (m0 + wm * WM) + static_cast<long long>(n0 + wn * WN) * ldc;
  if (beta == 0.f) {
    tcec::store_matrix_sync_with_mul<w::col_major>(cw, fc, ldc, alpha);
  } else {
    tcec::fragment<w::accumulator, WM, WN, BK, T, void, Policy> fin;
    tcec::load_matrix_sync(fin, cw, ldc, w::mem_col_major);
    fc.integrate();
    for (unsigned i = 0; i < fc.num_elements; i++)
      fc.x(i) = alpha * fc.x(i) + beta * fin.x(i);
    tcec::store_matrix_sync(cw, fc, ldc, w::mem_col_major);
  }
}


} // namespace wmmae_harness
