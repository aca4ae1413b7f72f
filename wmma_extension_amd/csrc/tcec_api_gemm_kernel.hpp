// A tiled, batched SGEMM written only against the public device API of this
// library (tcec::fragment, load_matrix_sync, mma_sync, store_matrix_sync,
// utils::cp_async), the way a user of the reference writes one: the shape of
// the reference's bgemm_kernel / mma_core / dmem2smem
// (test/tcec/batch_gemm.cu:74-116, 196-257, 261-386).
//
//   * fp32 tiles of A (row-major) and B (column-major) are staged in LDS by
//     utils::cp_async, two stages: the copies of stage s+1 are in flight while
//     stage s is multiplied;
//   * every wave splits the elements it needs while loading its fragments
//     (tcec::load_matrix_sync; k is contiguous in both tiles, so the loads
//     are 16 bytes wide) and multiplies with tcec::mma_sync;
//   * the operand fragments are double buffered over the k steps of a stage.
//
// Rows of a staged tile are exactly SK = 32 floats (128 bytes), unpadded, with
// the eight 16-byte pieces of row r stored at piece index p ^ ((r / 2) & 5)
// (tcec::row_major_swizzled / col_major_swizzled): a 16-byte LDS read is served
// sixteen lanes at a time - eight rows of one k group and eight rows of the
// next - and with this permutation they hit all 64 banks once.  No row padding
// does that (every padded stride costs a two-way conflict; the reference's
// skew of 8 floats, batch_gemm.cu:11, is made for 32 banks and 32 lanes).  The
// direct global->LDS copy of gfx950 writes lane-linear destinations, so the
// copy walks the tile image linearly, 16 bytes per lane
// (cp_async_lane_linear), and each lane fetches the logical piece that belongs
// at its place.
//
// Two workgroups of four waves share a compute unit (64 KiB of LDS and at
// most 256 registers each, WAVES_PER_SIMD = 2): while one waits at its
// barrier or for its copies, the other computes.  (One workgroup per compute
// unit with up to 512 registers measured slower for every policy, the
// three-term split included: 144 against 183 TFLOPS at 4096^3.)
//
// Three things the compiler has to be told for the stage loop to become one
// basic block whose MFMAs and conversions it can interleave: the wave index is
// wave-uniform (readfirstlane), the tile pointers handed to load_matrix_sync
// are 16-byte aligned (__builtin_assume_aligned: its 16-byte path is then
// chosen at compile time), and the wait for the copies stays where it is
// written (cp_async::wait_all is a scheduling barrier).
#pragma once
#include <wmma_extension/tcec/tcec.hpp>
#include <wmma_extension/utils.hpp>

namespace wmmae_harness {
namespace w = mtk::wmma;
namespace tcec = mtk::wmma::tcec;
namespace cpa = mtk::wmma::utils::cp_async;

struct ApiGemmShape {
  static constexpr int BM = 128, BN = 128; // block tile
  static constexpr int SK = 32;            // k per stage
  static constexpr int WM = 64, WN = 64;   // wave tile (2 x 2 waves)
  static constexpr int WK = 32;            // k per fragment
  static constexpr int LD = SK;            // unpadded rows, pieces swizzled
  static constexpr int STAGES = 2;
  static constexpr int THREADS = 256;
  static constexpr int STAGE_FLOATS = (BM + BN) * LD;
  static constexpr int LDS_BYTES = STAGES * STAGE_FLOATS * 4;
};

// Copy ROWS x SK floats (row r at src + r*ld) into a swizzled tile (see above).
// A pass of the workgroup moves THREADS / 8 whole rows: thread t writes
// physical piece t % 8 of row t / 8 and fetches the logical piece
// (t % 8) ^ swizzled_piece(row) for it; the rows of a pass are a multiple of
// 16, so a thread's logical piece and source offset are the same in every pass.
template <int ROWS, int SK, int THREADS>
__device__ __forceinline__ void stage_tile(float *const dst,
                                           const float *const src,
                                           const long long ld) {
  static_assert(SK == 32, "rows of 128 bytes");
  constexpr int RP = THREADS / 8; // rows per pass
  static_assert(RP % 16 == 0 && ROWS % RP == 0, "whole passes of whole rows");
  const int tid = static_cast<int>(threadIdx.x);
  const int r_in = tid / 8;
  const int c = (tid % 8) ^ static_cast<int>(tcec::swizzled_piece(r_in));
  const float *const from = src + r_in * ld + 4 * c;
#pragma unroll
  for (int r0 = 0; r0 < ROWS; r0 += RP)
    cpa::cp_async_lane_linear<16>(dst + 4 * (r0 * 8 + tid), from + r0 * ld);
}

// C tile = alpha * A tile * B tile + beta * C tile for one 128 x 128 tile of
// one batch entry.  A: m x k row-major (lda), B: k x n column-major (ldb), C:
// m x n column-major (ldc); m, n multiples of 128, k of 32; batch entry y at
// base + y*stride or, when the pointer arrays are set, at ptrs[y].
// ROUNDING: 0 tcec::mma_sync (the reference's default for the policy), 1
// mma_rn_sync, 2 mma_rz_sync.
template <class T, class Policy, int WAVES_PER_SIMD, int ROUNDING = 0>
__global__ void __launch_bounds__(ApiGemmShape::THREADS, WAVES_PER_SIMD)
    tcec_api_gemm_kernel(const int m, const int n, const int k,
                         const float alpha, const float *const A,
                         const float *const *const a_ptrs, const int lda,
                         const long long stride_a, const float *const B,
                         const float *const *const b_ptrs, const int ldb,
                         const long long stride_b, const float beta,
                         float *const C, float *const *const c_ptrs,
                         const int ldc, const long long stride_c) {
  using S = ApiGemmShape;
  extern __shared__ __attribute__((aligned(16))) float smem[];

  // tile of this workgroup: consecutive block ids run on different XCDs, so
  // ids are regrouped to give each XCD (id % 8) one contiguous run of tiles,
  // walked column by column through bands of eight tile rows
  const unsigned tiles_m = m / S::BM, tiles_n = n / S::BN;
  const unsigned tiles = tiles_m * tiles_n;
  const unsigned entry = blockIdx.x / tiles;
  unsigned t = blockIdx.x - entry * tiles;
  if (tiles % 8 == 0)
    t = (t % 8) * (tiles / 8) + t / 8;
  const unsigned band = t / (8 * tiles_n);
  const unsigned band_rows = tiles_m - 8 * band < 8 ? tiles_m - 8 * band : 8;
  const unsigned in_band = t - band * 8 * tiles_n;
  const unsigned tn = in_band / band_rows;
  const unsigned tm = 8 * band + in_band - tn * band_rows;

  const float *const a_base =
      (a_ptrs != nullptr ? a_ptrs[entry] : A + entry * stride_a) +
      static_cast<long long>(tm * S::BM) * lda;
  const float *const b_base =
      (b_ptrs != nullptr ? b_ptrs[entry] : B + entry * stride_b) +
      static_cast<long long>(tn * S::BN) * ldb;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int wm = wave % 2, wn = wave / 2;

  using FragA =
      tcec::fragment<w::matrix_a, S::WM, S::WN, S::WK, T, w::row_major, Policy>;
  using FragB =
      tcec::fragment<w::matrix_b, S::WM, S::WN, S::WK, T, w::col_major, Policy>;
  using FragC =
      tcec::fragment<w::accumulator, S::WM, S::WN, S::WK, T, void, Policy>;
  FragC fc;
  tcec::fill_zero(fc);
  const auto mma = [](FragC &d, const FragA &a, const FragB &b) {
    if constexpr (ROUNDING == 1)
      tcec::mma_rn_sync(d, a, b, d);
    else if constexpr (ROUNDING == 2)
      tcec::mma_rz_sync(d, a, b, d);
    else
      tcec::mma_sync(d, a, b, d);
  };

  auto stage_in = [&](const int stage, const int k0) {
    float *const sa = smem + stage * S::STAGE_FLOATS;
    float *const sb = sa + S::BM * S::LD;
    stage_tile<S::BM, S::SK, S::THREADS>(sa, a_base + k0, lda);
    stage_tile<S::BN, S::SK, S::THREADS>(sb, b_base + k0, ldb);
    // (no cp_async::commit(): the loop waits with wait_all(), which needs no
    // groups, and commit() costs a round trip to its bookkeeping in LDS)
  };

  stage_in(0, 0);
  cpa::wait_all();
  __syncthreads();

  int stage = 0;
  for (int k0 = 0; k0 < k; k0 += S::SK) {
    if (k0 + S::SK < k)
      stage_in(1 - stage, k0 + S::SK);

    const float *const sa =
        static_cast<const float *>(__builtin_assume_aligned(
            smem + stage * S::STAGE_FLOATS + wm * S::WM * S::LD, 16));
    const float *const sb =
        static_cast<const float *>(__builtin_assume_aligned(
            smem + stage * S::STAGE_FLOATS + (S::BM + wn * S::WN) * S::LD, 16));
    // fragments double buffered over the k steps of the stage
    FragA fa[2];
    FragB fb[2];
    tcec::load_matrix_sync<tcec::row_major_swizzled>(fa[0], sa, S::LD, false);
    tcec::load_matrix_sync<tcec::col_major_swizzled>(fb[0], sb, S::LD, false);
#pragma unroll
    for (int kk = S::WK; kk < S::SK; kk += S::WK) {
      const int cur = (kk / S::WK) & 1;
      tcec::load_matrix_sync<tcec::row_major_swizzled>(fa[cur], sa + kk, S::LD,
                                                       false);
      tcec::load_matrix_sync<tcec::col_major_swizzled>(fb[cur], sb + kk, S::LD,
                                                       false);
      mma(fc, fa[1 - cur], fb[1 - cur]);
    }
    constexpr int last = ((S::SK / S::WK) - 1) & 1;
    mma(fc, fa[last], fb[last]);

    cpa::wait_all();
    __syncthreads();
    stage = 1 - stage;
  }

  float *const cw = (c_ptrs != nullptr ? c_ptrs[entry] : C + entry * stride_c) +
                    (tm * S::BM + wm * S::WM) +
                    static_cast<long long>(tn * S::BN + wn * S::WN) * ldc;
  if (beta == 0.f) {
    tcec::store_matrix_sync_with_mul<w::col_major>(cw, fc, ldc, alpha);
  } else {
    FragC fin;
    tcec::load_matrix_sync(fin, cw, ldc, w::mem_col_major);
    fc.integrate();
#pragma unroll
    for (unsigned i = 0; i < fc.num_elements; i++) // (the roundings written out)
      fc.x(i) = __builtin_fmaf(alpha, fc.x(i), beta * fin.x(i));
    tcec::store_matrix_sync(cw, fc, ldc, w::mem_col_major);
  }
}

} // namespace wmmae_harness
