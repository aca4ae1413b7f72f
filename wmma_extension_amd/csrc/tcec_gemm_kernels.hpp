// TCEC SGEMM for gfx950: operand split + fragment-major packing, and the MFMA
// GEMM kernel that consumes the packed operands.
//
// The reference's only tiled GEMM (test/tcec/batch_gemm.cu:196-386) stages
// fp32 tiles in shared memory and lets every warp convert and split the
// elements it needs each time it loads a fragment (tcec/tcec.hpp:213-229).
// Here each fp32 element is split exactly once, by split_pack_kernel, into
// 16-bit terms that are written to HBM already in the register order of the
// v_mfma_f32_16x16x32 operand ("fragment-major"):
//
//   packed[rb][kt][term][lane] : one 16-byte chunk per lane; lane l holds
//       row 16*rb + l%16, k = 32*kt + 8*(l/16) .. +7 of that term
//
// so one 1 KiB chunk is one MFMA operand for a whole wave.  The GEMM kernel
// then moves chunks HBM -> LDS -> registers with perfectly linear 128-bit
// accesses (no padding, no swizzle, no bank conflicts) and does no
// conversion work in its K loop.  Both operands use the same packing
// ("rows" are the m index for A and the n index for B), so any BLAS
// transpose combination is handled by the strides given to the split kernel.
//
// Why 16x16x32 and not 32x32x16 (same nominal flop rate, half the
// instructions): the MFMA rate of this chip is power limited as soon as the
// operands are not constant.  Measured on MI355X, back-to-back MFMAs on random
// fp16 data sustain 1.87-1.9 PFLOP/s with 16x16x32 and 1.66 PFLOP/s with
// 32x32x16 (2.4 PFLOP/s on all-zero data for both).
#pragma once
#include <wmma_extension/tcec/tcec.hpp>

namespace wmmae_gemm {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kChunkRows = 16; // rows per packed chunk (MFMA M / N)
constexpr int kChunkK = 32;    // k per packed chunk (MFMA K) = one pipeline stage

// Text put in front of every MFMA issued from inline asm.  Empty: the build
// checks the generated code instead (wmma_extension_amd/isa_check.py) for
// vector-ALU writes of an MFMA's source registers directly before it, which
// the hardware does not interlock and the compiler does not see.  "s_nop 0\n\t"
// makes such a place harmless wherever it may appear, at 0.3 to 1 % for the
// kernels on packed operands and 13 % for the one that splits its own.
#ifndef WMMAE_MFMA_GUARD
#define WMMAE_MFMA_GUARD ""
#endif
template <int I> using ic = std::integral_constant<int, I>;
// Compile-time loop: f(std::integral_constant<int, I>) for I in [B, E).
template <int B, int E, class F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (B < E) {
    f(std::integral_constant<int, B>{});
    static_for<B + 1, E>(f);
  }
}

// The value the lane with the lowest lane-number bit flipped holds (DPP
// quad_perm [1, 0, 3, 2]); every lane of the wave must be active.
__device__ __forceinline__ float neighbour_lane(const float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF,
                                      true));
}
// The epilogue's arithmetic, spelled out so that every kernel and every store
// path rounds alike whatever the compiler would contract: the error sum is
// folded in with one fma, alpha is a multiplication of its own, and beta * C
// enters with one fma.
__device__ __forceinline__ f32x4 epilogue_fold(const f32x4 main_sum,
                                                   const f32x4 err_sum,
                                                   const float inv_scale) {
  return __builtin_elementwise_fma(
      err_sum, f32x4{inv_scale, inv_scale, inv_scale, inv_scale}, main_sum);
}
__device__ __forceinline__ f32x4 epilogue_beta(const f32x4 scaled,
                                                   const float beta,
                                                   const f32x4 c_old) {
  return __builtin_elementwise_fma(f32x4{beta, beta, beta, beta}, c_old,
                                   scaled);
}
__device__ __forceinline__ float epilogue_beta(const float scaled,
                                               const float beta,
                                               const float c_old) {
  return __builtin_fmaf(beta, c_old, scaled);
}
// Row permutation of k group q (0..3) of a chunk written by the DIRECT
// variant of tcec_gemm_kernel.
__host__ __device__ constexpr unsigned direct_swizzle(const unsigned q) {
  return 12u * (q & 1u) ^ 4u * (q >> 1);
}
// DIRECT == 2 (rows of k floats, k not a multiple of 32): the pieces of a
// lane's read address in a row's last, shorter stage, shared by the kernel and
// by a host-side check that no read leaves its row.  A lane reads four floats;
// the one whose four would end past the row reads the row's last four instead.
//   kDirectBias       : floats by which the row block's base is moved back and
//                       every lane offset forward, so that a lane reading up
//                       to three floats before the stage's start keeps an
//                       offset >= 0
//   direct_tail_shift : floats a lane moves back, `left` = floats from the
//                       stage's start to the row's end
//   direct_read_first : first float, counted from the row's start, that lane
//                       `lane` reads in stage `stage` (`tail`: that variant)
constexpr int kDirectBias = 4;
__host__ __device__ constexpr int direct_tail_shift(const unsigned lane,
                                                    const int left) {
  const int s = 4 * static_cast<int>(lane & 7u) + 4 - left;
  return s > 0 ? s : 0;
}
__host__ __device__ constexpr long long
direct_read_first(const bool tail, const int k, const int stage,
                  const unsigned lane) {
  const long long base = 32ll * stage - (tail ? kDirectBias : 0);
  const long long lane_off = 4ll * (lane & 7u) + (tail ? kDirectBias : 0);
  return base + lane_off - (tail ? direct_tail_shift(lane, k - 32 * stage) : 0);
}
// Number of LDS reads that have been issued once `count` MFMAs of a step are
// out: read r is due after MFMA number (r+1)*span/nfrag.
__host__ __device__ constexpr int reads_due(const int count, const int span,
                                            const int nfrag) {
  int r = 0;
  while (r < nfrag && ((r + 1) * span) / nfrag <= count)
    r++;
  return r;
}
// MFMA of a step after which LDS read r of the next stage goes out when the A
// fragments are recycled (GemmConfig::RECYCLE_A): the first `first_reads` (B
// and A's last tile row, which have registers of their own) spread over the
// first tile row's `row_mfma` MFMAs, the A fragments of tile row i right after
// the last MFMA of that row.
__host__ __device__ constexpr int recycled_read_slot(const int r,
                                                     const int first_reads,
                                                     const int row_mfma,
                                                     const int terms) {
  return r < first_reads ? (r * row_mfma) / first_reads
                         : ((r - first_reads) / terms + 1) * row_mfma +
                               2 * ((r - first_reads) % terms);
}
// DIRECT: number of producer micro-operations that have gone out once `n`
// MFMAs of a step are out.  Micro-operations and LDS reads together are spread
// evenly over the MFMAs: after every MFMA the micro-operations make up what
// the reads due there leave of the common rate.
__host__ __device__ constexpr int
direct_uops_before(const int n, const bool recycle, const int nuop,
                   const int nfrag, const int nmfma, const int span,
                   const int first_reads, const int row_mfma, const int terms) {
  int prev = 0;
  for (int m = 1; m <= n; m++) {
    int reads = 0; // issued after the MFMAs 0 .. m-1
    if (recycle) {
      for (int r = 0; r < nfrag; r++)
        reads += recycled_read_slot(r, first_reads, row_mfma, terms) < m;
    } else {
      reads = m == nmfma ? nfrag : reads_due(m, span, nfrag);
    }
    int t = (m * (nuop + nfrag)) / nmfma - reads;
    t = t < prev ? prev : t;
    prev = t > nuop ? nuop : t;
  }
  return n >= nmfma ? nuop : prev;
}

// --------------------------------------------------------------------------
// split_pack_kernel: X (fp32, element (r,k) at X[r*row_stride + k*k_stride])
// -> packed terms.  One thread per (chunk, lane).  Rows >= rows and k >= K are
// zero filled, so the GEMM kernel needs no edge handling on its loads.
// Batch entry y (entry0 + blockIdx.y: a launch covers at most 65535 entries,
// the host loops over longer batches) reads X + y*batch_stride, or ptrs[y]
// when ptrs is set (the reference's harness passes arrays of matrix pointers,
// test/tcec/batch_gemm.cu:433-443).
//   T      : split tag (half, bfloat16, precision::tf32)
//   TERMS  : number of terms stored (1 = leading term only, i.e. no correction)
//   KT     : number of 32-wide k chunks per row block; chunks = row blocks * KT
// --------------------------------------------------------------------------
struct PackOperand {
  const float *X;             // entry y at X + y*batch_stride ...
  const float *const *ptrs;   // ... or at ptrs[y] when set
  long long row_stride, k_stride, batch_stride;
  int rows;
  long long chunks;           // row blocks * KT
  u32x4 *out;                 // entry y at out + y*chunks*TERMS*64
};

// the work of one 256-thread block: four chunks of batch entry `entry`
template <class T, int TERMS>
__device__ __forceinline__ void split_pack_block(const PackOperand &o,
                                                 const int K, const int KT,
                                                 const unsigned block,
                                                 const unsigned entry) {
  using traits = mtk::wmma::tcec::detail::split_traits<T>;
  using S = typename traits::storage;
  static_assert(TERMS >= 1 && TERMS <= traits::num_terms, "bad TERMS");
  const unsigned lane = threadIdx.x & 63u;
  const long long chunk =
      (static_cast<long long>(block) * 256 + threadIdx.x) >> 6;
  if (chunk >= o.chunks)
    return;
  const long long rb = chunk / KT;
  const int kc = static_cast<int>(chunk - rb * KT);
  const long long r = rb * kChunkRows + (lane & 15u);
  const int k0 = kc * kChunkK + 8 * static_cast<int>(lane >> 4);

  float v[8];
#pragma unroll
  for (int x = 0; x < 8; x++)
    v[x] = 0.f;
  if (r < o.rows && k0 < K) {
    // batch entry: base + stride, or a device array of matrix pointers
    const float *const base =
        o.ptrs != nullptr ? o.ptrs[entry] : o.X + entry * o.batch_stride;
    const float *p =
        base + r * o.row_stride + static_cast<long long>(k0) * o.k_stride;
    if (o.k_stride == 1 && k0 + 8 <= K &&
        (reinterpret_cast<uintptr_t>(p) & 15u) == 0) {
      const f32x4 lo = *reinterpret_cast<const f32x4 *>(p);
      const f32x4 hi = *reinterpret_cast<const f32x4 *>(p + 4);
#pragma unroll
      for (int x = 0; x < 4; x++) {
        v[x] = lo[x];
        v[4 + x] = hi[x];
      }
    } else {
#pragma unroll
      for (int x = 0; x < 8; x++)
        if (k0 + x < K)
          v[x] = p[x * o.k_stride];
    }
  }

  typedef S s8 __attribute__((ext_vector_type(8)));
  s8 t[3];
#pragma unroll
  for (int x = 0; x < 8; x++) {
    S t0, t1, t2;
    traits::split(v[x], t0, t1, t2);
    t[0][x] = t0;
    t[1][x] = t1;
    t[2][x] = t2;
  }
  u32x4 *dst =
      o.out + entry * (o.chunks * (TERMS * 64)) + chunk * (TERMS * 64) + lane;
#pragma unroll
  for (int p = 0; p < TERMS; p++)
    dst[p * 64] = __builtin_bit_cast(u32x4, t[p]);
}

template <class T, int TERMS>
__global__ void __launch_bounds__(256)
    split_pack_kernel(const PackOperand o, const int K, const int KT,
                      const unsigned entry0) {
  split_pack_block<T, TERMS>(o, K, KT, blockIdx.x, entry0 + blockIdx.y);
}

// Both operands of a product in one launch (the GEMM entry points pack A and B
// back to back; for small products a launch costs as much as the packing):
// blocks [0, blocks_a) take A, the rest B.
template <class T, int TERMS>
__global__ void __launch_bounds__(256)
    split_pack_pair_kernel(const PackOperand a, const PackOperand b,
                           const unsigned blocks_a, const int K, const int KT,
                           const unsigned entry0) {
  if (blockIdx.x < blocks_a)
    split_pack_block<T, TERMS>(a, K, KT, blockIdx.x, entry0 + blockIdx.y);
  else
    split_pack_block<T, TERMS>(b, K, KT, blockIdx.x - blocks_a,
                               entry0 + blockIdx.y);
}

// --------------------------------------------------------------------------
// scale_c_kernel: C = beta * C, the whole result when k == 0.
// --------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
    scale_c_kernel(float *__restrict__ C, const int M, const int N,
                   const long long ldc, const long long batch_stride_c,
                   float *const *__restrict__ c_ptrs, const float beta,
                   const unsigned entry0) {
  const long long e = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= static_cast<long long>(M) * N)
    return;
  const long long entry = entry0 + blockIdx.y;
  float *const cb =
      c_ptrs != nullptr ? c_ptrs[entry] : C + entry * batch_stride_c;
  float *const p = cb + (e % M) + (e / M) * ldc;
  *p = beta == 0.f ? 0.f : beta * *p;
}

// --------------------------------------------------------------------------
// reduce_splits_kernel: C = alpha * sum_z partial[z] + beta * C for split-K.
// partial[z][batch] are dense column-major M x N slices; the sum runs over z
// in ascending order in double precision, so the result does not depend on
// the launch geometry.  A thread owns VEC consecutive elements of a slice
// (VEC == 4: M, ldc and the entries' bases are multiples of four floats, so
// the four are rows of one column and every access is one 16-byte piece).
// --------------------------------------------------------------------------
template <int VEC>
__global__ void __launch_bounds__(256)
    reduce_splits_kernel(const float *__restrict__ partial, const int splits,
                         float *__restrict__ C, const int M, const int N,
                         const long long ldc, const long long batch_stride_c,
                         float *const *__restrict__ c_ptrs, const float alpha,
                         const float beta, const long long batches,
                         const unsigned entry0) {
  static_assert(VEC == 1 || VEC == 4, "one element or one 16-byte piece");
  const long long e =
      (static_cast<long long>(blockIdx.x) * 256 + threadIdx.x) * VEC;
  const long long mn = static_cast<long long>(M) * N;
  if (e >= mn)
    return;
  const long long entry = entry0 + blockIdx.y;
  double s[VEC];
#pragma unroll
  for (int x = 0; x < VEC; x++)
    s[x] = 0.;
  for (int z = 0; z < splits; z++) {
    const float *const src = partial + (z * batches + entry) * mn + e;
    if constexpr (VEC == 4) {
      const f32x4 v = *reinterpret_cast<const f32x4 *>(src);
#pragma unroll
      for (int x = 0; x < 4; x++)
        s[x] += static_cast<double>(v[x]);
    } else {
      s[0] += static_cast<double>(*src);
    }
  }
  float *const cb =
      c_ptrs != nullptr ? c_ptrs[entry] : C + entry * batch_stride_c;
  float *const p = cb + (e % M) + (e / M) * ldc;
  if constexpr (VEC == 4) {
    f32x4 out;
    f32x4 old = {0.f, 0.f, 0.f, 0.f};
    if (beta != 0.f)
      old = *reinterpret_cast<const f32x4 *>(p);
#pragma unroll
    for (int x = 0; x < 4; x++) {
      const float v = alpha * static_cast<float>(s[x]);
      out[x] = beta == 0.f ? v : v + beta * old[x];
    }
    *reinterpret_cast<f32x4 *>(p) = out;
  } else {
    const float v = alpha * static_cast<float>(s[0]);
    *p = beta == 0.f ? v : v + beta * *p;
  }
}

// --------------------------------------------------------------------------
// Tile id -> tile coordinates.  Ids x, x+8, x+16, ... run on XCD x, 32 of
// them at a time.  With `interleave`, these 32 get one GROUP x (32/GROUP)
// patch of a column-by-column walk through GROUP tile rows (a patch that is
// close to square in elements needs the fewest L2 fills), and the eight XCDs
// get eight neighbouring patches, which share the patches' A row panels: what
// misses in one XCD's L2 is then in flight to, or already in, the memory-side
// cache for the others.  The ids beyond the last full round of 8 x 32 are cut
// into eight runs, one per XCD.  Without `interleave` the ids walk the patches
// in order (one XCD owns the whole tile grid).
// --------------------------------------------------------------------------
template <unsigned GROUP>
__device__ __forceinline__ void tile_of(unsigned pid, const unsigned num_tiles,
                                        const unsigned tiles_m,
                                        const unsigned tiles_n,
                                        const bool interleave, int &tm,
                                        int &tn) {
  constexpr unsigned XCDS = 8, PATCH = 32;
  if (interleave) {
    const unsigned full = num_tiles / (XCDS * PATCH) * (XCDS * PATCH);
    if (pid < full) {
      const unsigned xcd = pid % XCDS, local = pid / XCDS;
      pid = ((local / PATCH) * XCDS + xcd) * PATCH + local % PATCH;
    } else {
      const unsigned rem = num_tiles - full, t = pid - full;
      const unsigned per = (rem + XCDS - 1) / XCDS;
      const unsigned tall = (rem % XCDS == 0) ? XCDS : (rem % XCDS);
      const unsigned xcd = t % XCDS, local = t / XCDS;
      pid = full + (xcd < tall ? xcd * per + local
                               : tall * per + (xcd - tall) * (per - 1) + local);
    }
  }
  const unsigned width = GROUP * tiles_n;
  const unsigned group = pid / width;
  const unsigned first_m = group * GROUP;
  const unsigned gsz = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
  const unsigned in_group = pid - group * width;
  const unsigned col = in_group / gsz;
  tm = static_cast<int>(first_m + in_group - col * gsz);
  tn = static_cast<int>(col);
}

// --------------------------------------------------------------------------
// reduce_tail_kernel: C tile = alpha * sum_z partial[z][t] + beta * C tile for
// the tail tiles t (tile ids tail_begin + t) that tcec_gemm_kernel has cut
// into K slices.  partial[z][t] are dense column-major BM x BN tiles; the sum
// runs over z in ascending order in double precision.  grid: (tail tiles,
// BM*BN/1024), a thread owns four consecutive rows of one column.
// --------------------------------------------------------------------------
template <int BM, int BN>
__global__ void __launch_bounds__(256)
    reduce_tail_kernel(const float *__restrict__ partial, const int slices,
                       const unsigned tail_begin, const unsigned num_tiles,
                       const int tiles_m, const int tiles_n,
                       float *__restrict__ C, const int M, const int N,
                       const long long ldc, const float alpha,
                       const float beta) {
  const unsigned t = blockIdx.x, tail_tiles = gridDim.x;
  int tm, tn;
  tile_of<(BM > BN ? 4u : 8u)>(tail_begin + t, num_tiles, tiles_m, tiles_n,
                               true, tm, tn);
  const int e4 = static_cast<int>(blockIdx.y) * 256 + threadIdx.x;
  const int col_l = e4 / (BM / 4), row_l = 4 * (e4 % (BM / 4));
  const int row = tm * BM + row_l, col = tn * BN + col_l;
  if (col_l >= BN || col >= N || row >= M)
    return;
  double s[4] = {0., 0., 0., 0.};
  for (int z = 0; z < slices; z++) {
    const f32x4 v = *reinterpret_cast<const f32x4 *>(
        partial + (static_cast<long long>(z) * tail_tiles + t) * (BM * BN) +
        col_l * BM + row_l);
#pragma unroll
    for (int x = 0; x < 4; x++)
      s[x] += static_cast<double>(v[x]);
  }
  float *const p = C + row + static_cast<long long>(col) * ldc;
#pragma unroll
  for (int x = 0; x < 4; x++) {
    if (row + x < M) {
      const float v = alpha * static_cast<float>(s[x]);
      p[x] = beta == 0.f ? v : v + beta * p[x];
    }
  }
}

// --------------------------------------------------------------------------
// tcec_gemm_kernel: C = alpha * (A*B) + beta * C from packed operands.
//
//   MT      : MFMA element type (_Float16 or __bf16)
//   TERMS   : stored terms per operand (1, 2 or 3)
//   BM x BN : block tile, WGM x WGN waves, each wave (BM/WGM) x (BN/WGN),
//             built from 16x16 MFMA tiles
//   NSTAGE  : LDS ring depth; one stage is 32 of k.  Stages are filled by
//             direct global->LDS loads (global_load_lds_dwordx4, no staging
//             registers).  While stage s is being multiplied out of
//             registers, stage s+1 is being read from LDS into the second
//             fragment set and stages s+2 .. s+NSTAGE are in flight from
//             HBM/L2, which is what covers memory latency with a single
//             workgroup per compute unit.  The 256x128 tile with three terms
//             (72 KiB a stage, a ring of two; 144 registers of fragments a
//             stage) keeps one copy of the A fragments and refills a tile
//             row's registers for the next stage right after that row's
//             MFMAs have been issued (GemmConfig::RECYCLE_A): a quarter fewer
//             L2 -> LDS bytes and LDS reads per MFMA than the 128x128 tile,
//             16384^3 32.5 -> 29.5 ms.
//   RN_MAIN : accumulate the leading product with fp32 adds outside the
//             matrix core (the reference's mma_rn_sync, tcec/tcec.hpp:673-694)
//             instead of chaining it through the MFMA accumulator.  The gfx950
//             matrix core adds with round-to-nearest-even, so chaining is the
//             default.
//
// Products issued per (16x16 tile, 32 of k), all with fp32 accumulation:
//   TERMS 1: main += a0*b0
//   TERMS 2: err += a1*b0 + a0*b1;                          main += a0*b0
//   TERMS 3: err += a2*b0 + a0*b2 + a1*b1 + a1*b0 + a0*b1;  main += a0*b0
// and the result is main + err * inv_scale (reference: tcec.hpp:332-336).
// The error terms have their own accumulator so that their low-order bits
// are not rounded away against the much larger main sum.
//
// C is column major (element (i,j) at C[i + j*ldc]); an accumulator lane owns
// four consecutive rows of one column, i.e. one 16-byte store.
// --------------------------------------------------------------------------
// fp32 operands of the DIRECT variant of tcec_gemm_kernel, which splits them
// itself: op(A) as m rows of k contiguous floats (row i at A + i*lda), op(B)
// as n rows of k contiguous floats (row j at B + j*ldb); batch entry y at
// base + y*bs or, when the pointer arrays are set, at ptrs[y].
struct DirectSource {
  const float *A, *B;
  const float *const *a_ptrs, *const *b_ptrs;
  long long lda, ldb;
  long long a_bs, b_bs;
  // > 0: the workgroups of an XCD start in 32 phases, this many periods of 512
  // cycles apart (see the kernel's prologue)
  int stagger;
  // floats per row (k); the DIRECT == 2 variant reads a last stage of fewer
  // than 32
  int k;
};

template <class MT, int TERMS, int BM, int BN, int WGM, int WGN, int NSTAGE,
          bool RN_MAIN, int DIRECT = 0>
struct GemmConfig {
  static constexpr int NW = WGM * WGN;
  static constexpr int NTHREADS = NW * 64;
  static constexpr int WM = BM / WGM, WN = BN / WGN;
  static constexpr int MT_ = WM / 16, NT_ = WN / 16;
  static constexpr int CH_PER_RB = TERMS; // chunks of one 16-row block
  static constexpr int CH_A = (BM / 16) * CH_PER_RB; // chunks per stage
  static constexpr int CH_B = (BN / 16) * CH_PER_RB;
  static constexpr int NCH = CH_A + CH_B;
  static constexpr int CPW = NCH / NW; // chunks each wave requests per stage
  static constexpr int LDS_BYTES = NSTAGE * NCH * 1024;
  // Two sets of operand fragments (the stage being multiplied and the next
  // one) must fit the 256 vector registers beside the accumulators; when they
  // do not, the A fragments of all tile rows but the last exist once and are
  // refilled for the next stage as soon as their tile row has been issued.
  // (DIRECT needs room for the fp32 values in flight as well.)
  static constexpr bool RECYCLE_A =
      2 * TERMS * (MT_ + NT_) * 4 > (DIRECT ? 128 : 256);
  static_assert(!DIRECT || (NSTAGE == 2 && TERMS <= 2),
                "DIRECT: two LDS buffers, one or two terms");
  static_assert(NCH % NW == 0, "chunks must divide evenly over the waves");
  static_assert(WM % 16 == 0 && WN % 16 == 0, "wave tile must be MFMA tiles");
  static_assert(NSTAGE >= 2 && NSTAGE <= 4, "ring depth");
  static_assert(CPW * NSTAGE < 64, "vmcnt is a 6-bit counter");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS of one compute unit");
};

template <class MT, int TERMS, int BM, int BN, int WGM, int WGN, int NSTAGE,
          bool RN_MAIN, int DIRECT = 0>
__global__ void __launch_bounds__(WGM *WGN * 64)
    tcec_gemm_kernel(const u32x4 *__restrict__ Ap, const u32x4 *__restrict__ Bp,
                     float *__restrict__ C, const int M, const int N,
                     const int KT, const int rb_a, const int rb_b,
                     const long long ldc, const float alpha,
                     const float beta, const float inv_scale, const int tiles_m,
                     const int tiles_n, const int vec_store,
                     const long long batch_stride_a,
                     const long long batch_stride_b,
                     const long long batch_stride_c, const int split_stages,
                     float *__restrict__ partial,
                     float *const *__restrict__ c_ptrs, const int batches,
                     const int splits, const int entry_per_xcd,
                     const unsigned tail_begin, const int tail_stages,
                     float *__restrict__ tail_partial, const DirectSource ds) {
  using Cfg = GemmConfig<MT, TERMS, BM, BN, WGM, WGN, NSTAGE, RN_MAIN, DIRECT>;
  typedef MT ab_vec __attribute__((ext_vector_type(8)));
  constexpr int NCH = Cfg::NCH, CH_A = Cfg::CH_A, CPW = Cfg::CPW;
  constexpr int MT_ = Cfg::MT_, NT_ = Cfg::NT_;
  constexpr int RBM = BM / 16, RBN = BN / 16;
  constexpr int CH_PER_RB = Cfg::CH_PER_RB;

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  u32x4 *const lds = reinterpret_cast<u32x4 *>(lds_raw);

  const unsigned lane = threadIdx.x & 63u;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave % WGM, wn = wave / WGM;

  // ---- work items.  One item is one output tile of one batch entry (and one
  // K slice under split-K).  A workgroup takes the items my_first,
  // my_first + my_step, ... of a list: the global -> LDS requests run on
  // across the item boundary, so that the next tile's first stages are
  // already in LDS when the current tile is stored.
  //   entry_per_xcd == 0: one list, tiles first, then batch entries, then
  //     slices, shared by all workgroups.  Within the tile grid, consecutive
  //     ids are spread over the 8 XCDs and then walk the grid in groups of
  //     GROUP tile rows, so that the workgroups resident on one XCD share A
  //     row panels and B column panels in its L2.
  //   entry_per_xcd == 1 (no split-K, gridDim.x a multiple of 8): XCD x, i.e.
  //     the workgroups with blockIdx.x % 8 == x, owns batch entries x, x+8,
  //     ...: the operands of an entry are then read into one L2 only.
  //   entry_per_xcd == 2 (split-K, gridDim.x a multiple of 8): the same list
  //     as for 0, cut into eight runs of ceil(items / 8), one per XCD.  A K
  //     slice of the operands is shared only by the tiles of that slice, so
  //     an XCD should hold as few slices as possible: 32 tiles x 8 slices
  //     become one whole slice per XCD, and each operand byte is read into
  //     one L2 instead of up to eight.
  // (the host keeps the item count below 2^31: 32-bit divisions only)
  constexpr unsigned XCDS = 8;
  const unsigned num_tiles = static_cast<unsigned>(tiles_m * tiles_n);
  const unsigned my_xcd = blockIdx.x % XCDS;
  const unsigned my_first = entry_per_xcd ? blockIdx.x / XCDS : blockIdx.x;
  const unsigned my_step = entry_per_xcd ? gridDim.x / XCDS : gridDim.x;
  const unsigned all_items = num_tiles * batches * splits;
  const unsigned run_len = (all_items + XCDS - 1) / XCDS; // entry_per_xcd == 2
  const unsigned run_begin = my_xcd * run_len;
  // K slices for the tiles of the last, partly empty round only (one entry,
  // no other split; tail_begin >= num_tiles switches it off): the tiles
  // tail_begin .. num_tiles-1 are cut into slices of tail_stages k stages,
  // the items after the whole tiles are (slice, tail tile) pairs, and a slice
  // writes its raw sums as a dense BM x BN tile to
  // tail_partial[slice][tail tile]; reduce_tail_kernel folds them into C.
  const unsigned tail_tiles = tail_begin < num_tiles ? num_tiles - tail_begin : 0;
  const unsigned tail_slices =
      tail_tiles ? (KT + tail_stages - 1) / tail_stages : 0;
  const unsigned list_items =
      entry_per_xcd == 1 ? num_tiles * ((batches - my_xcd + XCDS - 1) / XCDS)
      : entry_per_xcd == 2
          ? (run_begin >= all_items           ? 0u
             : all_items - run_begin < run_len ? all_items - run_begin
                                               : run_len)
      : tail_tiles ? tail_begin + tail_tiles * tail_slices
                   : all_items;
  if (my_first >= list_items)
    return; // nothing for this workgroup (before any barrier)
  const int n_my =
      static_cast<int>((list_items - my_first + my_step - 1) / my_step);
  struct Item {
    int tm, tn, batch, z;
    int tail; // index among the tail tiles, -1 for a whole tile
  };
  auto decode = [&](const int i) {
    const unsigned v = (entry_per_xcd == 2 ? run_begin : 0u) + my_first +
                       static_cast<unsigned>(i) * my_step;
    Item it;
    it.tail = -1;
    unsigned rest = v / num_tiles;
    unsigned pid = v - rest * num_tiles;
    if (tail_tiles && v >= tail_begin) {
      const unsigned w = v - tail_begin;
      it.z = static_cast<int>(w / tail_tiles);
      it.tail = static_cast<int>(w - it.z * tail_tiles);
      it.batch = 0;
      pid = tail_begin + it.tail;
    } else if (entry_per_xcd == 1) {
      it.z = 0;
      it.batch = static_cast<int>(my_xcd + XCDS * rest);
    } else {
      it.z = static_cast<int>(rest / batches);
      it.batch = static_cast<int>(rest - it.z * batches);
    }
    tile_of<(BM > BN ? 4u : 8u)>(pid, num_tiles, tiles_m, tiles_n,
                                 !entry_per_xcd, it.tm, it.tn);
    return it;
  };
  // Split-K: with `partial` set, slice z covers split_stages k stages from
  // z*split_stages on and the workgroup writes its raw sum (no alpha / beta)
  // to partial[z][batch] as a dense column-major M x N matrix;
  // reduce_splits_kernel adds the slices.  Used when there are too few output
  // tiles to fill the chip.
  auto slice_stages = [&](const Item &it) {
    return it.tail >= 0 ? tail_stages : split_stages;
  };
  auto stages_of = [&](const Item &it) {
    if (partial == nullptr && it.tail < 0)
      return KT;
    const int per = slice_stages(it);
    const int begin = it.z * per;
    return KT - begin < per ? KT - begin : per;
  };

  // ---- request cursor: the item and stage requested next, and the global
  // sources of the chunks this wave requests every stage of that item.
  // Row blocks past the end of a packed operand are clamped to the last real
  // one: the rows / columns computed from them are never stored.
  // The sources are wave-uniform byte addresses kept in scalar registers (the
  // empty asm statements pin them there); a lane adds its own 16-byte offset
  // in the request instruction.
  // A wave requests all terms of RPW row blocks per stage; the terms of one
  // row block and stage are adjacent in the packed operand, so one address
  // per row block serves them through the instruction's immediate offset.
  // Which row blocks: w, w + NW, w + 2 NW, ... with one or two terms (the
  // waves then ask for neighbouring row blocks at the same time; batched
  // 1024x1024x256 measured 276 against 258 effective TFLOPS) and for the
  // three-term 256x128 tile (16384^3: 29.5 against 30.0 ms), w*RPW ..
  // w*RPW + RPW-1 for the three-term 128x128 tile (16384^3: 240 against 219).
  // DIRECT: the sources are fp32 rows instead (gsrc[g]: first row of the row
  // block at the cursor's k) and a stage is 32 floats further along the rows.
  // A row block is fetched by two loads of eight rows each, eight lanes to a
  // row (one whole 128-byte line; lane l: row l/8 or 8 + l/8, clamped to the
  // operand's last row, floats 4*(l%8) .. +3: voff[g][0..1]).
  constexpr unsigned STAGE_BYTES =
      DIRECT ? 32u * 4u : CH_PER_RB * 1024u;          // one stage of a row block
  constexpr int RPW = CPW / CH_PER_RB;                // row blocks per wave
  constexpr bool STRIDED_RB = TERMS <= 2 || Cfg::RECYCLE_A;
  constexpr int RB_STEP = STRIDED_RB ? Cfg::NW : 1; // between a wave's row blocks
  static_assert(CPW % CH_PER_RB == 0, "a wave requests whole row blocks");
  unsigned long long gsrc[RPW];
  unsigned voff[DIRECT ? RPW : 1][2];
  unsigned lane_off = lane * 16u;
  int req_item = 0, req_st = 0, req_stages = 0;
  // DIRECT == 2 (k not a multiple of 32, k >= 4): floats from the start of the
  // cursor's stage to the end of the rows, the same for the stage whose values
  // wait in registers, and what a lane subtracts from its offset so that it
  // reads inside the rows.  In a row's last, shorter stage a lane whose four
  // floats would end past the row reads the row's last four floats instead
  // (`tail_shift` floats further back); before the split its values are moved
  // up by that shift and followed by zeros (zero_tail below).  The packed
  // operands are padded with zeros, so the results are the same bits.  (Moving
  // the offsets themselves when the cursor enters and leaves such a stage,
  // instead of one subtraction per load, was slower: 1024^2 x 1000 x 256 1.96
  // against 1.79 ms.)
  constexpr bool TAIL = DIRECT == 2;
  int req_left = 0, raw_left = 0;
  unsigned tail_off = 0;
  auto tail_shift = [&](const int left) {
    return direct_tail_shift(lane, left);
  };
  auto set_tail_off = [&]() {
    if constexpr (TAIL)
      tail_off = 4u * static_cast<unsigned>(tail_shift(req_left));
  };
  auto set_sources = [&](const int i) {
    const Item it = decode(i);
    req_stages = stages_of(it);
    const long long first_stage =
        partial != nullptr || it.tail >= 0
            ? static_cast<long long>(it.z) * slice_stages(it)
            : 0;
    if constexpr (TAIL) {
      req_left = ds.k - static_cast<int>(first_stage) * 32;
      set_tail_off();
    }
    if constexpr (DIRECT) {
      // the pointer arrays are read with scalar loads (constant address space)
      typedef const float *const __attribute__((address_space(4))) *ptr_array_t;
      const float *const Ab = ds.a_ptrs != nullptr
                                  ? ((ptr_array_t)ds.a_ptrs)[it.batch]
                                  : ds.A + it.batch * ds.a_bs;
      const float *const Bb = ds.b_ptrs != nullptr
                                  ? ((ptr_array_t)ds.b_ptrs)[it.batch]
                                  : ds.B + it.batch * ds.b_bs;
#pragma unroll
      for (int g = 0; g < RPW; g++) {
        const int r = STRIDED_RB ? wave + Cfg::NW * g : wave * RPW + g;
        const bool is_a = r < RBM;
        const int last = (is_a ? M : N) - 1;
        int row0 = is_a ? it.tm * BM + 16 * r : it.tn * BN + 16 * (r - RBM);
        row0 = row0 < last ? row0 : last;
        const long long ld = is_a ? ds.lda : ds.ldb;
        // (TAIL: base and offsets biased by four floats, so that a lane that
        // reads up to three floats before the stage's start - rows that end
        // one to three floats into their last stage - keeps an offset >= 0)
        gsrc[g] = reinterpret_cast<unsigned long long>(
            (is_a ? Ab : Bb) + row0 * ld + first_stage * 32 -
            (TAIL ? kDirectBias : 0));
        asm volatile("" : "+s"(gsrc[g]));
#pragma unroll
        for (int h = 0; h < 2; h++) {
          int mine = row0 + 8 * h + static_cast<int>(lane >> 3);
          mine = (mine < last ? mine : last) - row0;
          voff[g][h] = static_cast<unsigned>(mine * ld) * 4u +
                       16u * (lane & 7u) + (TAIL ? 4u * kDirectBias : 0u);
        }
      }
      return;
    }
#pragma unroll
    for (int g = 0; g < RPW; g++) {
      // row block inside the stage: A's, then B's
      const int r = STRIDED_RB ? wave + Cfg::NW * g : wave * RPW + g;
      const bool is_a = r < RBM;
      int rb = is_a ? it.tm * RBM + r : it.tn * RBN + (r - RBM);
      const int rb_end = is_a ? rb_a : rb_b;
      rb = rb < rb_end ? rb : rb_end - 1;
      const u32x4 *const base = is_a ? Ap + it.batch * batch_stride_a
                                     : Bp + it.batch * batch_stride_b;
      gsrc[g] = reinterpret_cast<unsigned long long>(
          base +
          (static_cast<long long>(rb) * KT + first_stage) * (CH_PER_RB * 64));
      asm volatile("" : "+s"(gsrc[g]));
    }
  };
  // after the last stage of the last item the cursor stays where it is: the
  // few redundant requests keep the in-flight count constant, so one
  // s_waitcnt immediate serves the whole loop
  auto advance_request = [&]() {
    if constexpr (TAIL)
      raw_left = req_left; // of the stage just loaded
    if (req_st + 1 < req_stages) {
      req_st++;
#pragma unroll
      for (int g = 0; g < RPW; g++) {
        gsrc[g] += STAGE_BYTES;
        asm volatile("" : "+s"(gsrc[g]));
      }
      if constexpr (TAIL) {
        req_left -= 32;
        set_tail_off();
      }
    } else if (req_item + 1 < n_my) {
      req_item++;
      req_st = 0;
      set_sources(req_item);
    }
  };

  f32x4 acc_main[MT_][NT_], acc_err[MT_][NT_];
  auto clear_acc = [&]() {
#pragma unroll
    for (int i = 0; i < MT_; i++)
#pragma unroll
      for (int j = 0; j < NT_; j++) {
        acc_main[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        acc_err[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
  };

  // Request chunk Q (of this wave's CPW chunks) of the cursor's stage; w_base
  // is the LDS byte offset of the wave's first chunk in the target buffer.
  auto wave_base = [&](const int buf) {
    return (buf * NCH + wave * (STRIDED_RB ? CH_PER_RB : CPW)) * 1024;
  };
  auto issue_chunk = [&](const int w_base, auto Q) {
    constexpr int q = decltype(Q)::value;
    // first chunk of the row block; the immediate offset of the instruction
    // moves the global and the LDS address alike to the chunk of term q%TERMS
    // (the lane offset is redefined in place once per row block: the address
    // is then formed here, as the instruction's scalar base + 32-bit lane
    // offset, and not hoisted into vector register pairs)
    if constexpr (q % CH_PER_RB == 0)
      asm volatile("" : "+v"(lane_off));
    __builtin_amdgcn_global_load_lds(
        reinterpret_cast<const __attribute__((address_space(1))) char *>(
            gsrc[q / CH_PER_RB]) +
            lane_off,
        (__attribute__((address_space(3))) void *)(lds_raw + w_base +
                                                   (q / CH_PER_RB) * RB_STEP *
                                                       CH_PER_RB * 1024),
        16, (q % CH_PER_RB) * 1024, 0);
  };

  // DIRECT: what a wave does per stage for each of its RPW row blocks instead
  // of the requests above.  A lane's eight floats (four from each of the two
  // loads of a row block) stay in registers from the load to the split one
  // step later:
  //   load_half  : the lane's four floats of half h (rows 8h .. 8h+7) of row
  //                block g at the cursor's stage
  //   split_step : one instruction of the split of a pair of them -> one
  //                register of each term
  //   write_half : the terms of a half as 8-byte halves of the 16-byte
  //                fragment positions of the stage image in LDS, where the
  //                packed operands would have been copied to
  using SplitTag = typename std::conditional<std::is_same<MT, _Float16>::value,
                                             mtk::wmma::half,
                                             mtk::wmma::bfloat16>::type;
  typedef MT s2_t __attribute__((ext_vector_type(2)));
  float raw[DIRECT ? RPW : 1][8];
  unsigned term[2][2];
  s2_t lead_h;     // a pair's leading terms and what its residual terms are
  float prep_r[2]; // rounded from, between the instructions of its split
  auto load_half = [&](auto G, auto H) {
    constexpr int g = decltype(G)::value, h = decltype(H)::value;
    // 16-byte loads; the address need only be a float's (global memory is
    // accessed in unaligned mode), so any leading dimension and base work
    typedef f32x4 __attribute__((aligned(4))) f32x4_u;
    typedef const __attribute__((address_space(1))) f32x4_u *vec_ptr;
    const auto *const p =
        reinterpret_cast<const __attribute__((address_space(1))) char *>(
            gsrc[g]);
    // (the offset is redefined in place so that the address is formed here,
    // as the instruction's scalar base + 32-bit lane offset, and not hoisted
    // into a vector register pair)
    asm volatile("" : "+v"(voff[g][h]));
    const f32x4 v = *reinterpret_cast<vec_ptr>(
        p + (TAIL ? voff[g][h] - tail_off : voff[g][h]));
#pragma unroll
    for (int x = 0; x < 4; x++)
      raw[g][4 * h + x] = v[x];
  };
  // instruction PH of the split of pair Q of row block G: 0 leading terms,
  // 1 and 2 what the residuals of the pair's two values are rounded from,
  // 3 and 4 the residual terms
  auto split_step = [&](auto G, auto Q, auto PH) {
    constexpr int g = decltype(G)::value, q = decltype(Q)::value,
                  ph = decltype(PH)::value;
    namespace sd = mtk::wmma::tcec::detail;
    if constexpr (ph == 0) {
      lead_h = sd::split2_lead<SplitTag>(
          sd::f32x2_t{raw[g][2 * q], raw[g][2 * q + 1]});
      term[0][q % 2] = __builtin_bit_cast(unsigned, lead_h);
    } else if constexpr (TERMS >= 2 && ph == 1) {
      prep_r[0] = sd::split2_prep<SplitTag, 0>(raw[g][2 * q], lead_h);
    } else if constexpr (TERMS >= 2 && ph == 2) {
      prep_r[1] = sd::split2_prep<SplitTag, 1>(raw[g][2 * q + 1], lead_h);
    } else if constexpr (TERMS >= 2 && ph == 3) {
      term[1][q % 2] = __builtin_bit_cast(
          unsigned, sd::split2_resid_lo<SplitTag>(lead_h, prep_r[0]));
    } else if constexpr (TERMS >= 2) {
      term[1][q % 2] = __builtin_bit_cast(
          unsigned,
          sd::split2_resid_hi<SplitTag>(
              __builtin_bit_cast(s2_t, term[1][q % 2]), lead_h, prep_r[0],
              prep_r[1]));
    }
  };
  // A lane's four values of a load are half of a fragment position (row r,
  // k group q = k/8 of the stage): position r + 16*q of the chunk, stored at
  // 16-byte slot 16*q + (r ^ swz(q)), swz = 0, 12, 4, 8.  The lanes of a
  // load that hold the same row differ in q; without the permutation their
  // 8-byte writes fall on the same banks (measured at 8192^3: bank-conflict
  // cycles 6.1e8 with slots in position order, 4.1e8 with a rotation by 4*q,
  // 2.0e8 with this one; the 16-byte fragment reads, lane = position, stay
  // conflict free).
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  unsigned woff[2];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const unsigned r = 8u * h + (lane >> 3), q = (lane & 7u) >> 1;
    woff[h] = 256u * q + 16u * (r ^ direct_swizzle(q)) + 8u * (lane & 1u);
  }
  auto write_half = [&](const int w_base, auto G, auto H) {
    constexpr int g = decltype(G)::value, h = decltype(H)::value;
#pragma unroll
    for (int t = 0; t < TERMS; t++)
      *reinterpret_cast<u32x2 *>(lds_raw + w_base +
                                 g * RB_STEP * CH_PER_RB * 1024 + t * 1024 +
                                 woff[h]) = u32x2{term[t][0], term[t][1]};
  };
  // TAIL: when the stage waiting in registers is a row's last, shorter one, the
  // lanes that read further back take their own floats from what they read
  // (value x is the one read at x + shift) and zeros past the row's end, before
  // any of the stage is split (one branch per step; the rare side waits for all
  // of the stage's loads at once)
  auto zero_tail = [&]() {
    if constexpr (TAIL) {
      if (__builtin_expect(raw_left < 32, 0)) {
        const int shift = tail_shift(raw_left);
        if (shift > 0) {
#pragma unroll
          for (int g = 0; g < RPW; g++)
#pragma unroll
            for (int h = 0; h < 2; h++) {
              const float v0 = raw[g][4 * h], v1 = raw[g][4 * h + 1],
                          v2 = raw[g][4 * h + 2], v3 = raw[g][4 * h + 3];
              raw[g][4 * h] = shift == 1 ? v1 : shift == 2 ? v2 : shift == 3 ? v3 : 0.f;
              raw[g][4 * h + 1] = shift == 1 ? v2 : shift == 2 ? v3 : 0.f;
              raw[g][4 * h + 2] = shift == 1 ? v3 : 0.f;
              raw[g][4 * h + 3] = 0.f;
            }
        }
      }
    }
  };
  // A step's producer work, cut into micro-operations of one instruction each
  // (a half's writes: one per term) so that no matrix instruction is followed
  // by a burst of vector instructions.  The matrix pipe cannot run ahead of the
  // wave's issue: five vector instructions after every fourth MFMA cost a bare
  // stream of these MFMAs 15 %, the same five spread evenly nothing.  Per row
  // block and half (the eight rows of one load): the five instructions of each
  // of its two pairs, the writes of the half, the load of the same half of the
  // stage after.
  constexpr int UOPS_PER_HALF = 2 * 5 + 2;
  constexpr int NUOP = RPW * 2 * UOPS_PER_HALF;
  auto direct_uop = [&](const int w_base, auto U) {
    constexpr int u = decltype(U)::value, g = u / (2 * UOPS_PER_HALF),
                  h = (u / UOPS_PER_HALF) % 2, o = u % UOPS_PER_HALF;
    if constexpr (o < 10)
      split_step(ic<g>{}, ic<2 * h + o / 5>{}, ic<o % 5>{});
    else if constexpr (o == 10)
      write_half(w_base, ic<g>{}, ic<h>{});
    else
      load_half(ic<g>{}, ic<h>{});
  };

  // In-place accumulate, written as inline assembly so that every accumulator
  // stays in one fixed accumulation register for the whole K loop (with the
  // largest tile the accumulators fill the register file exactly, and the
  // register allocator otherwise shuffles them every iteration).  The only
  // dependence between the MFMAs of a step is an MFMA whose accumulator is
  // the destination of the one just before it, same shape and same
  // registers, which the matrix core takes back to back without software
  // wait states (the compiler emits none for the builtin either).  Small wave
  // tiles use the builtin.
  constexpr bool USE_ASM = MT_ * NT_ >= 8;
  auto mfma_acc = [](f32x4 &z, const ab_vec x, const ab_vec y) {
    if constexpr (std::is_same<MT, _Float16>::value)
      asm volatile(WMMAE_MFMA_GUARD "v_mfma_f32_16x16x32_f16 %0, %1, %2, %0"
                   : "+a"(z)
                   : "v"(x), "v"(y));
    else
      asm volatile(WMMAE_MFMA_GUARD "v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                   : "+a"(z)
                   : "v"(x), "v"(y));
  };
  auto mfma = [](const ab_vec x, const ab_vec y, const f32x4 z) -> f32x4 {
    if constexpr (std::is_same<MT, _Float16>::value)
      return __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, z, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, z, 0, 0, 0);
  };

  // Operand fragments of one stage: TERMS chunks per 16-row block.  With
  // RECYCLE_A a Frags holds the B fragments and the A fragments of the last
  // tile row only; the other tile rows' A fragments live once, in a_once.
  constexpr bool RECYCLE = Cfg::RECYCLE_A;
  struct Frags {
    ab_vec a[TERMS][RECYCLE ? 1 : MT_];
    ab_vec b[TERMS][NT_];
  };
  ab_vec a_once[TERMS][RECYCLE ? MT_ - 1 : 1];
  auto a_frag = [&](const Frags &f, auto T_, auto I_) -> const ab_vec & {
    constexpr int t = decltype(T_)::value, i = decltype(I_)::value;
    if constexpr (!RECYCLE)
      return f.a[t][i];
    else if constexpr (i < MT_ - 1)
      return a_once[t][i];
    else
      return f.a[t][0];
  };
  constexpr int NFRAG = TERMS * (MT_ + NT_);
  // 16-byte slot of this lane's fragment inside a chunk: the lane itself, or
  // with DIRECT the permuted slot the chunks were written with
  const unsigned frag_slot =
      DIRECT ? (lane & 48u) + ((lane & 15u) ^ direct_swizzle(lane >> 4)) : lane;
  // fragment IDX of a stage (compile-time index, so that every fragment is a
  // fixed register): B fragments first, then A (RECYCLE: A's last tile row
  // first, then rows 0 .. MT_-2)
  auto read_frag = [&](Frags &f, const int r_base, auto IDX) {
    constexpr int r = decltype(IDX)::value;
    const u32x4 *const stage =
        reinterpret_cast<const u32x4 *>(lds_raw + r_base) + frag_slot;
    if constexpr (r < TERMS * NT_) {
      constexpr int j = r / TERMS, t = r % TERMS;
      const u32x4 *const sb = stage + (CH_A + wn * NT_ * CH_PER_RB) * 64;
      f.b[t][j] = __builtin_bit_cast(ab_vec, sb[(j * CH_PER_RB + t) * 64]);
    } else {
      constexpr int ra = r - TERMS * NT_, t = ra % TERMS;
      constexpr int i = !RECYCLE ? ra / TERMS
                                 : (ra < TERMS ? MT_ - 1 : ra / TERMS - 1);
      const u32x4 *const sa = stage + (wm * MT_ * CH_PER_RB) * 64;
      const ab_vec v =
          __builtin_bit_cast(ab_vec, sa[(i * CH_PER_RB + t) * 64]);
      if constexpr (!RECYCLE)
        f.a[t][i] = v;
      else if constexpr (i < MT_ - 1)
        a_once[t][i] = v;
      else
        f.a[t][0] = v;
    }
  };

  // MFMAs of one step in issue order: tile after tile, and for every tile the
  // error products (smallest first) and then the main product.
  constexpr int NPROD = TERMS == 1 ? 1 : (TERMS == 2 ? 3 : 6);
  constexpr int NTILE = MT_ * NT_;
  constexpr int NMFMA = NPROD * NTILE;
  // LDS read r of the next stage goes out after MFMA number (r+1)*SPAN/NFRAG:
  // the reads are spread over the first three quarters of the step (the LGKM
  // counter only tracks 15 outstanding operations)
  // The requests of a step are spread over the whole step; with a ring of two
  // stages they must have landed when the next step begins and go out in the
  // step's first half (16384^3, three terms, 256x128 tile, requests within the
  // first 1/8, 1/4, 1/3, 1/2, 2/3, 3/4, 5/6 of the step and over all of it:
  // 33.1, 31.4, 30.3, 29.4, 29.3, 30.6, 31.3, 32.8 ms).
    constexpr int REQ_SPAN = NSTAGE == 2 ? (NMFMA / 2 > 0 ? NMFMA / 2 : 1) : NMFMA;
  // MFMA after which the last request of a step goes out
  constexpr int N_ADVANCE = (REQ_SPAN * (CPW - 1)) / CPW;
  constexpr int SPAN = (NMFMA * 3) / 4 > 0 ? (NMFMA * 3) / 4 : 1;
  // RECYCLE: MFMA after which read r of the next stage goes out.  The B
  // fragments and A's last tile row (separate registers) during the first tile
  // row; the A fragments of tile row i, which overwrite the current stage's,
  // right after the last MFMA of that row has been issued (the matrix core
  // has taken its operands by then; the LDS data arrives much later).
  constexpr int ROW_MFMA = NT_ * NPROD;
  constexpr int FIRST_READS = TERMS * (NT_ + 1);
  constexpr auto recycle_slot = [](const int r) constexpr {
    return recycled_read_slot(r, FIRST_READS, ROW_MFMA, TERMS);
  };

  // One pipeline step: multiply the fragments of stage st (already in
  // registers) while the fragments of stage st+1 are read from LDS and stage
  // st+NSTAGE is requested from HBM.  After the barrier every wave holds
  // stage st in registers, so its LDS buffer is free for the new request.
  // Memory instructions are spread between the MFMAs so that the single wave
  // of a SIMD never sits on a full memory queue while the matrix core idles.
  // `skip_waits` > 0: the requests this step depends on were awaited before
  // the previous tile's stores went out (see the epilogue), only the barrier
  // is needed.
  int skip_waits = 0;
  auto step = [&](const Frags &cur, Frags &nxt, const int wbuf,
                  const int rbuf) {
    // LDS offsets of this step, worked out before the barrier so that nothing
    // stands between it and the first MFMA
    int w_base = wave_base(wbuf);
    int r_base = rbuf * (NCH * 1024);
    asm volatile("" : "+s"(w_base), "+s"(r_base));
    // own loads of the next stage landed; own LDS reads of this stage finished
    // the requests of the stage read next are older than those of the
    // NSTAGE-2 stages after it (the branch sits before the barrier, where
    // the wave waits anyway)
    // (DIRECT: the stage read next was written to LDS by the waves
    // themselves during the last step; the barrier publishes it)
    if constexpr (!DIRECT) {
      if (skip_waits > 0)
        skip_waits--;
      else
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(CPW * (NSTAGE - 2))
                     : "memory");
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    zero_tail();

    static_for<0, NMFMA>([&](auto N_) {
      constexpr int n = decltype(N_)::value;
      // Tile-major order: the products of one tile follow each other (the
      // error products chained through its error accumulator, then the main
      // product), tiles in serpentine order so that neighbouring tiles share
      // the A fragment along a row and the B fragment at the turn.  Each
      // accumulator sees the same sequence of products as in a product-major
      // sweep, so the result bits do not depend on this choice; a chain of
      // MFMAs on one accumulator costs the matrix core less power than the
      // same MFMAs spread over many accumulators, and under the power limit
      // that is time (16384^3, three bf16 terms: 35.0 -> 33.1 ms; 4096^3 fp16:
      // 0.289 -> 0.280 ms).  The hardware supports back-to-back dependent
      // MFMAs of one shape on one destination without wait states.
      constexpr int p = n % NPROD;
      constexpr int tile = n / NPROD;
      constexpr int i = tile / NT_;
      constexpr int j = (i % 2) ? NT_ - 1 - tile % NT_ : tile % NT_;
      // (term of A, term of B) of product p
      constexpr int ta =
          TERMS == 1   ? 0
          : TERMS == 2 ? (p == 0 ? 1 : 0)
                       : (p == 0 ? 2 : p == 1 ? 0 : p == 2 ? 1 : p == 3 ? 1 : 0);
      constexpr int tb =
          TERMS == 1   ? 0
          : TERMS == 2 ? (p == 1 ? 1 : 0)
                       : (p == 0 ? 0 : p == 1 ? 2 : p == 2 ? 1 : p == 3 ? 0
                                                           : p == 4   ? 1
                                                                      : 0);
      constexpr bool is_main = p == NPROD - 1;
      if constexpr (is_main && RN_MAIN) {
        acc_main[i][j] += mfma(a_frag(cur, ic<0>{}, ic<i>{}), cur.b[0][j],
                               f32x4{0.f, 0.f, 0.f, 0.f});
      } else if constexpr (USE_ASM) {
        mfma_acc(is_main ? acc_main[i][j] : acc_err[i][j],
                 a_frag(cur, ic<ta>{}, ic<i>{}), cur.b[tb][j]);
      } else if constexpr (is_main) {
        acc_main[i][j] = mfma(a_frag(cur, ic<ta>{}, ic<i>{}), cur.b[tb][j],
                              acc_main[i][j]);
      } else {
        acc_err[i][j] = mfma(a_frag(cur, ic<ta>{}, ic<i>{}), cur.b[tb][j],
                             acc_err[i][j]);
      }
      if constexpr (DIRECT) {
        // split the stage after next (loaded during the last step) into the
        // buffer the current stage has left, load the stage after that: the
        // micro-operations spread evenly over the step
        constexpr int ulo =
            direct_uops_before(n, RECYCLE, NUOP, NFRAG, NMFMA, SPAN,
                               FIRST_READS, ROW_MFMA, TERMS);
        constexpr int uhi =
            direct_uops_before(n + 1, RECYCLE, NUOP, NFRAG, NMFMA, SPAN,
                               FIRST_READS, ROW_MFMA, TERMS);
        static_assert(ulo <= uhi && uhi <= NUOP &&
                          (n + 1 < NMFMA || uhi == NUOP),
                      "every micro-operation of a step is issued once");
        static_for<ulo, uhi>([&](auto U) {
          direct_uop(w_base, U);
          __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (n == NMFMA - 1) {
          advance_request();
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        // global->LDS requests due after this MFMA
        constexpr int qlo = (n * CPW + REQ_SPAN - 1) / REQ_SPAN;
        constexpr int qhi = ((n + 1) * CPW + REQ_SPAN - 1) / REQ_SPAN;
        static_for<(qlo < CPW ? qlo : CPW), (qhi < CPW ? qhi : CPW)>(
            [&](auto Q) {
              issue_chunk(w_base, Q);
              __builtin_amdgcn_sched_barrier(0);
            });
        // all requests of this step are out: move the cursor on while the
        // remaining MFMAs run
        if constexpr (n == N_ADVANCE) {
          advance_request();
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // LDS reads due after this MFMA
      if constexpr (RECYCLE) {
        static_for<0, NFRAG>([&](auto R_) {
          if constexpr (recycle_slot(decltype(R_)::value) == n) {
            read_frag(nxt, r_base, R_);
            __builtin_amdgcn_sched_barrier(0);
          }
        });
      } else {
        constexpr int lo = n == 0 ? 0 : reads_due(n, SPAN, NFRAG);
        constexpr int hi =
            n + 1 == NMFMA ? NFRAG : reads_due(n + 1, SPAN, NFRAG);
        static_for<lo, hi>([&](auto R_) {
          read_frag(nxt, r_base, R_);
          __builtin_amdgcn_sched_barrier(0);
        });
      }
    });
  };

  // ---- epilogue of one item: recombine, scale, store
  const int M_ = M, N_ = N;
  auto store_item = [&](const Item &it) {
    const bool to_tail = it.tail >= 0;
    const bool to_partial = partial != nullptr || to_tail;
    float *const Cb =
        to_tail ? tail_partial +
                      (static_cast<long long>(it.z) * tail_tiles + it.tail) *
                          (BM * BN)
        : to_partial
            ? partial + (static_cast<long long>(it.z) * batches + it.batch) *
                            (static_cast<long long>(M) * N)
            : (c_ptrs != nullptr ? c_ptrs[it.batch]
                                 : C + it.batch * batch_stride_c);
    // a tail slice stores its whole tile, tile-local, into its own BM x BN area
    const int M = to_tail ? BM : M_;
    const int N = to_tail ? BN : N_;
    const long long ld_out = to_tail ? BM : (to_partial ? M : ldc);
    const float a_out = to_partial ? 1.f : alpha;
    const float b_out = to_partial ? 0.f : beta;
    const int vec_out =
        to_tail      ? 1
        : to_partial ? (M % 4 == 0)
                     : (vec_store && (reinterpret_cast<uintptr_t>(Cb) & 15u) == 0);
    const int row_base = (to_tail ? 0 : it.tm * BM) + wm * Cfg::WM +
                         4 * static_cast<int>(lane >> 4);
    const int col_base = (to_tail ? 0 : it.tn * BN) + wn * Cfg::WN +
                         static_cast<int>(lane & 15u);
    // the value of tile (i, j) as it goes to memory, before beta
    const auto out_value = [&](const int i, const int j) {
      f32x4 v = acc_main[i][j];
      if constexpr (TERMS >= 2)
        v = epilogue_fold(v, acc_err[i][j], inv_scale);
      return v * a_out;
    };
    // (every destination is device memory: global-memory instructions, not
    // generic ones, which would also count as LDS operations and make the
    // compiler drain both memory counters before the next step's first
    // dependent instruction)
    typedef __attribute__((address_space(1))) float gfloat;
    typedef __attribute__((address_space(1))) f32x4 gf32x4;
    // one 16x16 tile: a lane stores rows 4q .. 4q+3 of its column, 16 bytes
    const auto store_tile = [&](const int i, const int j) {
      const int col = col_base + 16 * j;
      const int row = row_base + 16 * i;
      if (col >= N || row >= M)
        return;
      f32x4 v = out_value(i, j);
      gfloat *const dst =
          (gfloat *)(Cb + row + static_cast<long long>(col) * ld_out);
      if (vec_out && row + 3 < M) {
        if (b_out != 0.f)
          v = epilogue_beta(v, b_out, *reinterpret_cast<const gf32x4 *>(dst));
        *reinterpret_cast<gf32x4 *>(dst) = v;
      } else {
#pragma unroll
        for (int x = 0; x < 4; x++) {
          if (row + x < M) {
            float o = v[x];
            if (b_out != 0.f)
              o = epilogue_beta(o, b_out, dst[x]);
            dst[x] = o;
          }
        }
      }
    };
    // Two tiles of one tile column (32 rows x 16 columns, all inside C): as
    // above a store instruction would write 64 bytes of every column.  The
    // lanes of neighbouring columns swap one tile's values instead, so that
    // eight lanes cover 32 consecutive rows of one column: an instruction
    // writes whole 128-byte lines, first of the even columns, then of the odd.
    // Forced packed path, same box: 1024^2 x 128 x 256 entries 0.458 -> 0.434
    // ms, 2048^2 x 256 x 16 0.152 -> 0.145, one term 0.336 -> 0.314, 4096^3
    // 0.322 -> 0.318.  The kernel that splits the fp32 operands itself has no
    // register to spare: with the choice made per pair of tiles, as here, the
    // compiler keeps the accumulators' values in sight of three store paths
    // at once, and two more of its K loop's values went to scratch (c5b 1.45
    // -> 1.60 ms).  It decides once per item instead (below): the wave's whole
    // piece inside C -> every pair by the swap, else the plain loop; that
    // costs no scratch at all, and 1024 entries of 256^3 go from 0.175 to
    // 0.166 ms, 1024^2 x 128 x 256 entries from 0.389 to 0.355.  Not in the
    // round-to-nearest variants (their fragments then come back from AGPR
    // copies right in front of the MFMAs that read them, see
    // wmma_extension_amd/isa_check.py).
    constexpr bool WHOLE_LINES = !DIRECT && !RN_MAIN && MT_ % 2 == 0;
    const int odd = static_cast<int>(lane & 1u);
    const int blk_row0 = (to_tail ? 0 : it.tm * BM) + wm * Cfg::WM;
    const int blk_col0 = (to_tail ? 0 : it.tn * BN) + wn * Cfg::WN;
    const auto store_tile_pair = [&](const int i, const int j) {
      const f32x4 v0 = out_value(i, j), v1 = out_value(i + 1, j);
      f32x4 d1, d2;
#pragma unroll
      for (int x = 0; x < 4; x++) {
        // (through a function taking the element by value: __builtin_bit_cast
        // applied to `v0[x]` directly read element 0 for every x)
        const float n0 = neighbour_lane(v0[x]), n1 = neighbour_lane(v1[x]);
        d1[x] = odd ? n1 : v0[x]; // even column: own rows | neighbour's next 16
        d2[x] = odd ? v1[x] : n0; // odd column
      }
      const int row = row_base + 16 * (i + odd);
      const int col = col_base + 16 * j;
      gfloat *const dst1 =
          (gfloat *)(Cb + row + static_cast<long long>(col & ~1) * ld_out);
      gfloat *const dst2 =
          (gfloat *)(Cb + row + static_cast<long long>(col | 1) * ld_out);
      if (b_out != 0.f) {
        d1 = epilogue_beta(d1, b_out, *reinterpret_cast<const gf32x4 *>(dst1));
        d2 = epilogue_beta(d2, b_out, *reinterpret_cast<const gf32x4 *>(dst2));
      }
      *reinterpret_cast<gf32x4 *>(dst1) = d1;
      *reinterpret_cast<gf32x4 *>(dst2) = d2;
    };
    if constexpr (DIRECT && !RN_MAIN && MT_ % 2 == 0) {
      // the wave's whole piece inside C: every pair by the swap, no other
      // path in sight of the accumulators (one decision per item)
      if (vec_out && blk_row0 + Cfg::WM <= M && blk_col0 + Cfg::WN <= N) {
#pragma unroll
        for (int j = 0; j < NT_; j++)
#pragma unroll
          for (int i = 0; i < MT_; i += 2)
            store_tile_pair(i, j);
        return;
      }
    }
#pragma unroll
    for (int j = 0; j < NT_; j++) {
      const bool cols_inside = blk_col0 + 16 * j + 16 <= N;
      if constexpr (WHOLE_LINES) {
#pragma unroll
        for (int i = 0; i < MT_; i += 2) {
          // (wave-uniform: both lanes of a swap take the same branch)
          if (vec_out && cols_inside && blk_row0 + 16 * i + 32 <= M) {
            store_tile_pair(i, j);
          } else {
            store_tile(i, j);
            store_tile(i + 1, j);
          }
        }
      } else {
        // (the loop as one piece, with the compiler's own contraction of
        // a * x + b * y, which comes out in the helpers' form: the kernel that
        // splits its own operands has no register to spare, and through
        // store_tile one more of its K loop's values went to scratch)
        const int col = col_base + 16 * j;
        if (col >= N)
          continue;
#pragma unroll
        for (int i = 0; i < MT_; i++) {
          const int row = row_base + 16 * i;
          if (row >= M)
            continue;
          f32x4 v = acc_main[i][j];
          if constexpr (TERMS >= 2)
            v += acc_err[i][j] * inv_scale;
          v *= a_out;
          gfloat *const dst =
              (gfloat *)(Cb + row + static_cast<long long>(col) * ld_out);
          if (vec_out && row + 3 < M) {
            if (b_out != 0.f)
              v += b_out * *reinterpret_cast<const gf32x4 *>(dst);
            *reinterpret_cast<gf32x4 *>(dst) = v;
          } else {
#pragma unroll
            for (int x = 0; x < 4; x++) {
              if (row + x < M) {
                float o = v[x];
                if (b_out != 0.f)
                  o += b_out * dst[x];
                dst[x] = o;
              }
            }
          }
        }
      }
    }
  };

  // DIRECT, launches bound by their bytes (batches of small matrices with few
  // k stages per tile): workgroups that start together stay in step, so the
  // whole chip fills its pipelines at once, stores its tiles at once and
  // finishes at once, and the memory system idles in between.  The host asks
  // for the 32 workgroups of an XCD to start a fraction of a microsecond apart
  // (1024 entries of 256^3: 0.186 -> 0.174 ms with 32 x 512 cycles, no gain
  // from 2 or 4 phases, less from longer delays; launches bound by their
  // arithmetic only lose the delay and are not staggered).
  if constexpr (DIRECT) {
    if (ds.stagger > 0) {
      const int periods = static_cast<int>((blockIdx.x / XCDS) % 32u) * ds.stagger;
      for (int d = 0; d < periods; d++)
        __builtin_amdgcn_s_sleep(8); // 8 x 64 cycles
    }
  }
  // ---- prologue: request the first NSTAGE stages of the stream, fetch the
  // first stage's fragments
  set_sources(0);
  Frags f0, f1;
  if constexpr (DIRECT) {
    // stages 0 and 1 of the stream into the two LDS buffers, stage 2 into
    // the registers
    static_for<0, RPW>([&](auto G) {
      load_half(G, ic<0>{});
      load_half(G, ic<1>{});
    });
    advance_request();
#pragma unroll
    for (int s = 0; s < 2; s++) {
      zero_tail();
      static_for<0, NUOP>([&](auto U) { direct_uop(wave_base(s), U); });
      advance_request();
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  } else {
#pragma unroll
    for (int s = 0; s < NSTAGE; s++) {
      static_for<0, CPW>([&](auto Q) { issue_chunk(wave_base(s), Q); });
      advance_request();
    }
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(CPW * (NSTAGE - 1))
                 : "memory");
  }
  static_for<0, NFRAG>([&](auto R_) { read_frag(f0, 0, R_); });

  // ---- items; the stage loop is unrolled by two so that the fragment sets
  // swap by name.  Every step reads the fragments of the stream's next stage,
  // which after an item's last stage is the first stage of the next item.
  int wbuf = 0; // buffer of the stage being multiplied == next to be refilled
  auto next_buf = [](const int b2) { return b2 + 1 == NSTAGE ? 0 : b2 + 1; };
  for (int item = 0; item < n_my; item++) {
    const Item it = decode(item);
    const int num_stages = stages_of(it);
    clear_acc();
    int st = 0;
    for (; st + 1 < num_stages; st += 2) {
      const int b1 = next_buf(wbuf);
      step(f0, f1, wbuf, b1);
      const int b2 = next_buf(b1);
      step(f1, f0, b1, b2);
      wbuf = b2;
    }
    if (st < num_stages) {
      // odd stage count: the next item's first fragments arrive in f1
      const int b1 = next_buf(wbuf);
      step(f0, f1, wbuf, b1);
      wbuf = b1;
      f0 = f1;
    }
    // The stores of C share the memory counter with the requests, and loads
    // and stores need not complete in issue order, so a counted wait behind
    // the stores would have to sit them out.  Everything requested so far is
    // awaited here instead, before the stores go out; the steps that only
    // depend on those requests skip their counted wait.  The no-ops cover the
    // matrix core's write-to-VALU-read distance for the last accumulate
    // instructions, which the compiler cannot see.
    // (DIRECT: the loads in flight fill registers, which the compiler tracks
    // itself; they need not have landed here.)
    if constexpr (DIRECT)
      asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    // (the reads of the accumulators must not be scheduled above the no-ops)
    __builtin_amdgcn_sched_barrier(0);
    skip_waits = NSTAGE - 1;
    store_item(it);
  }
  // the redundant tail requests must not outlive the workgroup's LDS allocation
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
}

} // namespace wmmae_gemm
