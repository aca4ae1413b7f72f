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
//   packed[rb][kt][term][lane] : one 16-byte chunk per lane; lane l of the chunk
//       holds row 16*rb + l%16, k = 32*kt + 8*(l/16) .. +7 of that term
//
// so one 1 KiB chunk is one MFMA operand for a whole wave.  The GEMM kernel
// then moves chunks HBM -> LDS -> registers with perfectly linear 128-bit
// accesses (no padding, no swizzle, no bank conflicts) and does no
// conversion work in its K loop.  Both operands use the same packing
// ("rows" are the m index for A and the n index for B), so any BLAS
// transpose combination is handled by the strides given to the split kernel.
#pragma once
#include <wmma_extension/tcec/tcec.hpp>

namespace wmmae_gemm {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kChunkRows = 16; // rows per packed chunk (MFMA M / N)
constexpr int kChunkK = 32;    // k per packed chunk (MFMA K)

// --------------------------------------------------------------------------
// split_pack_kernel: X (fp32, element (r,k) at X[r*row_stride + k*k_stride])
// -> packed terms.  One thread per (chunk, lane).  Rows >= rows and k >= K are
// zero filled, so the GEMM kernel needs no edge handling on its loads.
//   T      : split tag (half, bfloat16, precision::tf32)
//   TERMS  : number of terms stored (1 = leading term only, i.e. no correction)
// --------------------------------------------------------------------------
template <class T, int TERMS>
__global__ void __launch_bounds__(256)
    split_pack_kernel(const float *__restrict__ X, const long long row_stride,
                      const long long k_stride, const int rows, const int K,
                      const int KT, const long long chunks,
                      const long long in_batch_stride,
                      u32x4 *__restrict__ out,
                      const long long out_batch_stride) {
  using traits = mtk::wmma::tcec::detail::split_traits<T>;
  using S = typename traits::storage;
  static_assert(TERMS >= 1 && TERMS <= traits::num_terms, "bad TERMS");
  const unsigned lane = threadIdx.x & 63u;
  const long long chunk =
      (static_cast<long long>(blockIdx.x) * 256 + threadIdx.x) >> 6;
  if (chunk >= chunks)
    return;
  const long long rb = chunk / KT;
  const int kt = static_cast<int>(chunk - rb * KT);
  const long long r = rb * kChunkRows + (lane & 15u);
  const int k0 = kt * kChunkK + 8 * static_cast<int>(lane >> 4);

  float v[8];
#pragma unroll
  for (int x = 0; x < 8; x++)
    v[x] = 0.f;
  if (r < rows && k0 < K) {
    const float *p = X + blockIdx.y * in_batch_stride + r * row_stride +
                     static_cast<long long>(k0) * k_stride;
    if (k_stride == 1 && k0 + 8 <= K &&
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
          v[x] = p[x * k_stride];
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
  u32x4 *o = out + blockIdx.y * out_batch_stride + chunk * (TERMS * 64) + lane;
#pragma unroll
  for (int p = 0; p < TERMS; p++)
    o[p * 64] = __builtin_bit_cast(u32x4, t[p]);
}

// --------------------------------------------------------------------------
// scale_c_kernel: C = beta * C, the whole result when k == 0.
// --------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
    scale_c_kernel(float *__restrict__ C, const int M, const int N,
                   const long long ldc, const long long batch_stride_c,
                   const float beta) {
  const long long e = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  if (e >= static_cast<long long>(M) * N)
    return;
  float *const p = C + blockIdx.y * batch_stride_c + (e % M) + (e / M) * ldc;
  *p = beta == 0.f ? 0.f : beta * *p;
}

// --------------------------------------------------------------------------
// tcec_gemm_kernel: C = alpha * (A*B) + beta * C from packed operands.
//
//   MT      : MFMA element type (_Float16 or __bf16)
//   TERMS   : stored terms per operand (1, 2 or 3)
//   BM x BN : block tile, WGM x WGN waves, each wave (BM/WGM) x (BN/WGN)
//   KS      : 32-wide k steps per LDS stage
//   RN_MAIN : accumulate the leading product with fp32 adds outside the
//             matrix core (the reference's mma_rn_sync, tcec/tcec.hpp:673-694)
//             instead of chaining it through the MFMA accumulator
//
// Products issued per (16x16 tile, k step), all with fp32 accumulation:
//   TERMS 1: main += a0*b0
//   TERMS 2: main += a0*b0;  err += a1*b0 + a0*b1
//   TERMS 3: main += a0*b0;  err += a2*b0 + a0*b2 + a1*b1 + a1*b0 + a0*b1
// and the result is main + err * inv_scale (reference: tcec.hpp:332-336).
// The error terms have their own accumulator so that their low-order bits
// are not rounded away against the much larger main sum.
//
// C is column major (element (i,j) at C[i + j*ldc]); an accumulator lane owns
// four consecutive rows of one column, i.e. one 16-byte store.
// --------------------------------------------------------------------------
template <class MT, int TERMS, int BM, int BN, int WGM, int WGN, int KS,
          bool RN_MAIN>
struct GemmConfig {
  static constexpr int NW = WGM * WGN;
  static constexpr int NTHREADS = NW * 64;
  static constexpr int WM = BM / WGM, WN = BN / WGN;
  static constexpr int MT_ = WM / 16, NT_ = WN / 16;
  static constexpr int CH_A = (BM / 16) * KS * TERMS; // chunks per stage
  static constexpr int CH_B = (BN / 16) * KS * TERMS;
  static constexpr int NCH = CH_A + CH_B;
  static constexpr int CPW = NCH / NW; // chunks each wave moves per stage
  static constexpr int STAGES = 2;
  static constexpr int LDS_BYTES = STAGES * NCH * 1024;
  static_assert(NCH % NW == 0, "chunks must divide evenly over the waves");
  static_assert(WM % 16 == 0 && WN % 16 == 0, "wave tile must be MFMA tiles");
};

template <class MT, int TERMS, int BM, int BN, int WGM, int WGN, int KS,
          bool RN_MAIN>
__global__ void __launch_bounds__(WGM *WGN * 64)
    tcec_gemm_kernel(const u32x4 *__restrict__ Ap, const u32x4 *__restrict__ Bp,
                     float *__restrict__ C, const int M, const int N,
                     const int KT, const int rb_a, const int rb_b,
                     const long long ldc, const float alpha,
                     const float beta, const float inv_scale, const int tiles_m,
                     const int tiles_n, const int vec_store,
                     const long long batch_stride_a,
                     const long long batch_stride_b,
                     const long long batch_stride_c) {
  using Cfg = GemmConfig<MT, TERMS, BM, BN, WGM, WGN, KS, RN_MAIN>;
  typedef MT ab_vec __attribute__((ext_vector_type(8)));
  constexpr int NCH = Cfg::NCH, CH_A = Cfg::CH_A, CPW = Cfg::CPW;
  constexpr int MT_ = Cfg::MT_, NT_ = Cfg::NT_;
  constexpr int RBM = BM / 16, RBN = BN / 16;
  constexpr int CH_PER_RB = KS * TERMS; // contiguous chunks of one row block

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  u32x4 *const lds = reinterpret_cast<u32x4 *>(lds_raw);

  const unsigned lane = threadIdx.x & 63u;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave % WGM, wn = wave / WGM;

  // ---- block -> tile: spread consecutive ids over the 8 XCDs, then walk the
  // tile grid in groups of 8 tile rows so that the blocks resident on one XCD
  // share A row panels and B column panels in that XCD's L2.
  const int num_tiles = tiles_m * tiles_n;
  int pid = blockIdx.x;
  {
    constexpr int XCDS = 8;
    const int per = (num_tiles + XCDS - 1) / XCDS;
    const int tall = (num_tiles % XCDS == 0) ? XCDS : (num_tiles % XCDS);
    const int xcd = pid % XCDS, local = pid / XCDS;
    pid = xcd < tall ? xcd * per + local
                     : tall * per + (xcd - tall) * (per - 1) + local;
  }
  int tm, tn;
  {
    constexpr int GROUP = 8;
    const int width = GROUP * tiles_n;
    const int group = pid / width;
    const int first_m = group * GROUP;
    const int gsz = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    const int in_group = pid - group * width;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
  }
  const long long batch = blockIdx.y;

  // ---- global sources of the chunks this wave moves every stage
  // Row blocks past the end of a packed operand are clamped to the last real
  // one: the rows / columns computed from them are never stored.
  const u32x4 *gsrc[CPW];
  int slot[CPW];
#pragma unroll
  for (int q = 0; q < CPW; q++) {
    const int c = wave + Cfg::NW * q; // chunk index inside the stage
    slot[q] = c;
    if (c < CH_A) {
      const int rbl = c / CH_PER_RB, j = c % CH_PER_RB;
      int rb = tm * RBM + rbl;
      rb = rb < rb_a ? rb : rb_a - 1;
      gsrc[q] = Ap + batch * batch_stride_a +
                (static_cast<long long>(rb) * KT * TERMS + j) * 64;
    } else {
      const int cb = c - CH_A;
      const int rbl = cb / CH_PER_RB, j = cb % CH_PER_RB;
      int rb = tn * RBN + rbl;
      rb = rb < rb_b ? rb : rb_b - 1;
      gsrc[q] = Bp + batch * batch_stride_b +
                (static_cast<long long>(rb) * KT * TERMS + j) * 64;
    }
  }

  f32x4 acc_main[MT_][NT_], acc_err[MT_][NT_];
#pragma unroll
  for (int i = 0; i < MT_; i++)
#pragma unroll
    for (int j = 0; j < NT_; j++) {
      acc_main[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      acc_err[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

  u32x4 pre[CPW];
  const int num_stages = KT / KS; // host guarantees KT % KS == 0
  auto load_global = [&](const int st) {
    const long long off = static_cast<long long>(st) * (CH_PER_RB * 64) + lane;
#pragma unroll
    for (int q = 0; q < CPW; q++)
      pre[q] = gsrc[q][off];
  };
  auto store_lds = [&](const int buf) {
#pragma unroll
    for (int q = 0; q < CPW; q++)
      lds[(buf * NCH + slot[q]) * 64 + lane] = pre[q];
  };

  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int st = 0; st < num_stages; st++) {
    const int buf = st & 1;
    if (st + 1 < num_stages)
      load_global(st + 1);

    const u32x4 *const sa =
        lds + (buf * NCH + wm * MT_ * CH_PER_RB) * 64 + lane;
    const u32x4 *const sb =
        lds + (buf * NCH + CH_A + wn * NT_ * CH_PER_RB) * 64 + lane;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      ab_vec a[TERMS][MT_], b[TERMS][NT_];
#pragma unroll
      for (int i = 0; i < MT_; i++)
#pragma unroll
        for (int t = 0; t < TERMS; t++)
          a[t][i] = __builtin_bit_cast(
              ab_vec, sa[(i * CH_PER_RB + ks * TERMS + t) * 64]);
#pragma unroll
      for (int j = 0; j < NT_; j++)
#pragma unroll
        for (int t = 0; t < TERMS; t++)
          b[t][j] = __builtin_bit_cast(
              ab_vec, sb[(j * CH_PER_RB + ks * TERMS + t) * 64]);

      auto mfma = [](const ab_vec x, const ab_vec y, const f32x4 z) -> f32x4 {
        if constexpr (std::is_same<MT, _Float16>::value)
          return __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, z, 0, 0, 0);
        else
          return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, z, 0, 0, 0);
      };
      // error terms first (smallest products first), main product last
      if constexpr (TERMS >= 3) {
#pragma unroll
        for (int i = 0; i < MT_; i++)
#pragma unroll
          for (int j = 0; j < NT_; j++)
            acc_err[i][j] = mfma(a[2][i], b[0][j], acc_err[i][j]);
#pragma unroll
        for (int i = 0; i < MT_; i++)
#pragma unroll
          for (int j = 0; j < NT_; j++)
            acc_err[i][j] = mfma(a[0][i], b[2][j], acc_err[i][j]);
#pragma unroll
        for (int i = 0; i < MT_; i++)
#pragma unroll
          for (int j = 0; j < NT_; j++)
            acc_err[i][j] = mfma(a[1][i], b[1][j], acc_err[i][j]);
      }
      if constexpr (TERMS >= 2) {
#pragma unroll
        for (int i = 0; i < MT_; i++)
#pragma unroll
          for (int j = 0; j < NT_; j++)
            acc_err[i][j] = mfma(a[1][i], b[0][j], acc_err[i][j]);
#pragma unroll
        for (int i = 0; i < MT_; i++)
#pragma unroll
          for (int j = 0; j < NT_; j++)
            acc_err[i][j] = mfma(a[0][i], b[1][j], acc_err[i][j]);
      }
#pragma unroll
      for (int i = 0; i < MT_; i++)
#pragma unroll
        for (int j = 0; j < NT_; j++) {
          if constexpr (RN_MAIN) {
            const f32x4 tmp =
                mfma(a[0][i], b[0][j], f32x4{0.f, 0.f, 0.f, 0.f});
            acc_main[i][j] += tmp;
          } else {
            acc_main[i][j] = mfma(a[0][i], b[0][j], acc_main[i][j]);
          }
        }
    }

    if (st + 1 < num_stages)
      store_lds(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: recombine, scale, store
  float *const Cb = C + batch * batch_stride_c;
  const int row_base = tm * BM + wm * Cfg::WM + 4 * static_cast<int>(lane >> 4);
  const int col_base = tn * BN + wn * Cfg::WN + static_cast<int>(lane & 15u);
#pragma unroll
  for (int j = 0; j < NT_; j++) {
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
      v *= alpha;
      float *const dst = Cb + row + static_cast<long long>(col) * ldc;
      if (vec_store && row + 3 < M) {
        if (beta != 0.f)
          v += beta * *reinterpret_cast<const f32x4 *>(dst);
        *reinterpret_cast<f32x4 *>(dst) = v;
      } else {
#pragma unroll
        for (int x = 0; x < 4; x++) {
          if (row + x < M) {
            float o = v[x];
            if (beta != 0.f)
              o += beta * dst[x];
            dst[x] = o;
          }
        }
      }
    }
  }
}

} // namespace wmmae_gemm
