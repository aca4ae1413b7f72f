// TCEC SGEMM for gfx950 straight from the fp32 operands, for products that are
// bound by HBM rather than by the matrix cores (small matrices, usually
// batched: every element is needed by only a few workgroups).  The packed path
// (split_pack_kernel + tcec_gemm_kernel) would read and write every operand
// once more.  Here one kernel does it all:
//
//   HBM --global_load_lds--> raw fp32 ring in LDS (NRAW stages of 32 k)
//       --split in registers--> 16-bit terms in LDS, two stages, in the same
//         fragment-major chunk order the packed kernel uses
//       --ds_read_b128--> MFMA operands
//
// The reference's tiled GEMM has the same shape of data flow (fp32 tiles in
// shared memory, split at fragment load: test/tcec/batch_gemm.cu:196-386,
// tcec/tcec.hpp:213-229) but splits every element once per warp that needs it;
// here every element of a tile is split once per workgroup.
//
// Each wave requests, and later converts, the same row blocks, so the raw ring
// needs no workgroup barrier: the wave's own s_waitcnt vmcnt is enough.  The
// only barrier of a stage publishes the converted terms.
//
// Workgroups are persistent.  A workgroup walks a list of output tiles and
// treats (tile, k stage) pairs as one stream, so the loads of the next tile
// are in flight while the current one finishes and is written back: with
// 8 stages a tile (k = 256) a pipeline refill per tile would cost as much as
// the tile.  With eight or more batch entries, an XCD (blockIdx % 8) takes
// whole batch entries, so the tiles that share an operand panel share an L2.
//
// Raw layout of one 16-row block of a stage (2 KiB = 16 rows x 128 bytes).
// When k is contiguous and 16-byte aligned, two 16-byte requests per lane:
// request h covers rows 8h..8h+7, lane l fetching row 8h + l/8, so that eight
// lanes take one whole 128-byte line (requests that touch half lines ran the
// read stream at 4.1 instead of 5.2-6 TB/s).  Within its row, lane l fetches
// 16-byte piece (l%8) ^ (2*((l/16)%4) + h): the pieces of a row are stored
// permuted so that the conversion - where lane l needs the 32 bytes
// k = 8*(l/16) .. +7 of row r = l%16, found as two 16-byte halves at byte
// r*128 + 32*((l/16) ^ ((r/2)%4)), in swapped order for r >= 8 - does
// not have the sixteen rows of a read start in the same LDS banks (each
// ds_read_b128 of sixteen lanes covers all 64 banks once).  Otherwise (any
// stride, any alignment) eight 4-byte requests per lane, element e of the
// lane's eight into slot [e][l], read back from the same slots.
// Rows past the matrix are clamped to the last row (their results are never
// stored); k past K is clamped in the request and zeroed at the conversion.
//
// Operand element (r, l) of op(A) is A[r*a_rs + l*a_ks] (rows = m), of op(B) it
// is B[r*b_rs + l*b_ks] (rows = n); batch entry y is base + y*stride or ptrs[y].
// The products, their order and the epilogue are those of tcec_gemm_kernel, so
// both paths give the same bits.
#pragma once
#include "tcec_gemm_kernels.hpp"

namespace wmmae_gemm {

struct FusedParams {
  const float *A;
  const float *const *a_ptrs;
  long long a_rs, a_ks, a_bs;
  const float *B;
  const float *const *b_ptrs;
  long long b_rs, b_ks, b_bs;
  float *C;
  float *const *c_ptrs;
  long long ldc, c_bs;
  int M, N, K, batch;
  int tiles_m, tiles_per_batch;
  // XCD x (block index mod 8) owns the batch entries x, x+8, ... (set by the
  // launcher for 8 or more entries that spread evenly enough)
  int grouped;
  // 16-byte requests are possible as far as the host can tell: k contiguous,
  // K and the strides multiples of 4, base pointers aligned (pointer-array
  // entries are checked by the kernel)
  int vec_a, vec_b;
  int vec_store;
  // accumulate the leading product with fp32 adds outside the matrix core
  // (tcec_gemm_kernel's RN_MAIN; the reference's mma_rn_sync)
  int rn_main;
  float alpha, beta, inv_scale;
};

template <int TERMS, int BM, int BN, int NW = (BM * BN >= 128 * 128 ? 8 : 4)>
struct FusedConfig {
  static constexpr int NWAVES = NW;       // 2 x NW/2 waves
  static constexpr int NTHREADS = 64 * NW;
  static constexpr int RBA = BM / 16, RBB = BN / 16, NRB = RBA + RBB;
  static constexpr int NQ = NRB / NW; // row blocks per wave and stage
  static constexpr int RAW_STAGE_BYTES = NRB * 2048;
  static constexpr int FRAG_BYTES = 2 * NRB * TERMS * 1024;
  static constexpr int FIT = (160 * 1024 - FRAG_BYTES) / RAW_STAGE_BYTES;
  static constexpr int NRAW = FIT > 4 ? 4 : FIT;
  static constexpr int LDS_BYTES = NRAW * RAW_STAGE_BYTES + FRAG_BYTES;
  static_assert(RBA % NW == 0 && RBB % NW == 0,
                "row blocks divide over the waves");
  static_assert(NRAW >= 2, "raw ring too shallow");
};

template <int N> __device__ __forceinline__ void wait_vmcnt_at_most() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N > 63 ? 63 : N) : "memory");
}

template <class T, int TERMS, int BM, int BN,
          int NW = FusedConfig<TERMS, BM, BN>::NWAVES>
__global__ void __launch_bounds__(64 * NW)
    tcec_gemm_fused_kernel(const FusedParams p) {
  using traits = mtk::wmma::tcec::detail::split_traits<T>;
  using S = typename traits::storage;
  typedef S ab_vec __attribute__((ext_vector_type(8)));
  using Cfg = FusedConfig<TERMS, BM, BN, NW>;
  constexpr int RBA = Cfg::RBA, NRB = Cfg::NRB, NQ = Cfg::NQ;
  constexpr int NRAW = Cfg::NRAW;
  constexpr int WGN = NW / 2;
  constexpr int WM = BM / 2, WN = BN / WGN; // 2 x NW/2 waves
  constexpr int MT_ = WM / 16, NT_ = WN / 16;

  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[];
  u32x4 *const frag =
      reinterpret_cast<u32x4 *>(lds_raw + NRAW * Cfg::RAW_STAGE_BYTES);

  const unsigned lane = threadIdx.x & 63u;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  const int r16 = static_cast<int>(lane & 15u);
  const int g8 = 8 * static_cast<int>(lane >> 4);
  const int M = p.M, N = p.N, K = p.K;

  // ---- this workgroup's tiles: v = first + i*stride while v < count
  const int tpb = p.tiles_per_batch;
  const bool grouped = p.grouped != 0;
  const int xcd = grouped ? static_cast<int>(blockIdx.x & 7u) : 0;
  const int first = grouped ? static_cast<int>(blockIdx.x >> 3)
                            : static_cast<int>(blockIdx.x);
  const int stride = grouped ? static_cast<int>(gridDim.x >> 3)
                             : static_cast<int>(gridDim.x);
  const int count = grouped ? ((p.batch - xcd + 7) >> 3) * tpb : p.batch * tpb;
  if (first >= count)
    return;
  const int n_my = (count - first + stride - 1) / stride;
  auto decode = [&](const int i, int &entry, int &tm, int &tn) __attribute__((always_inline)) {
    const int v = first + i * stride;
    const int bi = v / tpb;
    const int t = v - bi * tpb;
    entry = grouped ? bi * 8 + xcd : bi;
    tn = t / p.tiles_m;
    tm = t - tn * p.tiles_m;
  };

  // ---- request width (uniform over the workgroup)
  int vec_a = p.vec_a, vec_b = p.vec_b;
  if (p.a_ptrs != nullptr || p.b_ptrs != nullptr) {
    int low_a = 0, low_b = 0;
    for (int i = threadIdx.x; i < n_my; i += 64 * NW) {
      int entry, tm, tn;
      decode(i, entry, tm, tn);
      if (p.a_ptrs != nullptr)
        low_a |= static_cast<int>(
            reinterpret_cast<uintptr_t>(p.a_ptrs[entry]) & 15u);
      if (p.b_ptrs != nullptr)
        low_b |= static_cast<int>(
            reinterpret_cast<uintptr_t>(p.b_ptrs[entry]) & 15u);
    }
    // workgroup-wide OR through the (still unused) start of the LDS ring
    int *const flags = reinterpret_cast<int *>(lds_raw);
    const int any_a = __builtin_amdgcn_ballot_w64(low_a != 0) != 0;
    const int any_b = __builtin_amdgcn_ballot_w64(low_b != 0) != 0;
    if (lane == 0)
      flags[wave] = any_a | (any_b << 1);
    __syncthreads();
    int all = 0;
#pragma unroll
    for (int w = 0; w < NW; w++)
      all |= flags[w];
    __syncthreads();
    if (all & 1)
      vec_a = 0;
    if (all & 2)
      vec_b = 0;
  }
  vec_a = __builtin_amdgcn_readfirstlane(vec_a);
  vec_b = __builtin_amdgcn_readfirstlane(vec_b);

  const int num_k = (K + 31) / 32;
  const int total = n_my * num_k; // stages in this workgroup's stream

  // ---- requests
  typedef const __attribute__((address_space(1))) float *gptr_t;
  gptr_t rowptr[NQ][2]; // [.][h]: row of request h (16-byte mode); [.][0] else
  auto set_rows = [&](auto VEC, const int i) __attribute__((always_inline)) {
    int entry, tm, tn;
    decode(i, entry, tm, tn);
    // the pointer arrays are read with scalar loads (constant address space):
    // a vector load here would make the compiler wait for every outstanding
    // request of the ring before it can use the pointer
    typedef const float *const __attribute__((address_space(4))) *ptr_array_t;
    const float *const Ab = p.a_ptrs != nullptr
                                ? ((ptr_array_t)p.a_ptrs)[entry]
                                : p.A + static_cast<long long>(entry) * p.a_bs;
    const float *const Bb = p.b_ptrs != nullptr
                                ? ((ptr_array_t)p.b_ptrs)[entry]
                                : p.B + static_cast<long long>(entry) * p.b_bs;
#pragma unroll
    for (int q = 0; q < NQ; q++) {
      const int rbl = wave + NW * q;
      const bool is_a = NW * q < RBA;
      const int row0 = is_a ? tm * BM + rbl * 16 : tn * BN + (rbl - RBA) * 16;
      const int last = is_a ? M - 1 : N - 1;
      const float *const base = is_a ? Ab : Bb;
      const long long rs = is_a ? p.a_rs : p.b_rs;
#pragma unroll
      for (int h = 0; h < 2; h++) {
        // 16-byte mode: row 8h + lane/8; 4-byte mode: row lane%16
        int r = row0 + (decltype(VEC)::value
                            ? 8 * h + static_cast<int>(lane >> 3)
                            : r16);
        r = r < last ? r : last;
        rowptr[q][h] = (gptr_t)(base + static_cast<long long>(r) * rs);
      }
    }
  };
  // VEC: std::true_type for 16-byte requests (both operands), else 4-byte ones
  auto issue = [&](auto VEC, const int ks, const int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < NQ; q++) {
      const int rbl = wave + NW * q;
      unsigned char *const dst =
          lds_raw + slot * Cfg::RAW_STAGE_BYTES + rbl * 2048;
      if constexpr (decltype(VEC)::value) {
        // K % 4 == 0 here: a piece is all in or all out
        const int piece =
            static_cast<int>((lane & 7u) ^ (2u * ((lane >> 4) & 3u)));
#pragma unroll
        for (int h = 0; h < 2; h++) {
          int k = ks * 32 + 4 * (piece ^ h);
          k = k < K ? k : 0;
          __builtin_amdgcn_global_load_lds(
              (const __attribute__((address_space(1))) void *)(rowptr[q][h] +
                                                                k),
              (__attribute__((address_space(3))) void *)(dst + h * 1024), 16, 0,
              0);
        }
      } else {
        const long long kst = NW * q < RBA ? p.a_ks : p.b_ks;
#pragma unroll
        for (int e = 0; e < 8; e++) {
          int k = ks * 32 + g8 + e;
          k = k < K ? k : K - 1;
          __builtin_amdgcn_global_load_lds(
              (const __attribute__((address_space(1))) void *)(rowptr[q][0] +
                                                                k * kst),
              (__attribute__((address_space(3))) void *)(dst + e * 256), 4, 0,
              0);
        }
      }
    }
  };
  // leave NRAW-1 stages of this wave's requests in flight
  auto wait_oldest_stage = [&](auto VEC) __attribute__((always_inline)) {
    constexpr int per_stage = NQ * (decltype(VEC)::value ? 2 : 8);
    wait_vmcnt_at_most<(NRAW - 1) * per_stage>();
  };
  // byte offset of this lane's eight floats inside a raw row block (16-byte mode)
  const int vec_off =
      r16 * 128 + 32 * static_cast<int>((lane >> 4) ^ ((lane >> 1) & 3u));
  const int vec_off_lo = vec_off + 16 * (r16 >> 3);
  const int vec_off_hi = vec_off + 16 * (1 - (r16 >> 3));
  // conversion, first half: this lane's eight floats of each of the wave's
  // row blocks, out of raw slot `slot`
  auto load_raw = [&](auto VEC, const int slot, float (&v)[NQ][8]) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < NQ; q++) {
      const int rbl = wave + NW * q;
      const unsigned char *const src =
          lds_raw + slot * Cfg::RAW_STAGE_BYTES + rbl * 2048;
      if constexpr (decltype(VEC)::value) {
        const f32x4 lo = *reinterpret_cast<const f32x4 *>(src + vec_off_lo);
        const f32x4 hi = *reinterpret_cast<const f32x4 *>(src + vec_off_hi);
#pragma unroll
        for (int x = 0; x < 4; x++) {
          v[q][x] = lo[x];
          v[q][4 + x] = hi[x];
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++)
          v[q][e] = reinterpret_cast<const float *>(src)[e * 64 + lane];
      }
    }
  };
  // conversion, second half: split and write the terms of k stage `ks` into
  // fragment buffer `buf`
  auto split_store = [&](const int ks, const int buf, float (&v)[NQ][8]) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < NQ; q++) {
      const int rbl = wave + NW * q;
      // k past K was clamped in the request: zero it (last stage only)
      if (ks * 32 + 32 > K) {
        const int left = K - (ks * 32 + g8);
#pragma unroll
        for (int x = 0; x < 8; x++)
          v[q][x] = x < left ? v[q][x] : 0.f;
      }
      // the split of split_traits<T>, four elements at a time in the form
      // that uses the packed conversions (and for fp16 the mixed-precision
      // fma): t0 = RN16(v), t1 = RN16((v - t0) * scale), t2 = RN16((v - t0) - t1)
      S term[3][8];
#pragma unroll
      for (int x = 0; x < 8; x += 4) {
        const mtk::wmma::tcec::detail::f32x4_t vv = {v[q][x], v[q][x + 1],
                                                     v[q][x + 2], v[q][x + 3]};
        mtk::wmma::tcec::detail::split4<T>(vv, &term[0][x], &term[1][x],
                                           &term[2][x]);
      }
      ab_vec t[3];
#pragma unroll
      for (int c = 0; c < TERMS; c++)
#pragma unroll
        for (int x = 0; x < 8; x++)
          t[c][x] = term[c][x];
#pragma unroll
      for (int c = 0; c < TERMS; c++)
        frag[((buf * NRB + rbl) * TERMS + c) * 64 + lane] =
            __builtin_bit_cast(u32x4, t[c]);
    }
  };
  auto mfma = [](const ab_vec x, const ab_vec y, const f32x4 z) -> f32x4 {
    if constexpr (std::is_same<S, _Float16>::value)
      return __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y, z, 0, 0, 0);
    else
      return __builtin_amdgcn_mfma_f32_16x16x32_bf16(x, y, z, 0, 0, 0);
  };

  f32x4 acc_main[MT_][NT_], acc_err[MT_][NT_];
  auto clear_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < MT_; i++)
#pragma unroll
      for (int j = 0; j < NT_; j++) {
        acc_main[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
        acc_err[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
  };
  auto store_tile = [&](const int i_tile) __attribute__((always_inline)) {
    int entry, tm, tn;
    decode(i_tile, entry, tm, tn);
    typedef float *const __attribute__((address_space(4))) *out_array_t;
    float *const Cb = p.c_ptrs != nullptr
                          ? ((out_array_t)p.c_ptrs)[entry]
                          : p.C + static_cast<long long>(entry) * p.c_bs;
    const int vec_out =
        p.vec_store && (reinterpret_cast<uintptr_t>(Cb) & 15u) == 0;
    const float alpha = p.alpha, beta = p.beta;
    const int row_base = tm * BM + wm * WM + 4 * static_cast<int>(lane >> 4);
    const int col_base = tn * BN + wn * WN + r16;
    const auto out_value = [&](const int i, const int j) {
      f32x4 o = acc_main[i][j];
      if constexpr (TERMS >= 2)
        o = epilogue_fold(o, acc_err[i][j], p.inv_scale);
      return o * alpha;
    };
    // one 16x16 tile: a lane stores rows 4q .. 4q+3 of its column, 16 bytes
    const auto store_one = [&](const int i, const int j) {
      const int col = col_base + 16 * j;
      const int row = row_base + 16 * i;
      if (col >= N || row >= M)
        return;
      f32x4 o = out_value(i, j);
      float *const dst = Cb + row + static_cast<long long>(col) * p.ldc;
      if (vec_out && row + 3 < M) {
        if (beta != 0.f)
          o = epilogue_beta(o, beta, *reinterpret_cast<const f32x4 *>(dst));
        *reinterpret_cast<f32x4 *>(dst) = o;
      } else {
#pragma unroll
        for (int x = 0; x < 4; x++) {
          if (row + x < M) {
            float e = o[x];
            if (beta != 0.f)
              e = epilogue_beta(e, beta, dst[x]);
            dst[x] = e;
          }
        }
      }
    };
    // two tiles of one tile column, all inside C: whole 128-byte lines per
    // store instruction after a swap between the lanes of neighbouring columns
    // (tcec_gemm_kernel's store_tile_pair)
    const int odd = static_cast<int>(lane & 1u);
    const auto store_pair = [&](const int i, const int j) {
      const f32x4 v0 = out_value(i, j), v1 = out_value(i + 1, j);
      f32x4 d1, d2;
#pragma unroll
      for (int x = 0; x < 4; x++) {
        const float n0 = neighbour_lane(v0[x]), n1 = neighbour_lane(v1[x]);
        d1[x] = odd ? n1 : v0[x];
        d2[x] = odd ? v1[x] : n0;
      }
      const int row = row_base + 16 * (i + odd);
      const int col = col_base + 16 * j;
      float *const dst1 = Cb + row + static_cast<long long>(col & ~1) * p.ldc;
      float *const dst2 = Cb + row + static_cast<long long>(col | 1) * p.ldc;
      if (beta != 0.f) {
        d1 = epilogue_beta(d1, beta, *reinterpret_cast<const f32x4 *>(dst1));
        d2 = epilogue_beta(d2, beta, *reinterpret_cast<const f32x4 *>(dst2));
      }
      *reinterpret_cast<f32x4 *>(dst1) = d1;
      *reinterpret_cast<f32x4 *>(dst2) = d2;
    };
    const int blk_row0 = tm * BM + wm * WM, blk_col0 = tn * BN + wn * WN;
#pragma unroll
    for (int j = 0; j < NT_; j++) {
      const bool cols_inside = blk_col0 + 16 * j + 16 <= N;
      if constexpr (MT_ % 2 == 0) {
#pragma unroll
        for (int i = 0; i < MT_; i += 2) {
          // (wave-uniform: both lanes of a swap take the same branch)
          if (vec_out && cols_inside && blk_row0 + 16 * i + 32 <= M) {
            store_pair(i, j);
          } else {
            store_one(i, j);
            store_one(i + 1, j);
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < MT_; i++)
          store_one(i, j);
      }
    }
  };

  // Pipeline, per wave and stream stage s (one iteration of the k loop):
  //   request stage s+1+NRAW into the raw slot that stage s+1 has left
  //   wait until the wave's requests of stage s+2 have landed, read them
  //   issue the MFMAs of stage s (fragments are in registers)
  //   read the fragments of stage s+1 (converted last iteration) into the
  //     same registers - the matrix core has fetched them by then
  //   split stage s+2 and write its terms over the fragment buffer of stage s
  //   barrier
  // so the LDS latencies sit behind the MFMAs and the conversion arithmetic,
  // and NRAW stages of requests are in flight while the wave computes.
  auto run = [&](auto VEC) __attribute__((always_inline)) {
    int req_tile = 0, req_ks = 0; // next (tile, k stage) to request
    auto advance_request = [&]() __attribute__((always_inline)) {
      if (req_ks + 1 < num_k) {
        req_ks++;
      } else if (req_tile + 1 < n_my) {
        req_tile++;
        req_ks = 0;
        set_rows(VEC, req_tile);
      } // else: stay on the last stage; the redundant requests land in free
        // slots and keep the in-flight count constant
    };
    int conv_ks = 0; // k stage of the stream stage converted next
    auto advance_conv = [&]() __attribute__((always_inline)) {
      conv_ks = conv_ks + 1 == num_k ? 0 : conv_ks + 1;
    };
    ab_vec a[TERMS][MT_], b[TERMS][NT_];
    auto read_frags = [&](const int buf) __attribute__((always_inline)) {
      const u32x4 *const sa =
          frag + ((buf * NRB + wm * MT_) * TERMS) * 64 + lane;
      const u32x4 *const sb =
          frag + ((buf * NRB + RBA + wn * NT_) * TERMS) * 64 + lane;
#pragma unroll
      for (int j = 0; j < NT_; j++)
#pragma unroll
        for (int t = 0; t < TERMS; t++)
          b[t][j] = __builtin_bit_cast(ab_vec, sb[(j * TERMS + t) * 64]);
#pragma unroll
      for (int i = 0; i < MT_; i++)
#pragma unroll
        for (int t = 0; t < TERMS; t++)
          a[t][i] = __builtin_bit_cast(ab_vec, sa[(i * TERMS + t) * 64]);
    };
    float v[NQ][8];

    // ---- prologue: fill the raw ring, convert stages 0 and 1, load stage 0
    set_rows(VEC, 0);
    for (int s = 0; s < NRAW; s++) {
      issue(VEC, req_ks, s);
      advance_request();
    }
    wait_oldest_stage(VEC); // stage 0
    load_raw(VEC, 0, v);
    split_store(conv_ks, 0, v);
    advance_conv();
    issue(VEC, req_ks, 0); // stage NRAW into the slot stage 0 has left
    advance_request();
    wait_oldest_stage(VEC); // stage 1
    load_raw(VEC, 1 % NRAW, v);
    split_store(conv_ks, 1, v);
    advance_conv();
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    read_frags(0);
    // every wave has stage 0 in registers before anybody overwrites its buffer
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

    // The k loop of a tile is a loop of its own so that the accumulators are
    // touched by nothing but MFMAs inside it (they stay in AGPRs); the stream
    // of requests and conversions runs on across the tile boundary.
    int slot_conv = 2 % NRAW; // raw slot of stage s+2
    int s = 0;                // stream index of the stage being multiplied
    for (int cur_tile = 0; cur_tile < n_my; cur_tile++) {
      clear_acc();
      for (int cur_ks = 0; cur_ks < num_k; cur_ks++, s++) {
        const int buf = s & 1;
        // refill the slot that stage s+1 has left (it was converted last
        // iteration): it is the one before slot_conv
        issue(VEC, req_ks, slot_conv == 0 ? NRAW - 1 : slot_conv - 1);
        advance_request();
        wait_oldest_stage(VEC); // stage s+2 (past the end: a redundant tail stage)
        load_raw(VEC, slot_conv, v);

        auto sweep = [&](f32x4(&acc)[MT_][NT_], const int ta, const int tb) __attribute__((always_inline)) {
#pragma unroll
          for (int i = 0; i < MT_; i++)
#pragma unroll
            for (int j = 0; j < NT_; j++)
              acc[i][j] = mfma(a[ta][i], b[tb][j], acc[i][j]);
        };
        auto multiply = [&]() __attribute__((always_inline)) {
          // same products and, per accumulator, the same order as
          // tcec_gemm_kernel.  (That kernel's tile-major issue order, a
          // tile's products back to back, was measured here too: this kernel
          // is not limited by the matrix core's power and ran 7 % slower.)
          if constexpr (TERMS >= 3) {
            sweep(acc_err, 2, 0);
            sweep(acc_err, 0, 2);
            sweep(acc_err, 1, 1);
          }
          if constexpr (TERMS >= 2) {
            sweep(acc_err, 1, 0);
            sweep(acc_err, 0, 1);
          }
          if (p.rn_main) {
#pragma unroll
            for (int i = 0; i < MT_; i++)
#pragma unroll
              for (int j = 0; j < NT_; j++)
                acc_main[i][j] +=
                    mfma(a[0][i], b[0][j], f32x4{0.f, 0.f, 0.f, 0.f});
          } else {
            sweep(acc_main, 0, 0);
          }
          // stage s+1 into the registers the MFMAs above have been fed from
          read_frags(buf ^ 1);
        };
        // The two waves that share a SIMD run the matrix phase and the
        // conversion phase in opposite order, so that one wave's MFMAs overlap
        // the other's vector arithmetic instead of colliding with its MFMAs.
        const bool matrix_first = NW < 8 || wave < NW / 2;
        if (matrix_first)
          multiply();
        // stage s+2 over the buffer of stage s, which every wave took into
        // registers before the last barrier
        split_store(conv_ks, buf, v);
        if (!matrix_first)
          multiply();
        advance_conv();
        slot_conv = slot_conv + 1 == NRAW ? 0 : slot_conv + 1;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      }
      store_tile(cur_tile);
    }
  };
  if (vec_a && vec_b)
    run(std::true_type{});
  else
    run(std::false_type{});
  // the redundant tail requests still write LDS: drain them before the end
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
}

} // namespace wmmae_gemm
