// One-wave and tile-stream kernels that exercise the public device API the
// way the reference's own test programs do.  They are compiled into the C-ABI
// library so that host tests can drive the header-only API without a
// compiler on the test machine.
//
//   primitive_tiles_kernel  : foreach / foreach_ij / load_vector / store_vector
//                             over a stream of 16x16 tiles
//                             (reference: test/primitive/foreach_ij.cu:20-92,
//                             wmma.load_vector.cu:44-72, wmma.store_vector.cu:36-42)
//   layout_dump_kernel      : integer tables of foreach_ij / foreach / foreach_v / map
//                             (reference: test/primitive/map.cu:11-58)
//   tcec_mma_tile_kernel    : one-wave D = A*B (+C) through tcec::load_matrix_sync /
//                             mma_sync / store_matrix_sync
//                             (reference: test/tcec/mma.cu:23-100)
//   tcec_matvec_kernel      : y = A*x through tcec::load_vector / store_vector
//                             (reference: test/tcec/matvec.cu:21-50)
//   tcec_elementwise_kernel : x(i) / dx(i) accessors, fill_fragment, neg, integrate
//                             (reference: test/tcec/elementwise.cu:7-26)
//   tcec_frag_dump_kernel   : split terms held by an operand fragment after
//                             load_matrix_sync or load_vector
//                             (reference: test/tcec/vector.cu:15-61)
//   tcec_api_gemm_kernel    : a tiled GEMM written against the public tcec:: API only
//                             (reference: test/tcec/batch_gemm.cu:196-386)
//   mfma_probe_kernel       : one raw MFMA on caller-supplied bit patterns
//   mfma_source_hazard_kernel: a vector-ALU write of an MFMA source register
//                             directly in front of a hand-placed MFMA
//   tcec_mma_complex_kernel : one-wave complex D = A*B (+C) through fragment_complex
//                             (reference: test/tcec/mma_complex.cu:22-101)
//   primitive_mma_kernel    : mma::load_matrix_sync -> mma_sync -> mma::store_matrix_sync
//   wrapper_mma_kernel      : the same through the tcec::detail function objects
//                             (reference: test/primitive/mma.cu:11-45)
//   foreach_ec_kernel       : A, dA, B, dB built through foreach, three MMAs
//                             (reference: test/primitive/foreach.cu:24-80)
//   gevm_kernel             : identity times a load_vector fragment, store_vector
//                             (reference: test/primitive/gevm.cu:22-43)
//   fragment_ops_kernel     : operators +, -, *, /, fma on fragments
//                             (reference: test/primitive/operators.cu:14-57)
//   fragment_eye_kernel     : add_eye / make_identity_matrix
//                             (reference: test/primitive/add_eye.cu:24-30)
//   direct_product_kernel   : make_direct_product_fragment(_c3) + one MMA
//                             (reference: test/primitive/direct_product.cu:44-99)
//   clock_samples_kernel    : (constant-rate clock, shader clock) pairs over time
//   cp_async_kernel         : utils::cp_async global -> LDS copies
//                             (reference: test/utils/cp_async.cu:15-25)
//   cp_async_pipeline_kernel: the same calls as a three-stage pipeline
//                             (commit / wait_group<2>, reference utils.hpp:29-64)
//   cast_kernel             : utils::cast (reference: test/utils/cast.cu)
//   print_fragment_kernel   : print_fragment of a primitive and a TCEC fragment
//                             (reference: test/primitive/print_fragment.cu)
#pragma once
#include <wmma_extension/operators.hpp>
#include <wmma_extension/tcec/complex.hpp>
#include <wmma_extension/tcec/tcec.hpp>
#include <wmma_extension/utils.hpp>
#include <wmma_extension/wmma_mma.hpp>

namespace wmmae_harness {
namespace w = mtk::wmma;
namespace tcec = mtk::wmma::tcec;

// --------------------------------------------------------------------------
// Fragment primitives over a stream of tiles.  One wave per tile, grid-stride,
// four waves per block.  Per tile (256 fp32 in):
//   a_row/a_col/b_row/b_col : (lane,reg) dump of a 16x16x16 half fragment filled
//                             through foreach_ij from the tile read in that layout
//   acc_out                 : tile read as a row-major accumulator through
//                             foreach(mem_row_major), written with
//                             store_matrix_sync(mem_col_major)  (a transpose)
//   vec_out[0]              : tile[0..15] -> load_vector(acc, col) -> store_vector(col)
//   vec_out[1]              : tile[16..31] -> load_vector(acc, row) -> store_vector(row)
// --------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
    primitive_tiles_kernel(const float *__restrict__ tiles,
                           const long long num_tiles,
                           w::half *__restrict__ a_row,
                           w::half *__restrict__ a_col,
                           w::half *__restrict__ b_row,
                           w::half *__restrict__ b_col,
                           float *__restrict__ acc_out,
                           float *__restrict__ vec_out) {
  const unsigned lane = w::detail::common::get_lane_id();
  const long long wave = (static_cast<long long>(blockIdx.x) * blockDim.x +
                          threadIdx.x) /
                         w::wave_size;
  const long long num_waves =
      static_cast<long long>(gridDim.x) * blockDim.x / w::wave_size;
  using FA_R = w::fragment<w::matrix_a, 16, 16, 16, w::half, w::row_major>;
  using FA_C = w::fragment<w::matrix_a, 16, 16, 16, w::half, w::col_major>;
  using FB_R = w::fragment<w::matrix_b, 16, 16, 16, w::half, w::row_major>;
  using FB_C = w::fragment<w::matrix_b, 16, 16, 16, w::half, w::col_major>;
  using FC = w::fragment<w::accumulator, 16, 16, 16, float>;

  // The tile is read from HBM once, 16 bytes per lane, into the wave's own
  // 1 KiB of LDS; the primitives below then gather from LDS (where a user of
  // the API keeps the tile it builds fragments from).  A wave's LDS accesses
  // execute in program order, so no barrier is needed between the copy and
  // the gathers, nor before the next tile overwrites the buffer.
  __shared__ __attribute__((aligned(16))) float staged[4][256];
  float *const tile = staged[threadIdx.x / w::wave_size];
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
  for (long long t = wave; t < num_tiles; t += num_waves) {
    // a lane's four halfs of a fragment as one 8-byte store that is not kept
    // in the caches: the dumps are written once and never read by this kernel
    // (measured: 5.78 -> 6.0 TB/s over the whole kernel)
    auto dump = [&](w::half *const out, const auto &f) {
      static_assert(sizeof(f.x) == 8, "four halfs per lane");
      u32x2 bits;
      __builtin_memcpy(&bits, f.x, 8);
      __builtin_nontemporal_store(
          bits, reinterpret_cast<u32x2 *>(out + (t * 64 + lane) * 4));
    };
    *reinterpret_cast<f32x4 *>(tile + 4 * lane) =
        *reinterpret_cast<const f32x4 *>(tiles + t * 256 + 4 * lane);
    {
      FA_R f;
      w::foreach_ij<FA_R>([&](const unsigned *list, const unsigned count,
                              const unsigned i, const unsigned j) {
        for (unsigned c = 0; c < count; c++)
          f.x[list[c]] = w::detail::common::cast<w::half>(tile[i * 16 + j]);
      });
      dump(a_row, f);
    }
    {
      FA_C f;
      w::foreach_ij<FA_C>([&](const unsigned *list, const unsigned count,
                              const unsigned i, const unsigned j) {
        for (unsigned c = 0; c < count; c++)
          f.x[list[c]] = w::detail::common::cast<w::half>(tile[i + j * 16]);
      });
      dump(a_col, f);
    }
    {
      FB_R f;
      w::foreach_ij<FB_R>([&](const unsigned *list, const unsigned count,
                              const unsigned i, const unsigned j) {
        for (unsigned c = 0; c < count; c++)
          f.x[list[c]] = w::detail::common::cast<w::half>(tile[i * 16 + j]);
      });
      dump(b_row, f);
    }
    {
      FB_C f;
      w::foreach_ij<FB_C>([&](const unsigned *list, const unsigned count,
                              const unsigned i, const unsigned j) {
        for (unsigned c = 0; c < count; c++)
          f.x[list[c]] = w::detail::common::cast<w::half>(tile[i + j * 16]);
      });
      dump(b_col, f);
    }
    {
      FC f;
      w::foreach<FC>(w::mem_row_major,
                     [&](const unsigned *list, const unsigned count,
                         const unsigned mem_index) {
                       for (unsigned c = 0; c < count; c++)
                         f.x[list[c]] = tile[mem_index];
                     });
      w::store_matrix_sync(acc_out + t * 256, f, 16, w::mem_col_major);
    }
    {
      FC f;
      w::load_vector(f, tile, w::mem_col_major);
      w::store_vector(vec_out + t * 32, f, w::mem_col_major);
      w::load_vector(f, tile + 16, w::mem_row_major);
      w::store_vector(vec_out + t * 32 + 16, f, w::mem_row_major);
    }
  }
}

// --------------------------------------------------------------------------
// Integer layout tables of one fragment type, one wave.
//   ij[(lane*R + reg)*2 + {0,1}]      = (i, j) from foreach_ij
//   mem_index[lane*R + reg]           = mem_index from foreach
//   v_index[lane*R + reg]             = mem_index from foreach_v, or -1 if the
//                                       register is not visited
//   map_tid/map_fid[i*cols + j]       = map(i, j)
// R = num_elements.  col selects col_major / mem_col_major.
// --------------------------------------------------------------------------
template <class Frag>
__global__ void __launch_bounds__(64)
    layout_dump_kernel(const int col, int *__restrict__ ij,
                       int *__restrict__ mem_index, int *__restrict__ v_index,
                       int *__restrict__ map_tid, int *__restrict__ map_fid) {
  constexpr bool is_acc = std::is_same<typename Frag::use, w::accumulator>::value;
  constexpr unsigned R = Frag::num_elements;
  const unsigned lane = w::detail::common::get_lane_id();
  for (unsigned x = 0; x < R; x++)
    v_index[lane * R + x] = -1;
  w::foreach_ij<Frag>([&](const unsigned *list, const unsigned count,
                          const unsigned i, const unsigned j) {
    for (unsigned c = 0; c < count; c++) {
      ij[(lane * R + list[c]) * 2 + 0] = i;
      ij[(lane * R + list[c]) * 2 + 1] = j;
    }
  });
  auto put_mem = [&](const unsigned *list, const unsigned count,
                     const unsigned idx) {
    for (unsigned c = 0; c < count; c++)
      mem_index[lane * R + list[c]] = idx;
  };
  auto put_v = [&](const unsigned *list, const unsigned count,
                   const unsigned idx) {
    for (unsigned c = 0; c < count; c++)
      v_index[lane * R + list[c]] = idx;
  };
  if constexpr (is_acc) {
    const w::layout_t l = col ? w::mem_col_major : w::mem_row_major;
    w::foreach<Frag>(l, put_mem);
    w::foreach_v<Frag>(l, put_v);
  } else {
    w::foreach<Frag>(put_mem);
    w::foreach_v<Frag>(put_v);
  }
  using L = typename Frag::layout_model;
  for (unsigned e = lane; e < L::rows * L::cols; e += w::wave_size) {
    unsigned tid[2], fid[2], n;
    w::map<Frag>(tid, fid, n, e / L::cols, e % L::cols);
    map_tid[e] = n == 1 ? int(tid[0]) : -1;
    map_fid[e] = n == 1 ? int(fid[0]) : -1;
  }
}

// --------------------------------------------------------------------------
// One-wave TCEC matrix product, m x n x k in one tcec::fragment each.
// A is m x k, B is k x n, C/D are m x n; memory layouts are run-time flags
// (1 = column major) and the leading dimensions are the dense ones.
// rounding: 0 = mma_sync (policy default), 1 = mma_rn_sync, 2 = mma_rz_sync.
// --------------------------------------------------------------------------
template <int m, int n, int k, class T, class Policy, class AL, class BL>
__global__ void __launch_bounds__(64)
    tcec_mma_tile_kernel(float *const d, const float *const a,
                         const float *const b, const float *const c,
                         const int a_col, const int b_col, const int c_col,
                         const int d_col, const int rounding) {
  tcec::fragment<w::matrix_a, m, n, k, T, AL, Policy> fa;
  tcec::fragment<w::matrix_b, m, n, k, T, BL, Policy> fb;
  tcec::fragment<w::accumulator, m, n, k, T, void, Policy> fc, fd;

  if (a_col)
    tcec::load_matrix_sync<w::col_major>(fa, a, m);
  else
    tcec::load_matrix_sync<w::row_major>(fa, a, k);
  if (b_col)
    tcec::load_matrix_sync<w::col_major>(fb, b, k);
  else
    tcec::load_matrix_sync<w::row_major>(fb, b, n);

  if (c != nullptr) {
    tcec::load_matrix_sync(fc, c, c_col ? m : n,
                           c_col ? w::mem_col_major : w::mem_row_major);
    if (rounding == 1)
      tcec::mma_rn_sync(fd, fa, fb, fc);
    else if (rounding == 2)
      tcec::mma_rz_sync(fd, fa, fb, fc);
    else
      tcec::mma_sync(fd, fa, fb, fc);
  } else {
    if (rounding == 1)
      tcec::mma_rn_sync(fd, fa, fb);
    else if (rounding == 2)
      tcec::mma_rz_sync(fd, fa, fb);
    else
      tcec::mma_sync(fd, fa, fb);
  }
  tcec::store_matrix_sync(d, fd, d_col ? m : n,
                          d_col ? w::mem_col_major : w::mem_row_major);
}

// Same product with the operand memory layout taken from the fragment Layout
// (the load_matrix_sync overload without a MatrixLayout argument).
template <int m, int n, int k, class T, class Policy, class AL, class BL>
__global__ void __launch_bounds__(64)
    tcec_mma_tile_native_kernel(float *const d, const float *const a,
                                const float *const b, const int d_col) {
  tcec::fragment<w::matrix_a, m, n, k, T, AL, Policy> fa;
  tcec::fragment<w::matrix_b, m, n, k, T, BL, Policy> fb;
  tcec::fragment<w::accumulator, m, n, k, T, void, Policy> fd;
  tcec::load_matrix_sync(fa, a, std::is_same<AL, w::col_major>::value ? m : k);
  tcec::load_matrix_sync(fb, b, std::is_same<BL, w::col_major>::value ? k : n);
  tcec::mma_sync(fd, fa, fb);
  tcec::store_matrix_sync(d, fd, d_col ? m : n,
                          d_col ? w::mem_col_major : w::mem_row_major);
}

// --------------------------------------------------------------------------
// y = A * x with x loaded by tcec::load_vector into the first column of a
// matrix_b fragment and y read back with tcec::store_vector (col), or
// y^T = x^T * A with x in the first row of a matrix_a fragment (row).
// A is N x N; a_col gives its memory layout.
// --------------------------------------------------------------------------
template <int N, class T, class Policy>
__global__ void __launch_bounds__(64)
    tcec_matvec_kernel(float *const y, const float *const a,
                       const float *const x, const int a_col,
                       const int left_vector) {
  tcec::fragment<w::accumulator, N, N, N, T, void, Policy> fc;
  tcec::fill_zero(fc);
  if (!left_vector) {
    tcec::fragment<w::matrix_a, N, N, N, T, w::row_major, Policy> fa;
    tcec::fragment<w::matrix_b, N, N, N, T, w::col_major, Policy> fx;
    tcec::fill_zero(fx);
    if (a_col)
      tcec::load_matrix_sync<w::col_major>(fa, a, N);
    else
      tcec::load_matrix_sync<w::row_major>(fa, a, N);
    tcec::load_vector(fx, x);
    tcec::mma_sync(fc, fa, fx, fc);
    tcec::store_vector(y, fc, w::mem_col_major);
  } else {
    tcec::fragment<w::matrix_a, N, N, N, T, w::row_major, Policy> fx;
    tcec::fragment<w::matrix_b, N, N, N, T, w::col_major, Policy> fa;
    tcec::fill_zero(fx);
    if (a_col)
      tcec::load_matrix_sync<w::col_major>(fa, a, N);
    else
      tcec::load_matrix_sync<w::row_major>(fa, a, N);
    tcec::load_vector(fx, x);
    tcec::mma_sync(fc, fx, fa, fc);
    tcec::store_vector(y, fc, w::mem_row_major);
  }
}

// --------------------------------------------------------------------------
// Raw split terms of an operand fragment.  src is a dense N x N fp32 matrix
// (or an N vector when from_vector != 0).  Output, 16-bit patterns:
//   terms[(term*num_elements + e)*64 + lane],  e = flat element index x(e)
// --------------------------------------------------------------------------
template <class Use, int N, class T, class Policy, class Layout>
__global__ void __launch_bounds__(64)
    tcec_frag_dump_kernel(unsigned short *const terms, const float *const src,
                          const int from_vector, const int mem_col) {
  using F = tcec::fragment<Use, N, N, N, T, Layout, Policy>;
  F f;
  tcec::fill_zero(f);
  if (from_vector) {
    tcec::load_vector(f, src);
  } else if (mem_col == 2) {
    // the swizzled staging tile: src (rows of matrix_a / columns of matrix_b,
    // N = 32 k each) is copied into LDS the way a GEMM stages it - lane l of a
    // pass writes physical piece l % 8 of line l / 8 and fetches the logical
    // piece that belongs there - and loaded with the swizzled layout tag
    static_assert(N == 32, "lines of 32 k");
    __shared__ __attribute__((aligned(16))) float tile[N * N];
    const unsigned t = threadIdx.x;
    namespace cpa = w::utils::cp_async;
    for (unsigned l0 = 0; l0 < unsigned(N); l0 += 8) {
      const unsigned line = l0 + t / 8;
      const unsigned piece = (t % 8) ^ tcec::swizzled_piece(line);
      cpa::cp_async<16>(tile + 4 * (8 * l0 + t), src + line * N + 4 * piece);
    }
    cpa::commit();
    cpa::wait_all();
    if constexpr (std::is_same<Use, w::matrix_a>::value)
      tcec::load_matrix_sync<tcec::row_major_swizzled>(f, tile, N);
    else
      tcec::load_matrix_sync<tcec::col_major_swizzled>(f, tile, N);
  } else {
    if (mem_col)
      tcec::load_matrix_sync<w::col_major>(f, src, N);
    else
      tcec::load_matrix_sync<w::row_major>(f, src, N);
  }
  const unsigned lane = w::detail::common::get_lane_id();
  for (unsigned e = 0; e < F::num_elements; e++) {
    const unsigned b = e / F::sub_frag_t::num_elements;
    const unsigned r = e % F::sub_frag_t::num_elements;
    terms[(0 * F::num_elements + e) * 64 + lane] =
        __builtin_bit_cast(unsigned short, f.sub_frag[b].x[r]);
    if constexpr (F::num_terms >= 2)
      terms[(1 * F::num_elements + e) * 64 + lane] =
          __builtin_bit_cast(unsigned short, f.sub_d_frag[b].x[r]);
    if constexpr (F::num_terms >= 3)
      terms[(2 * F::num_elements + e) * 64 + lane] =
          __builtin_bit_cast(unsigned short, f.sub_d2_frag[b].x[r]);
  }
}

// --------------------------------------------------------------------------
// Element access on a TCEC accumulator (N = 32): fill_fragment(base), then
// x(i) = lane*100 + i as in the reference's test, dx(i) = i (with_ec only),
// optional neg(), optional integrate(), then store column-major.
// out[0 .. N*N) receives the stored matrix; out[N*N + lane] the value of
// x(0) + x(num_elements-1) read back through the const accessors after the
// edits (before neg / integrate).
// (reference: test/tcec/elementwise.cu:7-26; tcec.hpp:40-98 accessors, neg,
// integrate; test/primitive/fill.cu)
// --------------------------------------------------------------------------
template <int N, class T, class Policy>
__global__ void __launch_bounds__(64)
    tcec_elementwise_kernel(float *const out, const float base,
                            const int do_neg, const int do_integrate) {
  using F = tcec::fragment<w::accumulator, N, N, N, T, void, Policy>;
  F frag;
  tcec::fill_fragment(frag, base);
  const unsigned lane = w::detail::common::get_lane_id();
  for (unsigned i = 0; i < F::num_elements; i++) {
    frag.x(i) += static_cast<float>(lane * 100 + i);
    if constexpr (F::num_terms >= 2)
      frag.dx(i) = static_cast<float>(i);
  }
  const F &cref = frag;
  out[N * N + lane] = cref.x(0) + cref.x(F::num_elements - 1);
  if (do_neg)
    frag = tcec::neg(frag);
  if (do_integrate)
    frag.integrate();
  tcec::store_matrix_sync(out, frag, N, w::mem_col_major);
}

// --------------------------------------------------------------------------
// One MFMA on caller-supplied bit patterns: D = A*B + C.
// a: M x K row-major 16-bit patterns, b: K x N row-major, c/d: M x N row-major fp32.
// Used to measure the matrix core's accumulate rounding and subnormal handling
// and to check the layout model against silicon.
// --------------------------------------------------------------------------
template <class T, int M, int N, int K>
__global__ void __launch_bounds__(64)
    mfma_probe_kernel(float *const d, const unsigned short *const a,
                      const unsigned short *const b, const float *const c) {
  using S = typename w::detail::common::storage_t<T>::type;
  w::fragment<w::matrix_a, M, N, K, T, w::row_major> fa;
  w::fragment<w::matrix_b, M, N, K, T, w::row_major> fb;
  w::fragment<w::accumulator, M, N, K, float> fc;
  w::foreach_ij<decltype(fa)>([&](const unsigned *list, const unsigned,
                                  const unsigned i, const unsigned j) {
    fa.x[list[0]] = __builtin_bit_cast(S, a[i * K + j]);
  });
  w::foreach_ij<decltype(fb)>([&](const unsigned *list, const unsigned,
                                  const unsigned i, const unsigned j) {
    fb.x[list[0]] = __builtin_bit_cast(S, b[i * N + j]);
  });
  w::load_matrix_sync(fc, c, N, w::mem_row_major);
  w::mma_sync(fc, fa, fb, fc);
  w::store_matrix_sync(d, fc, N, w::mem_row_major);
}

// --------------------------------------------------------------------------
// Probe of a pipeline hazard the compiler does not see when an MFMA is issued
// from inline asm: one wave multiplies a 16x32 tile of ones by a 32x16 tile of
// ones (bf16), after overwriting the last register of the A operand (two of a
// lane's eight k) with twos by a vector-ALU instruction placed PRODUCER and GAP
// wait states in front of the MFMA, all inside one asm statement.  Every
// element of D is 40 when the matrix core saw the new register contents and 32
// when it saw the old ones.  PRODUCER 0: v_mov_b32, 1: v_accvgpr_read_b32 (what
// a reload from an AGPR spill copy is); GAP 0: nothing in between, 1: s_nop 0,
// 2: s_nop 1, 3: one unrelated v_mov_b32.
// --------------------------------------------------------------------------
template <int PRODUCER, int GAP>
__global__ void __launch_bounds__(64)
    mfma_source_hazard_kernel(float *const d) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  const unsigned one = 0x3F803F80u, two = 0x40004000u; // bf16 pairs
  const u32x4 b = {one, one, one, one};
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#define WMMAE_HAZARD_ASM(PRODUCER_TEXT, GAP_TEXT)                              \
  asm volatile("v_mov_b32 v100, %2\n\tv_mov_b32 v101, %2\n\t"                  \
               "v_mov_b32 v102, %2\n\tv_mov_b32 v103, %2\n\t"                  \
               "v_accvgpr_write_b32 a200, %3\n\t"                              \
               "s_nop 7\n\ts_nop 7\n\t" PRODUCER_TEXT "\n\t" GAP_TEXT          \
               "v_mfma_f32_16x16x32_bf16 %0, v[100:103], %1, %0\n\t"           \
               "s_nop 15\n\ts_nop 15"                                          \
               : "+a"(acc)                                                     \
               : "v"(b), "v"(one), "v"(two)                                    \
               : "v100", "v101", "v102", "v103", "v104", "a200")
#define WMMAE_HAZARD_GAP(PRODUCER_TEXT)                                        \
  if constexpr (GAP == 0)                                                      \
    WMMAE_HAZARD_ASM(PRODUCER_TEXT, "");                                       \
  else if constexpr (GAP == 1)                                                 \
    WMMAE_HAZARD_ASM(PRODUCER_TEXT, "s_nop 0\n\t");                            \
  else if constexpr (GAP == 2)                                                 \
    WMMAE_HAZARD_ASM(PRODUCER_TEXT, "s_nop 1\n\t");                            \
  else                                                                         \
    WMMAE_HAZARD_ASM(PRODUCER_TEXT, "v_mov_b32 v104, %2\n\t")
  if constexpr (PRODUCER == 0) {
    WMMAE_HAZARD_GAP("v_mov_b32 v103, %3");
  } else {
    WMMAE_HAZARD_GAP("v_accvgpr_read_b32 v103, a200");
  }
#undef WMMAE_HAZARD_GAP
#undef WMMAE_HAZARD_ASM
  reinterpret_cast<f32x4 *>(d)[threadIdx.x] = acc;
}

// --------------------------------------------------------------------------
// One-wave complex product D = A*B (+C), N x N x N, every operand in one
// tcec::fragment_complex; memory holds interleaved (re, im) pairs with dense
// leading dimension N.  mul != 1 exercises the scaled load of A and the scaled
// store (D = (mul*A)*B*(1/mul) + ..., exact for powers of two).
// --------------------------------------------------------------------------
template <int N, class T, class Policy, class AL, class BL>
__global__ void __launch_bounds__(64)
    tcec_mma_complex_kernel(tcec::complex_t *const d,
                            const tcec::complex_t *const a,
                            const tcec::complex_t *const b,
                            const tcec::complex_t *const c, const int a_col,
                            const int b_col, const int c_col, const int d_col,
                            const int rounding, const float mul) {
  tcec::fragment_complex<w::matrix_a, N, N, N, T, AL, Policy> fa;
  tcec::fragment_complex<w::matrix_b, N, N, N, T, BL, Policy> fb;
  tcec::fragment_complex<w::accumulator, N, N, N, T, void, Policy> fc, fd;
  if (a_col)
    tcec::load_matrix_sync_with_mul<w::col_major>(fa, a, N, mul);
  else
    tcec::load_matrix_sync_with_mul<w::row_major>(fa, a, N, mul);
  if (b_col)
    tcec::load_matrix_sync<w::col_major>(fb, b, N);
  else
    tcec::load_matrix_sync<w::row_major>(fb, b, N);
  tcec::fill_fragment(fd, 0.0f);
  if (c != nullptr) {
    tcec::load_matrix_sync(fc, c, N, c_col ? w::mem_col_major : w::mem_row_major);
    if (mul != 1.f) { // keep D = A*B + C after the scaled store
      for (unsigned i = 0; i < fc.real.num_elements; i++) {
        fc.real.x(i) *= mul;
        fc.imag.x(i) *= mul;
      }
    }
    if (rounding == 1)
      tcec::mma_rn_sync(fd, fa, fb, fc);
    else if (rounding == 2)
      tcec::mma_rz_sync(fd, fa, fb, fc);
    else
      tcec::mma_sync(fd, fa, fb, fc);
  } else {
    if (rounding == 1)
      tcec::mma_rn_sync(fd, fa, fb);
    else if (rounding == 2)
      tcec::mma_rz_sync(fd, fa, fb);
    else
      tcec::mma_sync(fd, fa, fb);
  }
  const w::layout_t dl = d_col ? w::mem_col_major : w::mem_row_major;
  if (mul != 1.f)
    tcec::store_matrix_sync(d, fd, N, 1.f / mul, dl);
  else
    tcec::store_matrix_sync(d, fd, N, dl);
  tcec::fill_zero(fd);
}

// --------------------------------------------------------------------------
// One MMA through the mtk::wmma::mma spelling of the primitives.  a: M x K,
// b: K x N, c/d: M x N fp32 images in the given layouts (dense leading
// dimensions); operands are cast to T while loading.
// --------------------------------------------------------------------------
template <class T, int M, int N, int K, class AL, class BL>
__global__ void __launch_bounds__(64)
    primitive_mma_kernel(float *const d, const float *const a,
                         const float *const b, const float *const c,
                         const int c_col, const int d_col) {
  namespace mma = w::mma;
  mma::fragment<w::matrix_a, M, N, K, T, AL> fa;
  mma::fragment<w::matrix_b, M, N, K, T, BL> fb;
  mma::fragment<w::accumulator, M, N, K, float> fc, fd;
  mma::load_matrix_sync(fa, a, std::is_same<AL, w::col_major>::value ? M : K);
  mma::load_matrix_sync(fb, b, std::is_same<BL, w::col_major>::value ? K : N);
  if (c != nullptr)
    mma::load_matrix_sync(fc, c, c_col ? M : N,
                          c_col ? w::mem_col_major : w::mem_row_major);
  else
    mma::fill_zero(fc);
  mma::mma_sync(fd, fa, fb, fc);
  mma::store_matrix_sync(d, fd, d_col ? M : N,
                         d_col ? w::mem_col_major : w::mem_row_major);
}

// --------------------------------------------------------------------------
// The same MMA through the policy-dispatched function objects of
// tcec::detail (foreach_ij_wrapper and foreach_wrapper with
// compute_mem_offset for the operands, load_matrix_sync_wrapper or
// fill_fragment_wrapper for C, mma_sync_wrapper, store_matrix_sync_wrapper).
// float operands take the fp32 policy, whose sub-fragments hold floats.
// --------------------------------------------------------------------------
template <class T, int M, int N, int K, class AL, class BL>
__global__ void __launch_bounds__(64)
    wrapper_mma_kernel(float *const d, const float *const a,
                       const float *const b, const float *const c,
                       const int c_col, const int d_col) {
  namespace td = tcec::detail;
  using Op = typename std::conditional<std::is_same<T, float>::value,
                                       tcec::op_simt, tcec::op_mfma>::type;
  using P = tcec::Policy<Op, tcec::with_ec, M, N, K>;
  td::policy_fragment_t<w::matrix_a, T, AL, P> fa;
  td::policy_fragment_t<w::matrix_b, T, BL, P> fb;
  td::policy_fragment_t<w::accumulator, float, void, P> fc, fd;
  using ET = typename decltype(fa)::element_type;
  td::fill_zero_wrapper<w::matrix_a, T, AL, P>{}(fa);
  td::fill_zero_wrapper<w::matrix_b, T, BL, P>{}(fb);
  const unsigned lda = std::is_same<AL, w::col_major>::value ? M : K;
  const unsigned ldb = std::is_same<BL, w::col_major>::value ? K : N;
  td::foreach_ij_wrapper<w::matrix_a, T, AL, P>{}(
      [&](const unsigned *list, const unsigned count, const unsigned i,
          const unsigned j) {
        const unsigned off = td::compute_mem_offset<M, K, AL>{}(i, j, lda, 0u, 0u);
        for (unsigned f = 0; f < count; f++)
          fa.x[list[f]] = w::detail::common::cast<ET>(a[off]);
      });
  td::foreach_wrapper<w::matrix_b, T, BL, P>{}(
      [&](const unsigned *list, const unsigned count,
          const unsigned mem_index) {
        const unsigned off =
            td::compute_mem_offset<K, N, BL>{}(mem_index, ldb, 0u, 0u);
        for (unsigned f = 0; f < count; f++)
          fb.x[list[f]] = w::detail::common::cast<ET>(b[off]);
      });
  if (c != nullptr)
    td::load_matrix_sync_wrapper<w::accumulator, float, void, P>{}(
        fc, c, c_col ? M : N, c_col ? w::mem_col_major : w::mem_row_major);
  else
    td::fill_fragment_wrapper<w::accumulator, float, void, P, float>{}(fc, 0.f);
  td::mma_sync_wrapper<T, AL, BL, float, P>{}(fd, fa, fb, fc);
  td::store_matrix_sync_wrapper<float, P>{}(
      d, fd, d_col ? M : N, d_col ? w::mem_col_major : w::mem_row_major);
}

// --------------------------------------------------------------------------
// Error-corrected 16x16x16 product written with foreach only: the callback's
// mem_index addresses the dense tile, the fragment registers receive the
// leading half and the residual half of every element, and three MMAs follow.
// a, b: 16x16 fp32, column-major for A and row-major for B as in the
// reference's test; d column-major.
// --------------------------------------------------------------------------
__global__ void __launch_bounds__(64)
    foreach_ec_kernel(float *const d, const float *const a,
                      const float *const b) {
  using FA = w::fragment<w::matrix_a, 16, 16, 16, w::half, w::col_major>;
  using FB = w::fragment<w::matrix_b, 16, 16, 16, w::half, w::row_major>;
  FA fa, fda;
  FB fb, fdb;
  w::fragment<w::accumulator, 16, 16, 16, float> fc;
  w::foreach<FA>([&](const unsigned *list, const unsigned count,
                     const unsigned mem_index) {
    const float v = a[mem_index];
    const w::half hv = w::detail::common::cast<w::half>(v);
    const w::half dv =
        w::detail::common::cast<w::half>(v - static_cast<float>(hv));
    for (unsigned f = 0; f < count; f++) {
      fa.x[list[f]] = hv;
      fda.x[list[f]] = dv;
    }
  });
  w::foreach<FB>([&](const unsigned *list, const unsigned count,
                     const unsigned mem_index) {
    const float v = b[mem_index];
    const w::half hv = w::detail::common::cast<w::half>(v);
    const w::half dv =
        w::detail::common::cast<w::half>(v - static_cast<float>(hv));
    for (unsigned f = 0; f < count; f++) {
      fb.x[list[f]] = hv;
      fdb.x[list[f]] = dv;
    }
  });
  w::fill_zero(fc);
  w::mma_sync(fc, fa, fdb, fc);
  w::mma_sync(fc, fda, fb, fc);
  w::mma_sync(fc, fa, fb, fc);
  w::foreach<decltype(fc)>(w::mem_col_major,
                           [&](const unsigned *list, const unsigned count,
                               const unsigned mem_index) {
                             for (unsigned f = 0; f < count; f++)
                               d[mem_index] = fc.x[list[f]];
                           });
}

// --------------------------------------------------------------------------
// y^T = x^T * E for a 16x16 matrix E (the reference uses the identity): x goes
// into the first row of a row_major matrix_a fragment through load_vector, the
// product's first row comes back through store_vector.
// --------------------------------------------------------------------------
__global__ void __launch_bounds__(64)
    gevm_kernel(float *const y, const float *const x, const float *const e) {
  w::fragment<w::matrix_a, 16, 16, 16, w::half, w::row_major> fa;
  w::fragment<w::matrix_b, 16, 16, 16, w::half, w::col_major> fb;
  w::fragment<w::accumulator, 16, 16, 16, float> fc;
  w::load_vector(fa, x);
  w::load_matrix_sync(fb, e, 16);
  w::fill_zero(fc);
  w::mma_sync(fc, fa, fb, fc);
  w::store_vector(y, fc, w::mem_row_major);
}

// --------------------------------------------------------------------------
// Fragment operators.  a, b: 16x16 row-major fp32 tiles, cast to T on the way
// in; out: the result fragment written back the same way.
//   op 0: a + b   1: a - b   2: a * alpha   3: a / alpha
//   op 4: fma(alpha, a, b)   5: fma(a, alpha, b)
// --------------------------------------------------------------------------
template <class Use, class T, class Layout>
__global__ void __launch_bounds__(64)
    fragment_ops_kernel(float *const out, const float *const a,
                        const float *const b, const float alpha, const int op) {
  using F = w::fragment<Use, 16, 16, 16, T, Layout>;
  using S = typename F::storage_element_type;
  F fa, fb, fr;
  w::detail::foreach_ij_core<F>([&](const unsigned *list, const unsigned,
                                    const unsigned i, const unsigned j) {
    fa.x[list[0]] = w::detail::common::cast<T>(a[i * 16 + j]);
    fb.x[list[0]] = w::detail::common::cast<T>(b[i * 16 + j]);
  });
  const S s = w::detail::common::cast<T>(alpha);
  switch (op) {
  case 0:
    fr = fa + fb;
    break;
  case 1:
    fr = fa - fb;
    break;
  case 2:
    fr = fa * s;
    break;
  case 3:
    fr = fa / s;
    break;
  case 4:
    fr = w::fma(s, fa, fb);
    break;
  default:
    fr = w::fma(fa, s, fb);
    break;
  }
  w::detail::foreach_ij_core<F>([&](const unsigned *list, const unsigned,
                                    const unsigned i, const unsigned j) {
    out[i * 16 + j] = static_cast<float>(fr.x[list[0]]);
  });
}

// fill(1) then add_eye(alpha), or make_identity_matrix; stored column-major.
template <int M, int N, int K>
__global__ void __launch_bounds__(64)
    fragment_eye_kernel(float *const out, const float alpha,
                        const int identity) {
  w::fragment<w::accumulator, M, N, K, float> frag;
  if (identity) {
    w::fill_fragment(frag, 7.0f); // must be overwritten
    w::make_identity_matrix(frag);
  } else {
    w::fill_fragment(frag, 1.0f);
    w::add_eye(frag, alpha);
  }
  w::store_matrix_sync(out, frag, M, w::mem_col_major);
}

// h (16x16, column-major) = u v^T through one MMA on direct-product fragments.
// from_float == 0: the 16-bit parts x, dx are prepared in LDS first and given
// to the (x, dx) overload; otherwise the fp32 overload splits on the fly.
template <class T, unsigned TERMS>
__global__ void __launch_bounds__(64)
    direct_product_kernel(float *const h, const float *const u,
                          const float *const v, const int from_float) {
  using S = typename w::detail::common::storage_t<T>::type;
  w::fragment<w::matrix_a, 16, 16, 16, T, w::col_major> fa;
  w::fragment<w::matrix_b, 16, 16, 16, T, w::row_major> fb;
  w::fragment<w::accumulator, 16, 16, 16, float> fc;
  __shared__ S su[16], sdu[16], sv[16], sdv[16];
  if (threadIdx.x < 16) {
    const float f = u[threadIdx.x];
    const S hv = w::detail::common::cast<T>(f);
    su[threadIdx.x] = hv;
    sdu[threadIdx.x] = w::detail::common::cast<T>(f - static_cast<float>(hv));
  } else if (threadIdx.x < 32) {
    const float f = v[threadIdx.x - 16];
    const S hv = w::detail::common::cast<T>(f);
    sv[threadIdx.x - 16] = hv;
    sdv[threadIdx.x - 16] = w::detail::common::cast<T>(f - static_cast<float>(hv));
  }
  __syncthreads();
  // start from junk so that `fill` is seen to work
  w::fill_fragment(fa, w::detail::common::cast<T>(3.0f));
  w::fill_fragment(fb, w::detail::common::cast<T>(3.0f));
  if (from_float) {
    if constexpr (TERMS == 3) {
      w::make_direct_product_fragment_c3(fa, u);
      w::make_direct_product_fragment_c3(fb, v);
    } else {
      w::make_direct_product_fragment(fa, u);
      w::make_direct_product_fragment(fb, v);
    }
  } else {
    if constexpr (TERMS == 3) {
      w::make_direct_product_fragment_c3(fa, su, sdu);
      w::make_direct_product_fragment_c3(fb, sv, sdv);
    } else {
      w::make_direct_product_fragment(fa, su, sdu);
      w::make_direct_product_fragment(fb, sv, sdv);
    }
  }
  w::fill_zero(fc);
  w::mma_sync(fc, fa, fb, fc);
  w::store_matrix_sync(h, fc, 16, w::mem_col_major);
}

// --------------------------------------------------------------------------
// Shader-clock sampler: one lane records (constant 100 MHz counter, shader
// cycle counter) pairs every `period` ticks of the constant counter, nsamples
// times, then ends.  Run beside another kernel (on a second stream) it shows
// how far the clock is pulled down while that kernel runs: on this chip the
// matrix cores are power limited as soon as the operands are not constant.
// The loop is bounded by the sample count and every wait by the constant
// counter, so the kernel always ends.
// --------------------------------------------------------------------------
__global__ void __launch_bounds__(64)
    clock_samples_kernel(unsigned long long *const out, const int nsamples,
                         const unsigned long long period) {
  if (threadIdx.x != 0)
    return;
  const unsigned long long t0 = wall_clock64();
  for (int i = 0; i < nsamples; i++) {
    const unsigned long long target = t0 + static_cast<unsigned long long>(i) * period;
    unsigned long long now = wall_clock64();
    while (now < target) {
      __builtin_amdgcn_s_sleep(8);
      now = wall_clock64();
    }
    out[2 * i] = now;
    out[2 * i + 1] = clock64();
  }
}

// --------------------------------------------------------------------------
// utils::cp_async: 128 threads move 256 elements of Size bytes through LDS.
//   mode 0: dst[t] <- smem[t] <- src[t] (the reference's test; lane-linear
//           destinations, served by the direct global->LDS load), both halves
//   mode 1: scattered destinations smem[(37 t + 5) % 128] (register path)
//   mode 2: only threads with t % 3 != 0 copy; the others' slots are zeroed
//           first (direct load under a partial execution mask)
//   mode 3: two groups in flight, wait_pending<1> releases the first
//   mode 4: mode 0 through cp_async_lane_linear (Size 4 or 16)
//   mode 5: mode 2 through cp_async_lane_linear (Size 4 or 16)
// --------------------------------------------------------------------------
template <unsigned Size>
__global__ void __launch_bounds__(128)
    cp_async_kernel(uint32_t *const dst, const uint32_t *const src,
                    const int mode) {
  namespace cpa = w::utils::cp_async;
  constexpr unsigned W = Size / 4; // words per element
  __shared__ __attribute__((aligned(16))) uint32_t smem[2][128 * W];
  const unsigned t = threadIdx.x;
  auto out = [&](const unsigned elem, const uint32_t *const from) {
    for (unsigned i = 0; i < W; i++)
      dst[elem * W + i] = from[i];
  };
  if (mode == 0) {
    cpa::cp_async<Size>(&smem[0][t * W], src + t * W);
    cpa::cp_async<Size>(&smem[1][t * W], src + (128 + t) * W);
    cpa::commit();
    cpa::wait_all();
    out(t, &smem[0][t * W]);
    out(128 + t, &smem[1][t * W]);
  } else if (mode == 1) {
    const unsigned p = (37 * t + 5) % 128;
    cpa::cp_async<Size>(&smem[0][p * W], src + t * W);
    cpa::cp_async<Size>(&smem[1][p * W], src + (128 + t) * W);
    cpa::commit();
    cpa::wait_group<0>();
    out(t, &smem[0][p * W]);
    out(128 + t, &smem[1][p * W]);
  } else if (mode == 2) {
    for (unsigned i = 0; i < W; i++)
      smem[0][t * W + i] = smem[1][t * W + i] = 0u;
    __syncthreads();
    if (t % 3 != 0) {
      cpa::cp_async<Size>(&smem[0][t * W], src + t * W);
      cpa::cp_async<Size>(&smem[1][t * W], src + (128 + t) * W);
    }
    cpa::commit();
    cpa::wait_all();
    out(t, &smem[0][t * W]);
    out(128 + t, &smem[1][t * W]);
  } else if (mode == 4 || mode == 5) {
    if constexpr (Size != 8) {
      if (mode == 5) {
        for (unsigned i = 0; i < W; i++)
          smem[0][t * W + i] = smem[1][t * W + i] = 0u;
        __syncthreads();
      }
      if (mode == 4 || t % 3 != 0) {
        cpa::cp_async_lane_linear<Size>(&smem[0][t * W], src + t * W);
        cpa::cp_async_lane_linear<Size>(&smem[1][t * W], src + (128 + t) * W);
      }
      cpa::commit();
      cpa::wait_all();
      out(t, &smem[0][t * W]);
      out(128 + t, &smem[1][t * W]);
    }
  } else {
    cpa::cp_async<Size>(&smem[0][t * W], src + t * W);
    cpa::commit();
    cpa::cp_async<Size>(&smem[1][t * W], src + (128 + t) * W);
    cpa::commit();
    cpa::wait_pending<1>(); // the first copy has landed, the second may fly
    out(t, &smem[0][t * W]);
    cpa::wait_all();
    out(128 + t, &smem[1][t * W]);
  }
}

// utils::cp_async as a three-stage pipeline written with the reference's group
// calls only (cp_async, commit, wait_group<2>; the use its utils.hpp:29-64 is
// made for): one wave moves `groups` (<= 8) groups of `copies` (<= 4) copies
// (64 lanes x Size bytes each) through a ring of three LDS buffers; while group
// g is consumed, groups g+1 and g+2 are in flight.  The consumer moves a group
// on inside LDS, and dst is written after the pipeline has drained, so that the
// copies are the wave's only vector-memory instructions while it runs and
// pending[] shows them alone: pending[0] is the wave's count of outstanding
// vector-memory instructions (the hardware's own counter) once the first three
// groups are out, pending[1 + g] the same right after the wait_group<2> that
// releases group g, pending[1 + groups] after wait_all.
template <unsigned Size>
__global__ void __launch_bounds__(64)
    cp_async_pipeline_kernel(uint32_t *const dst, const uint32_t *const src,
                             const int groups, const int copies,
                             int *const pending) {
  namespace cpa = w::utils::cp_async;
  constexpr unsigned W = Size / 4, STAGES = 3, MAX_COPIES = 4, MAX_GROUPS = 8;
  constexpr unsigned GROUP_WORDS = MAX_COPIES * 64 * W;
  __shared__ __attribute__((aligned(16))) uint32_t ring[STAGES][GROUP_WORDS];
  __shared__ __attribute__((aligned(16))) uint32_t landed[MAX_GROUPS][GROUP_WORDS];
  __shared__ int seen[MAX_GROUPS + 2];
  const unsigned lane = threadIdx.x;
  // vm_cnt of the wave: bits 3:0 and 23:22 of the instruction-buffer status
  auto outstanding = [&]() {
    const unsigned v = __builtin_amdgcn_s_getreg((31 << 11) | 7);
    return static_cast<int>((v & 15u) | (((v >> 22) & 3u) << 4));
  };
  auto issue = [&](const int g) {
    if (g < groups)
      for (int c = 0; c < copies; c++)
        cpa::cp_async<Size>(&ring[g % STAGES][(c * 64 + lane) * W],
                            src + (static_cast<size_t>(g * copies + c) * 64 + lane) * W);
    cpa::commit(); // (an empty group past the end keeps the group count in step)
  };
  for (int g = 0; g < static_cast<int>(STAGES); g++)
    issue(g);
  int now = outstanding();
  if (lane == 0)
    seen[0] = now;
  for (int g = 0; g < groups; g++) {
    cpa::wait_group<STAGES - 1>();
    now = outstanding();
    if (lane == 0)
      seen[1 + g] = now;
    for (int c = 0; c < copies; c++)
      for (unsigned i = 0; i < W; i++)
        landed[g][(c * 64 + lane) * W + i] =
            ring[g % STAGES][(c * 64 + lane) * W + i];
    // the buffer is refilled only after its contents have been read out
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    issue(g + STAGES);
  }
  cpa::wait_all();
  now = outstanding();
  if (lane == 0)
    seen[1 + groups] = now;
  __syncthreads();
  for (int g = 0; g < groups; g++)
    for (int c = 0; c < copies; c++)
      for (unsigned i = 0; i < W; i++)
        dst[(static_cast<size_t>(g * copies + c) * 64 + lane) * W + i] =
            landed[g][(c * 64 + lane) * W + i];
  for (int i = static_cast<int>(lane); i < groups + 2; i += 64)
    pending[i] = seen[i];
}

// print_fragment of both layers, one wave: a 16x16x16 half matrix_a fragment
// loaded from `src` (16x16 row-major) and a 32x32 TCEC accumulator filled
// with `base` whose error part is set to 2048 * lane (printed divided by the
// split's scale).  Output goes to the process's stdout through device printf.
// (reference: detail/print.hpp / tcec/detail/print.hpp:11-55, used by
// test/primitive/print_fragment.cu)
template <class T, class Policy>
__global__ void __launch_bounds__(64)
    print_fragment_kernel(const float *const src, const float base) {
  w::fragment<w::matrix_a, 16, 16, 16, w::half, w::row_major> fa;
  w::load_matrix_sync(fa, src, 16);
  w::print_fragment(fa, "prim_a");
  using F = tcec::fragment<w::accumulator, 32, 32, 32, T, void, Policy>;
  F frag;
  tcec::fill_fragment(frag, base);
  if constexpr (F::num_terms >= 2) {
    const unsigned lane = w::detail::common::get_lane_id();
    for (unsigned i = 0; i < F::num_elements; i++)
      frag.dx(i) = 2048.f * static_cast<float>(lane);
  }
  tcec::print_fragment(frag, "tcec_acc");
}

// utils::cast<DST>(in[i]) for DST = half, bfloat16 (16-bit patterns out),
// precision::tf32 and float (fp32 out).
template <class DST>
__global__ void __launch_bounds__(256)
    cast_kernel(const float *const in, void *const out, const long long n) {
  const long long i =
      static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n)
    return;
  const auto v = w::utils::cast<DST>(in[i]);
  if constexpr (sizeof(v) == 2)
    static_cast<unsigned short *>(out)[i] =
        __builtin_bit_cast(unsigned short, v);
  else
    static_cast<float *>(out)[i] = v;
}

} // namespace wmmae_harness
