// extern "C" boundary of libwmmae_tcec.so, GEMM driver part: argument
// validation, kernel selection and launches of the split pass, the packed
// GEMM and the single-kernel GEMM.  Declarations and per-entry documentation
// live in include/wmmae_tcec.h.
#include "capi_common.hpp"
#include <limits>
#include "tcec_gemm_fused_kernel.hpp"
#include "tcec_gemm_kernels.hpp"

namespace {
using namespace wmmae_capi;
using wmmae_gemm::u32x4;

// ------------------------------------------------------------ policy table
struct PolicyInfo {
  int terms;       // stored terms per operand
  bool bf16;       // MFMA element type
  float inv_scale; // factor applied to the error accumulator
};
inline bool policy_info(const int policy, PolicyInfo &p) {
  switch (policy) {
  case WMMAE_POLICY_F16_EC:
    p = {2, false, 1.f / 2048.f};
    return true;
  case WMMAE_POLICY_F16_NOEC:
    p = {1, false, 1.f};
    return true;
  case WMMAE_POLICY_BF16X3_EC:
    p = {3, true, 1.f};
    return true;
  case WMMAE_POLICY_BF16X2_EC:
    p = {2, true, 1.f};
    return true;
  case WMMAE_POLICY_BF16_NOEC:
    p = {1, true, 1.f};
    return true;
  default:
    return false;
  }
}

// packed operand geometry: 16-row blocks, 32-wide k chunks
inline long long packed_row_blocks(const int rows) { return ceil_div(rows, 16); }
inline int packed_k_tiles(const int k) {
  return static_cast<int>(ceil_div(k, 32));
}
// u32x4 elements of one packed matrix
inline long long packed_elems(const int rows, const int k, const int terms) {
  return packed_row_blocks(rows) * packed_k_tiles(k) * terms * 64;
}

// ------------------------------------------------------------------ pack
// One operand of a split launch as the caller describes it.
struct PackSource {
  int rows;
  const float *X;
  const float *const *ptrs;
  long long row_stride, k_stride, batch_stride;
  void *packed;
};

inline wmmae_gemm::PackOperand pack_operand(const PackSource &src,
                                            const int KT) {
  wmmae_gemm::PackOperand o;
  o.X = src.X;
  o.ptrs = src.ptrs;
  o.row_stride = src.row_stride;
  o.k_stride = src.k_stride;
  o.batch_stride = src.batch_stride;
  o.rows = src.rows;
  o.chunks = packed_row_blocks(src.rows) * KT;
  o.out = static_cast<u32x4 *>(src.packed);
  return o;
}

// The batch index of the split, scale and fold kernels is the grid's y
// coordinate, which ends at 65535: longer batches take one launch per 65535
// entries.
constexpr int kMaxGridY = 65535;

// Splits one operand (b == nullptr) or both operands of a product in a single
// launch.
template <class T, int TERMS>
int launch_pack(const int k, const int batch, const PackSource &a,
                const PackSource *const b, hipStream_t stream) {
  const int KT = packed_k_tiles(k);
  const wmmae_gemm::PackOperand oa = pack_operand(a, KT);
  const long long blocks_a = ceil_div(oa.chunks * 64, 256);
  if (b == nullptr) {
    if (blocks_a > 0x7fffffffLL)
      return WMMAE_STATUS_NOT_SUPPORTED;
    for (int e0 = 0; e0 < batch; e0 += kMaxGridY)
      hipLaunchKernelGGL((wmmae_gemm::split_pack_kernel<T, TERMS>),
                         dim3(static_cast<unsigned>(blocks_a),
                              std::min(batch - e0, kMaxGridY)),
                         dim3(256), 0, stream, oa, k, KT,
                         static_cast<unsigned>(e0));
    return launch_status();
  }
  const wmmae_gemm::PackOperand ob = pack_operand(*b, KT);
  const long long blocks_b = ceil_div(ob.chunks * 64, 256);
  if (blocks_a + blocks_b > 0x7fffffffLL)
    return WMMAE_STATUS_NOT_SUPPORTED;
  for (int e0 = 0; e0 < batch; e0 += kMaxGridY)
    hipLaunchKernelGGL((wmmae_gemm::split_pack_pair_kernel<T, TERMS>),
                       dim3(static_cast<unsigned>(blocks_a + blocks_b),
                            std::min(batch - e0, kMaxGridY)),
                       dim3(256), 0, stream, oa, ob,
                       static_cast<unsigned>(blocks_a), k, KT,
                       static_cast<unsigned>(e0));
  return launch_status();
}

int pack_dispatch(const int policy, const int k, const int batch,
                  const PackSource &a, const PackSource *const b,
                  hipStream_t stream) {
  switch (policy) {
  case WMMAE_POLICY_F16_EC:
    return launch_pack<w::half, 2>(k, batch, a, b, stream);
  case WMMAE_POLICY_F16_NOEC:
    return launch_pack<w::half, 1>(k, batch, a, b, stream);
  case WMMAE_POLICY_BF16X3_EC:
    return launch_pack<w::precision::tf32, 3>(k, batch, a, b, stream);
  case WMMAE_POLICY_BF16X2_EC:
    return launch_pack<w::bfloat16, 2>(k, batch, a, b, stream);
  case WMMAE_POLICY_BF16_NOEC:
    return launch_pack<w::bfloat16, 1>(k, batch, a, b, stream);
  default:
    return WMMAE_STATUS_INVALID_VALUE;
  }
}

// ------------------------------------------------------------------ gemm
struct GemmArgs {
  const u32x4 *a, *b;
  float *c;
  int m, n, k;
  long long ldc, stride_c;
  float alpha, beta, inv_scale;
  int batch, terms;
  float *const *c_ptrs; // device array of C pointers, or nullptr
  float *partial;  // split-K slices, or nullptr
  int splits;      // >= 1
  // room for the K slices of the tiles of a partly empty last round (used
  // only without split-K), or nullptr
  float *tail_ws;
  size_t tail_ws_bytes;
  hipStream_t stream;
  // fp32 operands for the kernel variant that splits them itself (a and b are
  // null then)
  bool is_direct = false;
  wmmae_gemm::DirectSource direct = {};
};

// Compute units of the current device, looked up once per device.
inline int device_cus() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess)
    return 256; // MI355X; also the answer when no device is visible
  const bool tracked = dev >= 0 && dev < 64;
  if (tracked) {
    const int c = cached[dev].load(std::memory_order_relaxed);
    if (c > 0)
      return c;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, dev) != hipSuccess ||
      prop.multiProcessorCount <= 0)
    return 256;
  if (tracked)
    cached[dev].store(prop.multiProcessorCount, std::memory_order_relaxed);
  return prop.multiProcessorCount;
}

// ------------------------------------------------ fitted cost parameters
// Every number the path and tile choices below are made with, in one place.
// All are fits to measurements on MI355X (256 compute units, one box of the
// pool each; the boxes differ by 3 to 5 % in what they sustain under the power
// limit).  The estimates have one form: launch cost + rounds of tiles over the
// compute units x (k stages of 32 x time per stage + time per tile), bounded
// below by the bytes moved.
namespace fit {
// -- packed GEMM, time of one k stage of one tile, by stored terms (1, 2, 3).
//    Sweep: 216 products, m = n = 512 .. 2048, k = 512 .. 4096, each run with
//    1, 2, 3, 4, 6 and 8 K slices; the slice count chosen with them is within
//    0.7 % of the best measured one on average (1.9 % on 120 random products
//    with m, n = 64 .. 2900, k = 400 .. 32000, 1 .. 100 entries, 1 .. 32
//    slices forced).
constexpr double kStage256x128[3] = {0.8e-6, 1.0e-6, 1.82e-6};
constexpr double kStage128x128[3] = {0.45e-6, 0.6e-6, 0.99e-6};
constexpr double kStage64x64 = 0.25e-6;
constexpr double kTileOverhead = 7e-6;    // pipeline fill + epilogue of a tile
constexpr double kFoldLaunch = 6e-6;      // the pass that adds the K slices
constexpr double kFoldBytesPerS = 3e12;   // ... reads and writes its planes at
constexpr double kSplitMustBeat = 0.95;   // a split has to win by 5 %
// -- tile choice, cost of a tile in units of one 128x128 tile.  Sweep: both
//    tiles forced on 124 products, 1024^2 .. 8192^2, k = 256 .. 4096, some
//    batched: the choice is within 0.4 % of the faster tile on average.
constexpr double kUnits256x128 = 2.0;
constexpr double kUnits128x128 = 1.2;     // one and two terms
//    Three terms (sweep: both tiles forced on 36 products, 1024^2 .. 8192^2,
//    k = 1024 .. 5000, some batched or rectangular: a round of 256x128 tiles
//    costs 1.8 rounds of 128x128 tiles, so the large tile wins when it halves
//    the rounds, 8 to 14 %, and loses otherwise, 3 % at 7 -> 4 rounds, 17 to
//    20 % at 3 -> 2).
constexpr double kUnits256x128Terms3 = 1.8;
constexpr double kUnits128x128Terms3 = 1.0;
constexpr double kUnits64x64 = 0.4;
constexpr double units256x128(const int terms) {
  return terms == 3 ? kUnits256x128Terms3 : kUnits256x128;
}
constexpr double units128x128(const int terms) {
  return terms == 3 ? kUnits128x128Terms3 : kUnits128x128;
}
// -- K slices for a partly empty last round: slices, pipeline refills, fold.
//    Sweep: 126 products, 2304^2 .. 8192^2, k = 2048 .. 8192, two policies.
constexpr double kTailOverhead = 0.2;
// -- which path: the single kernel, split passes + GEMM on packed operands, or
//    the GEMM kernel that splits the fp32 operands itself.  Fit: 1860 random
//    products (m, n = 45 .. 5000, k = 32 .. 32768, 1 .. 1024 entries, half of
//    them with dimensions that are multiples of nothing, all five policies),
//    each run with every path forced; the constants below minimise the
//    squared log error of each path's estimate on 1060 of them and on 137
//    structured products (the reference harness's grid with 256 entries,
//    squares 1024 .. 8192, the baseline workloads; weighted four times).  On
//    the 800 held out the path chosen with them is 1.4 % slower than always
//    taking the fastest forced path on average (37 of 800 above 1.10 x, six
//    above 1.25 x), on the structured ones 0.5 % (two above 1.10 x); the
//    constants before (fits to the harness's grid and to square products)
//    were 3 to 6 % slower on the same 800, 3.1 x at worst.  Whole default
//    calls on 400 further random products: 1.1 % (worst 1.48 x).
//    Rows: one, two, three terms.
struct PathRates {
  double launch, stage, tile, bytes_per_s; // seconds, seconds, seconds, B/s
  double split_bytes_per_s;                // packed path only
  // A k stage takes longer the fuller the chip is (power limit, contention in
  // L2 and HBM): stage * (1 + busy * (compute units with a tile / all compute
  // units, averaged over the rounds))
  double busy;
};
constexpr PathRates kFused[3] = {
    {6.01e-6, 0.643e-6, 2.88e-6, 5.32e12, 0., 0.101},
    {6.50e-6, 0.992e-6, 1.85e-6, 5.27e12, 0., 0.170},
    {5.37e-6, 1.39e-6, 2.22e-6, 5.14e12, 0., 0.141}};
constexpr PathRates kPacked[3] = {
    {8.35e-6, 0.131e-6, 3.07e-6, 3.65e12, 5.61e12, 0.359},
    {8.17e-6, 0.287e-6, 3.69e-6, 6.50e12, 5.57e12, 0.649},
    {7.10e-6, 0.652e-6, 4.65e-6, 6.50e12, 4.92e12, 0.361}};
// -- the packed path's GEMM kernel reading and splitting the fp32 operands
//    itself (256x128 tiles only; rows: one, two terms)
constexpr PathRates kDirect[2] = {
    {3.41e-6, 0.173e-6, 3.76e-6, 4.62e12, 0., 1.18},
    {5.00e-6, 0.355e-6, 3.65e-6, 4.92e12, 0., 0.750}};
// ... as the host sees it when it decides whether a launch of that kernel is
// bound by its bytes and should start its workgroups staggered (a fit of its
// own, to the reference harness's grid: 0.8 / 1.5 us per k stage of a 256x128
// tile and 6 us per tile, in units of half a tile)
constexpr PathRates kDirectStagger[2] = {
    {6.0e-6, 0.40e-6, 3.0e-6, 5.0e12, 0., 0.},
    {6.0e-6, 0.75e-6, 3.0e-6, 5.0e12, 0., 0.}};
// with K slices: the GEMM's time against the packed kernel's estimate for the
// same slices of 256x128 tiles (two terms: twelve K-sliced products, m, n =
// 64 .. 4096, k = 2048 .. 262144, each run on either path: with 1.4 the faster
// path is chosen for all of them, with 1.5 for eleven)
constexpr double kDirectSliceRatio[2] = {1.5, 1.4};
// Products that are cut into K slices (few output tiles): what the slice
// planner's time (split_time, whose constants are fitted for choosing the slice
// count) has to be scaled and shifted by to be the time of the whole call on
// each path; same fit as above.  Rows: scale, shift in seconds; by terms.
constexpr double kSlicedFused[2][3] = {{1.16, 1.08, 1.03},
                                       {-3.73e-6, -2.84e-6, -2.89e-6}};
constexpr double kSlicedPacked[2][3] = {{0.724, 0.954, 0.955},
                                        {-0.65e-6, -6.0e-6, -6.0e-6}};
constexpr double kSlicedDirect[2][2] = {{0.759, 0.890}, {-6.0e-6, -6.0e-6}};
// Calls issued back to back cannot complete faster than the host issues their
// launches (250 products below 1.5e8 flop, called in a loop: 11, 14.5 and 12 us
// per call in the median): what decides among the paths for tiny products -
// one launch for the single kernel and the direct kernel, two or three for
// the packed path.  Order: single kernel, packed, direct.
constexpr double kCallFloor[3] = {11.0e-6, 14.3e-6, 11.5e-6};
// k % 32 != 0: the kernel variant that reads a shorter last stage (1024^2 x 1000
// against x 1024, batch 256: 301 against 336 TFLOPS, of which 2.4 % are the k)
constexpr double kDirectTailStage = 1.47;
// the single kernel's 64x64 tile against its 128x128 tile (1024^3: 41 -> 27 us)
constexpr double kFusedSmallTileTime = 0.65; // whole tile, latency-bound sizes
constexpr double kFusedSmallStage = 0.599, kFusedSmallTile = 0.467;
// 4-byte instead of 16-byte requests: 114 random products with k % 4 != 0 ran
// at 0.55 of the packed path's speed in the median
constexpr double kFusedNarrowRequests = 3.50;
} // namespace fit

// XCDs (chiplets with an L2 of their own) behind the current device.  HIP does
// not report them; a gfx950 XCD has 32 active compute units in every partition
// mode (SPX 256 = 8 x 32, DPX 128, QPX 64, CPX 32), so the count follows from
// the compute units.  Consecutive workgroup ids go round-robin over the XCDs;
// the kernels' XCD-aware item lists are written for eight of them and are used
// only then (other counts take the plain shared list: same results, tiles not
// grouped by L2).
inline int device_xcds() {
  const int cus = device_cus();
  return cus % 32 == 0 ? cus / 32 : 1;
}
constexpr int kKernelXcds = 8; // the constant XCDS of the kernels' item lists

// Number of K slices of every tile, when the 256x128 output tiles cannot fill
// half the chip.  For every candidate (at most 32 slices of at least 6 stages)
// the GEMM's time is estimated the way gemm_by_size will run it: the tile that
// the slice count leads to, rounds of those tiles over the compute units,
// stages per slice at that tile's time per stage, a fixed time per tile, and
// for more than one slice the fold (a launch plus the planes written and
// read).  The cheapest count is taken, any split having to beat the uncut run
// by 5 %.  Times per stage and tile: fits to measurements on MI355X (216
// products, m = n = 512 .. 2048, k = 512 .. 4096, one to three terms, each run
// with 1, 2, 3, 4, 6 and 8 slices: the choice is within 0.7 % of the best measured count on
// average; "as many slices as fill the chip with 256x128 tiles" was 7 % off,
// over-cutting outputs from 1280^2 up and not cutting short loops at all).
// Whether the 256x128 tile is a candidate at all: only where the 128x128 tiles
// need more than one round over the compute units (in a single round the
// smaller tile always finishes first), and not for the one-term kernels on
// loops of 32 stages or fewer, where the stores of C dominate and the smaller
// tile measured 8 to 12 % faster.  (Forced-tile runs of 124 products: the
// choice below is within 0.4 % of the faster tile on average; requiring a full
// round of 256x128 tiles instead had cost 2 %, up to 13 % at 2560^2 .. 2816^2.)
inline bool big_tile_candidate(const int terms, const long long mid,
                               const int kt) {
  return mid > device_cus() && !(terms == 1 && kt <= 32);
}
// `direct`: the kernel that splits the fp32 operands itself, which has the
// 256x128 tile only and takes kDirectSliceRatio times the packed kernel's time
// (its slice count must be planned with its own tiles: 4096 x 64 x 4096 cut
// for the 128x128 tiles of the packed path left half the compute units
// without a 256x128 item, 48 against 39 us).
inline double split_time(const int terms, const int m, const int n,
                         const int batch, const int kt, const int slices,
                         const bool direct = false) {
  const long long cus = device_cus();
  const int stages = static_cast<int>(ceil_div(kt, slices));
  const long long z = ceil_div(kt, stages);
  const long long big = ceil_div(m, 256) * ceil_div(n, 128) * batch * z;
  const long long mid = ceil_div(m, 128) * ceil_div(n, 128) * batch * z;
  double stage_time, rounds;
  const double r_big = static_cast<double>(ceil_div(big, cus));
  const double r_mid = static_cast<double>(ceil_div(mid, cus));
  if (direct ||
      (big_tile_candidate(terms, mid, stages) &&
       r_big * fit::units256x128(terms) <= r_mid * fit::units128x128(terms))) {
    stage_time = fit::kStage256x128[terms - 1];
    rounds = r_big;
  } else if (mid >= cus || (m > 64 && n > 64)) {
    stage_time = fit::kStage128x128[terms - 1];
    rounds = r_mid;
  } else {
    stage_time = fit::kStage64x64;
    rounds = static_cast<double>(
        ceil_div(ceil_div(m, 64) * ceil_div(n, 64) * batch * z, cus));
  }
  double t = rounds * (stages * stage_time + fit::kTileOverhead);
  if (z > 1)
    t += fit::kFoldLaunch + static_cast<double>(z + 1) * m * n * batch * 4.0 /
                                fit::kFoldBytesPerS;
  return direct ? t * fit::kDirectSliceRatio[terms - 1] : t;
}
// Test hook (wmmae_tcec_force_k_slices): a slice count for the calling thread's
// next calls instead of the estimates' choice, so that two kernels can be run on
// the same cut of K and compared bit by bit.  0: the estimates choose.
thread_local int t_forced_k_slices = 0;
// Measurement hook (wmmae_tcec_time_gemm_kernel): events this thread's calls
// record on their stream right before the MFMA GEMM kernel and right after it
// (after the fold of its K slices where there is one).
thread_local hipEvent_t t_gemm_begin = nullptr, t_gemm_end = nullptr;
constexpr int kMaxSplits = 32, kMinStagesPerSplit = 6;
inline int choose_splits(const int terms, const int m, const int n, const int k,
                         const int batch, const bool direct = false) {
  const long long tiles = ceil_div(m, 256) * ceil_div(n, 128) * batch;
  const int kt = static_cast<int>(ceil_div(k, 32));
  if (t_forced_k_slices > 0) {
    const int s = std::max(
        1, std::min({t_forced_k_slices, kMaxSplits, kt / kMinStagesPerSplit}));
    return static_cast<int>(ceil_div(kt, ceil_div(kt, s)));
  }
  if (tiles * 2 > device_cus())
    return 1;
  int best = 1;
  double t_best =
      fit::kSplitMustBeat * split_time(terms, m, n, batch, kt, 1, direct);
  for (int s = 2; s <= kMaxSplits && s * kMinStagesPerSplit <= kt; s++) {
    if (ceil_div(kt, ceil_div(kt, s)) != s)
      continue; // the same slices as a smaller count
    const double t = split_time(terms, m, n, batch, kt, s, direct);
    if (t < t_best) {
      t_best = t;
      best = s;
    }
  }
  return best;
}

// K slices for the tiles of the last round only.  `tiles` output tiles run in
// rounds of `resident` (one workgroup per item, long K loops); when the last
// round is less than half full its tiles are cut into `slices` K slices of at
// least 32 stages each, so that the round takes about 1/slices of a tile's
// time (plus the pass that folds the slices).  slices == 1: not worth it.
struct TailPlan {
  long long full = 0, tail = 0; // tiles in whole rounds, tiles in the last
  int slices = 1, stages = 0;   // K slices of a tail tile, stages per slice
};
inline TailPlan plan_tail(const long long tiles, const long long resident,
                          const int KT) {
  TailPlan t;
  t.full = tiles / resident * resident;
  t.tail = tiles - t.full;
  if (t.full == 0 || t.tail == 0 || t.tail * 2 > resident || KT < 64)
    return t;
  long long s = std::min<long long>({resident / t.tail, KT / 32, 16});
  if (s < 2)
    return t;
  t.stages = static_cast<int>(ceil_div(KT, s));
  t.slices = static_cast<int>(ceil_div(KT, t.stages));
  return t;
}
// Time of `tiles` tiles in units of one tile, with and without that plan.
inline double rounds_cost(const long long tiles, const long long resident,
                          const int KT, const bool tail_allowed) {
  const TailPlan t = plan_tail(tiles, resident, KT);
  const double full_rounds = static_cast<double>(t.full / resident);
  if (t.tail == 0)
    return full_rounds;
  if (!tail_allowed || t.slices < 2)
    return full_rounds + 1.0;
  return full_rounds + 1.0 / t.slices + fit::kTailOverhead;
}

// Deepest LDS ring (at most 4 stages) that fits the 160 KiB of a compute unit.
constexpr int ring_depth(const int bm, const int bn, const int terms) {
  const int stage_bytes = (bm / 16 + bn / 16) * terms * 1024;
  const int fit = (160 * 1024) / stage_bytes;
  return fit > 4 ? 4 : fit;
}

// Workgroups of one GEMM kernel that a compute unit holds at a time: what the
// runtime's occupancy query says (registers, LDS and wave slots together),
// looked up once per kernel and device; the LDS bound alone where the query
// gives nothing (no device visible).  The persistent work-item modes give
// every resident workgroup a fixed share of the items, so a count the
// registers do not allow would leave the extra workgroups' shares to run after
// everything else (the one-term direct kernel: 48 KiB of LDS, three by that
// bound, but 512 registers a lane).
template <class MT, int TERMS, int BM, int BN, int WGM, int WGN, bool RN,
          int DIRECT = 0>
int workgroups_per_cu() {
  constexpr int NSTAGE = DIRECT ? 2 : ring_depth(BM, BN, TERMS);
  using Cfg =
      wmmae_gemm::GemmConfig<MT, TERMS, BM, BN, WGM, WGN, NSTAGE, RN, DIRECT>;
  constexpr int by_lds =
      (160 * 1024) / Cfg::LDS_BYTES > 4 ? 4 : (160 * 1024) / Cfg::LDS_BYTES;
  static std::atomic<int> cached[64];
  static std::atomic<unsigned long long> lds_allowed{0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    return by_lds;
  }
  const int c = cached[dev].load(std::memory_order_relaxed);
  if (c > 0)
    return c;
  auto kernel = wmmae_gemm::tcec_gemm_kernel<MT, TERMS, BM, BN, WGM, WGN,
                                             NSTAGE, RN, DIRECT>;
  int n = 0;
  if (allow_dynamic_lds(reinterpret_cast<const void *>(kernel), Cfg::LDS_BYTES,
                        lds_allowed) != hipSuccess ||
      hipOccupancyMaxActiveBlocksPerMultiprocessor(
          &n, reinterpret_cast<const void *>(kernel), Cfg::NTHREADS,
          Cfg::LDS_BYTES) != hipSuccess ||
      n <= 0) {
    (void)hipGetLastError();
    return by_lds;
  }
  n = n < by_lds ? n : by_lds;
  cached[dev].store(n, std::memory_order_relaxed);
  return n;
}

template <class MT, int TERMS, int BM, int BN, int WGM, int WGN, bool RN,
          int DIRECT = 0>
int launch_gemm(const GemmArgs &g) {
  constexpr int NSTAGE = DIRECT ? 2 : ring_depth(BM, BN, TERMS);
  using Cfg =
      wmmae_gemm::GemmConfig<MT, TERMS, BM, BN, WGM, WGN, NSTAGE, RN, DIRECT>;
  auto kernel = wmmae_gemm::tcec_gemm_kernel<MT, TERMS, BM, BN, WGM, WGN,
                                             NSTAGE, RN, DIRECT>;
  static std::atomic<unsigned long long> lds_allowed{0};
  WMMAE_HIP_TRY(allow_dynamic_lds(reinterpret_cast<const void *>(kernel),
                                  Cfg::LDS_BYTES, lds_allowed));
  const int tiles_m = static_cast<int>(ceil_div(g.m, BM));
  const int tiles_n = static_cast<int>(ceil_div(g.n, BN));
  const int KT = packed_k_tiles(g.k);
  const int rb_a = static_cast<int>(packed_row_blocks(g.m));
  const int rb_b = static_cast<int>(packed_row_blocks(g.n));
  // 16-byte stores need ldc % 4 == 0 and an aligned base; the base of each
  // batch entry is checked again inside the kernel
  const int vec_store =
      (g.ldc % 4 == 0) &&
      (g.c_ptrs != nullptr || (reinterpret_cast<uintptr_t>(g.c) % 16 == 0 &&
                               g.stride_c % 4 == 0));
  const int splits = g.partial != nullptr ? g.splits : 1;
  const int split_stages = static_cast<int>(ceil_div(KT, splits));
  const int zdim = static_cast<int>(ceil_div(KT, split_stages));
  const long long items =
      static_cast<long long>(tiles_m) * tiles_n * g.batch * zdim;
  if (items >= (1ll << 31)) // the kernel counts items in 32 bits
    return WMMAE_STATUS_INVALID_VALUE;
  // Who takes which item (the large tiles take most of a compute unit's LDS,
  // so one workgroup per unit is resident):
  //  * 8 or more batch entries: an XCD owns whole entries, so that an entry's
  //    operands are read into one L2 only (batch 256 of 1024x1024x256:
  //    196 -> 256 effective TFLOPS), persistent workgroups when there are
  //    more items than resident workgroups;
  // and with more items than resident workgroups otherwise
  //  * short K loops: persistent workgroups walking one shared list, their
  //    requests running ahead into the next item;
  //  * long K loops (64 stages = 2048 of k or more per item) of few entries:
  //    one workgroup per item, handed out by the hardware as compute units
  //    become free, which evens out compute units of unequal speed over many
  //    rounds (a fixed share per workgroup measured 7 % slower at 16384^3).
  const int per_cu =
      workgroups_per_cu<MT, TERMS, BM, BN, WGM, WGN, RN, DIRECT>();
  const long long resident = static_cast<long long>(device_cus()) * per_cu;
  int grid = static_cast<int>(std::min(items, resident));
  int entry_per_xcd = 0;
  const bool eight_xcds = device_xcds() == kKernelXcds;
  if (zdim > 1 && eight_xcds && resident >= 8 && resident % 8 == 0) {
    // split-K: eight runs of the item list, one per XCD, so that an XCD holds
    // as few K slices as possible; the grid is padded to whole runs
    entry_per_xcd = 2;
    grid = static_cast<int>(std::min(8 * ceil_div(items, 8), resident));
  }
  unsigned tail_begin = 0xffffffffu; // no tail slices
  TailPlan tail;
  // (an XCD that owns one entry more than the others must not cost more
  // rounds than the shared list would take: 9 entries of 128 tiles are 8
  // rounds on the XCD with two entries, 5 on the shared list)
  const bool by_xcd = eight_xcds && resident >= 8 && resident % 8 == 0;
  const long long owned_rounds =
      by_xcd ? ceil_div(static_cast<long long>(tiles_m) * tiles_n *
                            ceil_div(g.batch, 8),
                        resident / 8)
             : 0;
  if (zdim == 1 && g.batch >= 8 && by_xcd &&
      owned_rounds * 100 <= ceil_div(items, resident) * 115) {
    // also when every item gets a workgroup of its own: a workgroup for every
    // item of the XCD that owns the most entries
    entry_per_xcd = 1;
    grid = static_cast<int>(std::min(
        8ll * tiles_m * tiles_n * ceil_div(g.batch, 8), resident));
  } else if (items > resident && entry_per_xcd == 0) {
    if (split_stages >= 64) {
      grid = static_cast<int>(items);
      // one entry, no split-K, room for the slices: the tiles of a partly
      // empty last round are cut along K
      if (g.batch == 1 && zdim == 1 && g.c_ptrs == nullptr &&
          g.tail_ws != nullptr) {
        tail = plan_tail(items, resident, KT);
        const size_t need =
            static_cast<size_t>(tail.slices) * tail.tail * BM * BN * 4u;
        if (tail.slices >= 2 && need <= g.tail_ws_bytes) {
          tail_begin = static_cast<unsigned>(tail.full);
          grid = static_cast<int>(tail.full + tail.tail * tail.slices);
        } else {
          tail.slices = 1;
        }
      }
    }
  }
  if (t_gemm_begin != nullptr)
    WMMAE_HIP_TRY(hipEventRecord(t_gemm_begin, g.stream));
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(Cfg::NTHREADS), Cfg::LDS_BYTES,
                     g.stream, g.a, g.b,
                     g.c, g.m, g.n, KT, rb_a, rb_b, g.ldc, g.alpha, g.beta,
                     g.inv_scale, tiles_m, tiles_n, vec_store,
                     static_cast<long long>(rb_a) * KT * TERMS * 64,
                     static_cast<long long>(rb_b) * KT * TERMS * 64,
                     g.stride_c, split_stages,
                     zdim > 1 ? g.partial : static_cast<float *>(nullptr),
                     g.c_ptrs, g.batch, zdim, entry_per_xcd, tail_begin,
                     tail.stages, g.tail_ws, g.direct);
  int st = launch_status();
  if (st == WMMAE_STATUS_SUCCESS && tail_begin != 0xffffffffu) {
    hipLaunchKernelGGL((wmmae_gemm::reduce_tail_kernel<BM, BN>),
                       dim3(static_cast<unsigned>(tail.tail), BM * BN / 1024),
                       dim3(256), 0, g.stream, g.tail_ws, tail.slices,
                       tail_begin, static_cast<unsigned>(tiles_m * tiles_n),
                       tiles_m, tiles_n, g.c, g.m, g.n, g.ldc, g.alpha, g.beta);
    st = launch_status();
  }
  if (st == WMMAE_STATUS_SUCCESS && zdim > 1) {
    // 16 bytes per access where every slice column and every column of C starts
    // on a 16-byte boundary (entries of a pointer array: not known here)
    const bool vec = g.m % 4 == 0 && g.ldc % 4 == 0 && g.c_ptrs == nullptr &&
                     reinterpret_cast<uintptr_t>(g.c) % 16 == 0 &&
                     g.stride_c % 4 == 0 &&
                     reinterpret_cast<uintptr_t>(g.partial) % 16 == 0;
    const long long blocks =
        ceil_div(static_cast<long long>(g.m) * g.n, vec ? 1024 : 256);
    for (int e0 = 0; e0 < g.batch; e0 += kMaxGridY) {
      const dim3 grid(static_cast<unsigned>(blocks),
                      std::min(g.batch - e0, kMaxGridY));
      if (vec)
        hipLaunchKernelGGL(wmmae_gemm::reduce_splits_kernel<4>, grid, dim3(256),
                           0, g.stream, g.partial, zdim, g.c, g.m, g.n, g.ldc,
                           g.stride_c, g.c_ptrs, g.alpha, g.beta,
                           static_cast<long long>(g.batch),
                           static_cast<unsigned>(e0));
      else
        hipLaunchKernelGGL(wmmae_gemm::reduce_splits_kernel<1>, grid, dim3(256),
                           0, g.stream, g.partial, zdim, g.c, g.m, g.n, g.ldc,
                           g.stride_c, g.c_ptrs, g.alpha, g.beta,
                           static_cast<long long>(g.batch),
                           static_cast<unsigned>(e0));
    }
    st = launch_status();
  }
  if (st == WMMAE_STATUS_SUCCESS && t_gemm_end != nullptr)
    WMMAE_HIP_TRY(hipEventRecord(t_gemm_end, g.stream));
  return st;
}

// Tile choice: the 256x128 tile moves the fewest operand bytes per flop and is
// the choice whenever its rounds cost less; the tiles run in rounds
// of one per compute unit, so when the last round would be mostly empty the
// 128x128 tile (5 to 25 % slower per flop) can still finish sooner; 64x64
// tiles for problems too small to give the larger ones work.
template <class MT, int TERMS, bool RN> int gemm_by_size(const GemmArgs &g) {
  const int cus = device_cus();
  const long long z = g.partial != nullptr ? g.splits : 1;
  const long long big =
      ceil_div(g.m, 256) * ceil_div(g.n, 128) * g.batch * z;
  const long long mid =
      ceil_div(g.m, 128) * ceil_div(g.n, 128) * g.batch * z;
  if constexpr (TERMS <= 2 && !RN) {
    // (k a multiple of 32, or the variant with a shorter last stage)
    if (g.is_direct)
      return g.k % 32 == 0 ? launch_gemm<MT, TERMS, 256, 128, 2, 2, RN, 1>(g)
                           : launch_gemm<MT, TERMS, 256, 128, 2, 2, RN, 2>(g);
  }
  // (not with the separate fp32 adds of RN: their temporaries do not fit the
  // register file next to the large tile's accumulators)
  if constexpr (!RN) {
    const int KT = packed_k_tiles(g.k);
    if (big_tile_candidate(TERMS, mid, static_cast<int>(ceil_div(KT, z)))) {
      // time in units of one 128x128 tile: rounds * tile cost
      const bool tail_ok = g.batch == 1 && z == 1 && g.c_ptrs == nullptr &&
                           g.tail_ws != nullptr;
      const double t_big =
          rounds_cost(big, cus, KT, tail_ok) * fit::units256x128(TERMS);
      // (a 128x128 tile measured at 1.2 to 1.25 times half a 256x128 tile in
      // runs of two to eight rounds, 1.05 in long ones)
      const double t_mid =
          rounds_cost(mid, cus, KT, tail_ok) * fit::units128x128(TERMS);
      if (t_big <= t_mid)
        return launch_gemm<MT, TERMS, 256, 128, 2, 2, RN>(g);
    }
  }
  if (mid >= cus || (g.m > 64 && g.n > 64))
    return launch_gemm<MT, TERMS, 128, 128, 2, 2, RN>(g);
  return launch_gemm<MT, TERMS, 64, 64, 2, 2, RN>(g);
}

int gemm_dispatch(const int policy, const int flags, const GemmArgs &g) {
  const bool rn = (flags & WMMAE_FLAG_RN_MAIN) != 0;
  switch (policy) {
  case WMMAE_POLICY_F16_EC:
    return rn ? gemm_by_size<_Float16, 2, true>(g)
              : gemm_by_size<_Float16, 2, false>(g);
  case WMMAE_POLICY_F16_NOEC:
    return rn ? WMMAE_STATUS_NOT_SUPPORTED
              : gemm_by_size<_Float16, 1, false>(g);
  case WMMAE_POLICY_BF16X3_EC:
    return rn ? gemm_by_size<__bf16, 3, true>(g)
              : gemm_by_size<__bf16, 3, false>(g);
  case WMMAE_POLICY_BF16X2_EC:
    return rn ? WMMAE_STATUS_NOT_SUPPORTED
              : gemm_by_size<__bf16, 2, false>(g);
  case WMMAE_POLICY_BF16_NOEC:
    return rn ? WMMAE_STATUS_NOT_SUPPORTED : gemm_by_size<__bf16, 1, false>(g);
  default:
    return WMMAE_STATUS_INVALID_VALUE;
  }
}

// Resident workgroups per compute unit of the packed kernel a policy runs with
// tile shape 0 (256x128), 1 (128x128) or 2 (64x64): the number launch_gemm
// plans its rounds with, for the workspace query.
template <class MT, int TERMS> int per_cu_by_shape(const int shape) {
  switch (shape) {
  case 0:
    return workgroups_per_cu<MT, TERMS, 256, 128, 2, 2, false>();
  case 1:
    return workgroups_per_cu<MT, TERMS, 128, 128, 2, 2, false>();
  default:
    return workgroups_per_cu<MT, TERMS, 64, 64, 2, 2, false>();
  }
}
int per_cu_of(const int policy, const int shape) {
  switch (policy) {
  case WMMAE_POLICY_F16_EC:
    return per_cu_by_shape<_Float16, 2>(shape);
  case WMMAE_POLICY_F16_NOEC:
    return per_cu_by_shape<_Float16, 1>(shape);
  case WMMAE_POLICY_BF16X3_EC:
    return per_cu_by_shape<__bf16, 3>(shape);
  case WMMAE_POLICY_BF16X2_EC:
    return per_cu_by_shape<__bf16, 2>(shape);
  default:
    return per_cu_by_shape<__bf16, 1>(shape);
  }
}

// ------------------------------------------------------ fused small GEMM
struct FusedArgs {
  wmmae_gemm::FusedParams p;
  hipStream_t stream;
};

template <class T, int TERMS, int BM, int BN> int launch_fused(FusedArgs f) {
  using Cfg = wmmae_gemm::FusedConfig<TERMS, BM, BN>;
  auto kernel = wmmae_gemm::tcec_gemm_fused_kernel<T, TERMS, BM, BN>;
  static std::atomic<unsigned long long> lds_allowed{0};
  WMMAE_HIP_TRY(allow_dynamic_lds(reinterpret_cast<const void *>(kernel),
                                  Cfg::LDS_BYTES, lds_allowed));
  wmmae_gemm::FusedParams &p = f.p;
  p.tiles_m = static_cast<int>(ceil_div(p.M, BM));
  p.tiles_per_batch = p.tiles_m * static_cast<int>(ceil_div(p.N, BN));
  // one persistent workgroup per compute unit at most; with 8 or more batch
  // entries an XCD (block index mod 8) owns whole entries
  const int per_xcd_max = device_cus() / 8 > 0 ? device_cus() / 8 : 1;
  // (not when the XCD that owns one entry more than the others would need
  // over 15 % more rounds of tiles than an even spread)
  const long long all_tiles =
      static_cast<long long>(p.batch) * p.tiles_per_batch;
  p.grouped =
      device_xcds() == kKernelXcds && p.batch >= 8 &&
      ceil_div(ceil_div(p.batch, 8) * p.tiles_per_batch, per_xcd_max) * 100 <=
          ceil_div(all_tiles, 8ll * per_xcd_max) * 115;
  long long per_xcd = p.grouped
                          ? ceil_div(p.batch, 8) * p.tiles_per_batch
                          : ceil_div(static_cast<long long>(p.batch) *
                                         p.tiles_per_batch,
                                     8);
  if (per_xcd > per_xcd_max)
    per_xcd = per_xcd_max;
  const int grid = 8 * static_cast<int>(per_xcd);
  hipLaunchKernelGGL(kernel, dim3(grid), dim3(Cfg::NTHREADS), Cfg::LDS_BYTES,
                     f.stream,
                     p);
  return launch_status();
}

// 128x128 tiles, unless they leave compute units without work and 64x64 tiles
// (four times as many workgroups; one takes 0.65 of a 128x128 tile's time at
// these latency-bound sizes) finish sooner: 1024^3 went from 41 to 27 us.
inline bool fused_small_tiles(const int m, const int n, const int batch) {
  const long long cus = device_cus();
  const long long tiles128 = ceil_div(m, 128) * ceil_div(n, 128) * batch;
  const long long tiles64 = ceil_div(m, 64) * ceil_div(n, 64) * batch;
  return (m <= 64 && n <= 64) ||
         (tiles128 < cus && fit::kFusedSmallTileTime *
                                    static_cast<double>(ceil_div(tiles64, cus)) <
                                static_cast<double>(ceil_div(tiles128, cus)));
}
template <class T, int TERMS> int fused_by_size(const FusedArgs &f) {
  if (fused_small_tiles(f.p.M, f.p.N, f.p.batch))
    return launch_fused<T, TERMS, 64, 64>(f);
  return launch_fused<T, TERMS, 128, 128>(f);
}

int fused_dispatch(const int policy, const FusedArgs &f) {
  switch (policy) {
  case WMMAE_POLICY_F16_EC:
    return fused_by_size<w::half, 2>(f);
  case WMMAE_POLICY_F16_NOEC:
    return fused_by_size<w::half, 1>(f);
  case WMMAE_POLICY_BF16X3_EC:
    return fused_by_size<w::precision::tf32, 3>(f);
  case WMMAE_POLICY_BF16X2_EC:
    return fused_by_size<w::bfloat16, 2>(f);
  case WMMAE_POLICY_BF16_NOEC:
    return fused_by_size<w::bfloat16, 1>(f);
  default:
    return WMMAE_STATUS_INVALID_VALUE;
  }
}

// Which of the three paths?  The single ("fused") kernel moves only the fp32
// operands and C but needs about twice as long per 128x128x32 tile step and
// converts every element once per wave that uses it; the packed path first
// writes and re-reads the split operands, which pays off when every operand
// element is used by many tiles; the "direct" path is the packed path's GEMM
// kernel (256x128 tiles) loading the fp32 operands itself and splitting them
// on their way into LDS - no packed copy and no split pass, at 1.2 to 1.9
// times the time per k stage; it wins where an operand element is used by
// few tiles (batches of small and medium matrices, K-heavy products) and
// needs k contiguous in both operands, k at least 4 and at most two terms;
// same bits as the packed path.  All three times are estimated with the same
// shape, a launch cost plus rounds of tiles over the compute units times (k
// stages * time per stage + time per tile), bounded below by the bytes moved;
// products that are cut into K slices take the slice planner's time, rescaled.
// The constants and what they were fitted to: namespace fit.
// fused_vec: the fused kernel can request 16 bytes per lane from both
// operands (k contiguous, k and the strides multiples of 4, aligned bases).
// Without that it issues four times as many requests (3.5 times the time per
// stage), so such products take another path unless k is very short.
enum class Path { Fused, Packed, Direct };
// (see PathRates::busy)
inline double busy_factor(const fit::PathRates &r, const long long tiles) {
  const long long cus = device_cus();
  return 1.0 + r.busy * static_cast<double>(tiles) /
                   static_cast<double>(ceil_div(tiles, cus) * cus);
}
// the direct kernel's time without K slices: rounds of 256x128 tiles over the
// compute units, and the bytes it moves
struct DirectTimes {
  double tiles, bytes;
};
inline DirectTimes direct_times(const int m, const int n, const int k,
                                const int batch, const fit::PathRates &d) {
  const double kt = static_cast<double>(ceil_div(k, 32));
  const long long tiles256 = ceil_div(m, 256) * ceil_div(n, 128) * batch;
  const double ab = (static_cast<double>(m) + n) * k * batch;
  // (the variant for k % 32 != 0 spends one more instruction per load)
  const double stage = d.stage * busy_factor(d, tiles256) *
                       (k % 32 == 0 ? 1.0 : fit::kDirectTailStage);
  return {fit::kUnits256x128 *
              static_cast<double>(ceil_div(tiles256, device_cus())) *
              (kt * stage + d.tile),
          (4.0 * m * n * batch + 4.0 * ab) / d.bytes_per_s};
}
constexpr int kPathFlags =
    WMMAE_FLAG_PATH_PACKED | WMMAE_FLAG_PATH_FUSED | WMMAE_FLAG_PATH_DIRECT;
constexpr int kAllFlags = WMMAE_FLAG_RN_MAIN | kPathFlags;
inline bool one_path_at_most(const int flags) {
  const int f = flags & kPathFlags;
  return (f & (f - 1)) == 0;
}
// Estimated time of a call on each path, in seconds; a path that cannot run
// the product (or is not considered for it) has infinity.
struct PathEstimates {
  double fused, packed, direct;
};
inline PathEstimates estimate_paths(const int m, const int n, const int k,
                                    const int batch, const int terms,
                                    const bool fused_vec, const bool direct_ok) {
  constexpr double kNever = std::numeric_limits<double>::infinity();
  PathEstimates e{kNever, kNever, kNever};
  const fit::PathRates &f = fit::kFused[terms - 1], &p = fit::kPacked[terms - 1];
  const long long cus = device_cus();
  const int kti = static_cast<int>(ceil_div(k, 32));
  const double kt = static_cast<double>(kti);
  const double c_bytes = 4.0 * m * n * batch;
  const double ab = (static_cast<double>(m) + n) * k * batch; // operand elements
  const long long tiles64 = ceil_div(m, 64) * ceil_div(n, 64) * batch;
  const long long tiles128 = ceil_div(m, 128) * ceil_div(n, 128) * batch;
  const long long tiles256 = ceil_div(m, 256) * ceil_div(n, 128) * batch;

  // fused kernel: 128x128 tiles, or 64x64 ones (a third of the stage time,
  // half of the per-tile time) under fused_by_size's rule
  if (fused_vec || k <= 96) {
    const bool small = fused_small_tiles(m, n, batch);
    const long long f_tiles = small ? tiles64 : tiles128;
    const double f_rounds = static_cast<double>(ceil_div(f_tiles, cus));
    e.fused =
        f.launch +
        std::max(f_rounds * (kt * f.stage * busy_factor(f, f_tiles) *
                                 (fused_vec ? 1.0 : fit::kFusedNarrowRequests) *
                                 (small ? fit::kFusedSmallStage : 1.0) +
                             f.tile * (small ? fit::kFusedSmallTile : 1.0)),
                 (c_bytes + 4.0 * ab) / f.bytes_per_s);
  }
  const double split_pass = (4.0 + 2.0 * terms) * ab / p.split_bytes_per_s;
  const int splits = choose_splits(terms, m, n, k, batch);
  if (splits != 1) {
    // K slices: the split pass and the packed kernel's slices against the
    // slower stages of the direct kernel (cut into the slices that suit its own
    // tile)
    e.fused = e.fused * fit::kSlicedFused[0][terms - 1] +
              fit::kSlicedFused[1][terms - 1];
    e.packed = (p.launch + split_pass +
                split_time(terms, m, n, batch, kti, splits)) *
                   fit::kSlicedPacked[0][terms - 1] +
               fit::kSlicedPacked[1][terms - 1];
    if (direct_ok)
      e.direct =
          (fit::kDirect[terms - 1].launch +
           split_time(terms, m, n, batch, kti,
                      choose_splits(terms, m, n, k, batch, true), true)) *
              fit::kSlicedDirect[0][terms - 1] +
          fit::kSlicedDirect[1][terms - 1];
    return e;
  }
  // packed path: rounds in units of one 128x128 tile as gemm_by_size counts
  // them (a 256x128 tile 2.0 and a 128x128 tile 1.2 for one and two terms,
  // 1.8 and 1.0 for three, a 64x64 tile 0.4)
  double units;
  long long p_tiles;
  const double r128 = static_cast<double>(ceil_div(tiles128, cus));
  if (big_tile_candidate(terms, tiles128, kti) &&
      fit::units256x128(terms) * static_cast<double>(ceil_div(tiles256, cus)) <=
          fit::units128x128(terms) * r128) {
    units = fit::units256x128(terms) *
            static_cast<double>(ceil_div(tiles256, cus));
    p_tiles = tiles256;
  } else if (tiles128 >= cus || (m > 64 && n > 64)) {
    units = r128 * fit::units128x128(terms);
    p_tiles = tiles128;
  } else {
    units = fit::kUnits64x64 * static_cast<double>(ceil_div(tiles64, cus));
    p_tiles = tiles64;
  }
  e.packed = p.launch + split_pass +
             std::max(units * (kt * p.stage * busy_factor(p, p_tiles) + p.tile),
                      c_bytes / p.bytes_per_s);
  if (direct_ok) {
    const DirectTimes d =
        direct_times(m, n, k, batch, fit::kDirect[terms - 1]);
    // (it cuts K for its own tile even where the packed path would not)
    const int own = choose_splits(terms, m, n, k, batch, true);
    e.direct =
        own > 1 ? (fit::kDirect[terms - 1].launch +
                   split_time(terms, m, n, batch, kti, own, true)) *
                          fit::kSlicedDirect[0][terms - 1] +
                      fit::kSlicedDirect[1][terms - 1]
                : fit::kDirect[terms - 1].launch + std::max(d.tiles, d.bytes);
  }
  return e;
}
inline Path choose_path(const int m, const int n, const int k, const int batch,
                        const int flags, const int terms, const int policy,
                        const bool fused_vec, const bool direct_ok) {
  // (the round-to-nearest flag with a policy that has no such variant is
  // turned down by the packed path's dispatch)
  const bool rn_unsupported =
      (flags & WMMAE_FLAG_RN_MAIN) != 0 && policy != WMMAE_POLICY_F16_EC &&
      policy != WMMAE_POLICY_BF16X3_EC;
  if (k <= 0 || rn_unsupported)
    return Path::Packed;
  PathEstimates e = estimate_paths(m, n, k, batch, terms, fused_vec, direct_ok);
  e.fused = std::max(e.fused, fit::kCallFloor[0]);
  e.packed = std::max(e.packed, fit::kCallFloor[1]);
  e.direct = std::max(e.direct, fit::kCallFloor[2]);
  Path best = Path::Packed;
  double t_best = e.packed;
  if (e.fused < t_best) {
    t_best = e.fused;
    best = Path::Fused;
  }
  if (e.direct < t_best)
    best = Path::Direct;
  return best;
}
// what the direct kernel needs of a product (the operands' k strides are 1)
inline bool direct_possible(const int k, const int terms, const int flags,
                            const long long a_rs, const long long b_rs) {
  return k >= 4 && terms <= 2 &&
         (flags & WMMAE_FLAG_RN_MAIN) == 0 && a_rs < (1 << 24) &&
         b_rs < (1 << 24);
}

inline bool is_n(const char t) { return t == 'N' || t == 'n'; }
inline bool is_t(const char t) {
  return t == 'T' || t == 't' || t == 'C' || t == 'c';
}

} // namespace

// ===========================================================================
extern "C" {

const char *wmmae_status_string(const int status) {
  switch (status) {
  case WMMAE_STATUS_SUCCESS:
    return "success";
  case WMMAE_STATUS_INVALID_VALUE:
    return "invalid value";
  case WMMAE_STATUS_NULL_POINTER:
    return "null pointer";
  case WMMAE_STATUS_BAD_LEADING_DIM:
    return "leading dimension too small";
  case WMMAE_STATUS_NOT_SUPPORTED:
    return "not supported";
  case WMMAE_STATUS_WORKSPACE_TOO_SMALL:
    return "workspace too small";
  case WMMAE_STATUS_RUNTIME_ERROR:
    return "HIP runtime error";
  case WMMAE_STATUS_MISALIGNED:
    return "buffer not 16-byte aligned";
  default:
    return "unknown status";
  }
}

int wmmae_query(const int what, long long *const out) {
  if (out == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  if (what == 0) {
    *out = 100; // 0.1.0
    return WMMAE_STATUS_SUCCESS;
  }
  if (what == 3) {
    *out = 5;
    return WMMAE_STATUS_SUCCESS;
  }
  if (what == 1 || what == 2) {
    int dev = 0;
    hipDeviceProp_t prop;
    WMMAE_HIP_TRY(hipGetDevice(&dev));
    WMMAE_HIP_TRY(hipGetDeviceProperties(&prop, dev));
    *out = what == 1 ? prop.multiProcessorCount : prop.clockRate;
    return WMMAE_STATUS_SUCCESS;
  }
  return WMMAE_STATUS_INVALID_VALUE;
}

// ------------------------------------------------------------- pack / gemm
int wmmae_tcec_pack_bytes(const int rows, const int k, const int batch,
                          const int policy, size_t *const bytes) {
  PolicyInfo p;
  if (bytes == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  if (!policy_info(policy, p) || rows < 0 || k < 0 || batch < 0)
    return WMMAE_STATUS_INVALID_VALUE;
  *bytes = static_cast<size_t>(packed_elems(rows, k, p.terms)) * 16u *
           static_cast<size_t>(batch);
  return WMMAE_STATUS_SUCCESS;
}

} // extern "C"

namespace {
// Shared implementations; X / C may be given as a base pointer with a batch
// stride or as a device array of per-matrix pointers.
// Argument checks of one operand of a split; WMMAE_STATUS_SUCCESS with
// `nothing` set when there is nothing to write.
int pack_check(const int policy, const int rows, const int k,
               const float *const X, const float *const *const ptrs,
               const long long row_stride, const long long k_stride,
               const int batch, void *const packed, const size_t packed_bytes,
               bool &nothing) {
  PolicyInfo p;
  nothing = false;
  if (!policy_info(policy, p) || rows < 0 || k < 0 || batch < 0)
    return WMMAE_STATUS_INVALID_VALUE;
  if (rows == 0 || k == 0 || batch == 0) {
    nothing = true;
    return WMMAE_STATUS_SUCCESS;
  }
  if ((X == nullptr && ptrs == nullptr) || packed == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  if (row_stride < 1 || k_stride < 1 || (row_stride != 1 && k_stride != 1))
    return WMMAE_STATUS_BAD_LEADING_DIM;
  if (reinterpret_cast<uintptr_t>(packed) % 16 != 0)
    return WMMAE_STATUS_MISALIGNED;
  size_t need = 0;
  wmmae_tcec_pack_bytes(rows, k, batch, policy, &need);
  if (packed_bytes < need)
    return WMMAE_STATUS_WORKSPACE_TOO_SMALL;
  return WMMAE_STATUS_SUCCESS;
}

int pack_impl(const int policy, const int rows, const int k,
              const float *const X, const float *const *const ptrs,
              const long long row_stride, const long long k_stride,
              const long long batch_stride, const int batch, void *const packed,
              const size_t packed_bytes, void *const stream) {
  bool nothing = false;
  const int st = pack_check(policy, rows, k, X, ptrs, row_stride, k_stride,
                            batch, packed, packed_bytes, nothing);
  if (st != WMMAE_STATUS_SUCCESS || nothing)
    return st;
  const PackSource src{rows, X, ptrs, row_stride, k_stride, batch_stride, packed};
  return pack_dispatch(policy, k, batch, src, nullptr,
                       static_cast<hipStream_t>(stream));
}

// split-K, or K slices for a partly empty last round, only when the caller
// supplied room for the slices
void plan_k_slices(GemmArgs &g, void *const workspace,
                   const size_t workspace_bytes) {
  g.splits = choose_splits(g.terms, g.m, g.n, g.k, g.batch, g.is_direct);
  g.partial = nullptr;
  g.tail_ws = nullptr;
  g.tail_ws_bytes = 0;
  const bool ws_usable =
      workspace != nullptr && reinterpret_cast<uintptr_t>(workspace) % 16 == 0;
  if (g.splits > 1 && ws_usable &&
      workspace_bytes >=
          static_cast<size_t>(g.splits) * g.batch * g.m * g.n * 4u) {
    g.partial = static_cast<float *>(workspace);
  } else {
    g.splits = 1;
    if (ws_usable) {
      g.tail_ws = static_cast<float *>(workspace);
      g.tail_ws_bytes = workspace_bytes;
    }
  }
}

int gemm_packed_impl(const int policy, const int m, const int n, const int k,
                     const float *const alpha, const void *const packed_a,
                     const void *const packed_b, const float *const beta,
                     float *const C, float *const *const c_ptrs, const int ldc,
                     const long long stride_c, const int batch, const int flags,
                     void *const workspace, const size_t workspace_bytes,
                     void *const stream) {
  PolicyInfo p;
  if (!policy_info(policy, p) || m < 0 || n < 0 || k < 0 || batch < 0 ||
      (flags & ~WMMAE_FLAG_RN_MAIN) != 0)
    return WMMAE_STATUS_INVALID_VALUE;
  if (alpha == nullptr || beta == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  if (m == 0 || n == 0 || batch == 0)
    return WMMAE_STATUS_SUCCESS;
  if ((C == nullptr && c_ptrs == nullptr) ||
      (k > 0 && (packed_a == nullptr || packed_b == nullptr)))
    return WMMAE_STATUS_NULL_POINTER;
  if (ldc < m)
    return WMMAE_STATUS_BAD_LEADING_DIM;
  if (k > 0 && (reinterpret_cast<uintptr_t>(packed_a) % 16 != 0 ||
                reinterpret_cast<uintptr_t>(packed_b) % 16 != 0))
    return WMMAE_STATUS_MISALIGNED;
  if (k == 0) {
    const long long blocks = ceil_div(static_cast<long long>(m) * n, 256);
    if (blocks > 0x7fffffffLL)
      return WMMAE_STATUS_NOT_SUPPORTED;
    for (int e0 = 0; e0 < batch; e0 += kMaxGridY)
      hipLaunchKernelGGL(wmmae_gemm::scale_c_kernel,
                         dim3(static_cast<unsigned>(blocks),
                              std::min(batch - e0, kMaxGridY)),
                         dim3(256), 0, static_cast<hipStream_t>(stream), C, m, n,
                         static_cast<long long>(ldc), stride_c, c_ptrs, *beta,
                         static_cast<unsigned>(e0));
    return launch_status();
  }
  GemmArgs g;
  g.a = static_cast<const u32x4 *>(packed_a);
  g.b = static_cast<const u32x4 *>(packed_b);
  g.c = C;
  g.c_ptrs = c_ptrs;
  g.m = m;
  g.n = n;
  g.k = k;
  g.ldc = ldc;
  g.stride_c = stride_c;
  g.alpha = *alpha;
  g.beta = *beta;
  g.inv_scale = p.inv_scale;
  g.batch = batch;
  g.terms = p.terms;
  g.stream = static_cast<hipStream_t>(stream);
  plan_k_slices(g, workspace, workspace_bytes);
  return gemm_dispatch(policy, flags, g);
}

int sgemm_impl(const char transa, const char transb, const int m, const int n,
               const int k, const float *const alpha, const float *const A,
               const float *const *const a_ptrs, const int lda,
               const long long stride_a, const float *const B,
               const float *const *const b_ptrs, const int ldb,
               const long long stride_b, const float *const beta,
               float *const C, float *const *const c_ptrs, const int ldc,
               const long long stride_c, const int batch, const int policy,
               const int flags, void *workspace, const size_t workspace_bytes,
               void *const stream) {
  PolicyInfo p;
  if ((!is_n(transa) && !is_t(transa)) || (!is_n(transb) && !is_t(transb)) ||
      m < 0 || n < 0 || k < 0 || batch < 0 || !policy_info(policy, p) ||
      (flags & ~kAllFlags) != 0 || !one_path_at_most(flags))
    return WMMAE_STATUS_INVALID_VALUE;
  if (alpha == nullptr || beta == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  if (m == 0 || n == 0 || batch == 0)
    return WMMAE_STATUS_SUCCESS;
  if ((C == nullptr && c_ptrs == nullptr) ||
      (k > 0 && ((A == nullptr && a_ptrs == nullptr) ||
                 (B == nullptr && b_ptrs == nullptr))))
    return WMMAE_STATUS_NULL_POINTER;
  const int a_rows = is_n(transa) ? m : k; // rows of A as stored (column major)
  const int b_rows = is_n(transb) ? k : n;
  if (lda < (a_rows > 1 ? a_rows : 1) || ldb < (b_rows > 1 ? b_rows : 1) ||
      ldc < m)
    return WMMAE_STATUS_BAD_LEADING_DIM;

  const auto aligned16 = [](const void *ptr) {
    return reinterpret_cast<uintptr_t>(ptr) % 16 == 0;
  };
  // 16-byte requests of the fused kernel (entries of pointer arrays are
  // checked by the kernel itself)
  const long long a_rs = is_n(transa) ? 1 : lda, a_ks = is_n(transa) ? lda : 1;
  const long long b_rs = is_n(transb) ? ldb : 1, b_ks = is_n(transb) ? 1 : ldb;
  const bool vec_a = a_ks == 1 && k % 4 == 0 && a_rs % 4 == 0 &&
                     (a_ptrs != nullptr || (aligned16(A) && stride_a % 4 == 0));
  const bool vec_b = b_ks == 1 && k % 4 == 0 && b_rs % 4 == 0 &&
                     (b_ptrs != nullptr || (aligned16(B) && stride_b % 4 == 0));
  const bool direct_ok = a_ks == 1 && b_ks == 1 &&
                         direct_possible(k, p.terms, flags, a_rs, b_rs);
  const int rn = flags & WMMAE_FLAG_RN_MAIN;
  Path path = choose_path(m, n, k, batch, rn, p.terms, policy, vec_a && vec_b,
                          direct_ok);
  if ((flags & WMMAE_FLAG_PATH_DIRECT) != 0) {
    if (!direct_ok)
      return WMMAE_STATUS_NOT_SUPPORTED;
    path = Path::Direct;
  } else if ((flags & WMMAE_FLAG_PATH_FUSED) != 0) {
    if (k <= 0 || (rn != 0 && policy != WMMAE_POLICY_F16_EC &&
                   policy != WMMAE_POLICY_BF16X3_EC))
      return WMMAE_STATUS_NOT_SUPPORTED;
    path = Path::Fused;
  } else if ((flags & WMMAE_FLAG_PATH_PACKED) != 0) {
    path = Path::Packed;
  }
  if (path == Path::Direct) {
    // the planes of the K slices are the only workspace this path uses
    size_t bytes_c = 0;
    wmmae_tcec_gemm_packed_workspace_bytes(policy, m, n, k, batch, &bytes_c);
    hipStream_t s = static_cast<hipStream_t>(stream);
    void *ws = workspace;
    size_t ws_bytes = workspace_bytes;
    bool own = false;
    // (a caller's workspace that is not 16-byte aligned is left alone by
    // plan_k_slices: this path can do without, as the single kernel does)
    if (ws == nullptr && bytes_c > 0) {
      WMMAE_HIP_TRY(hipMallocAsync(&ws, bytes_c, s));
      ws_bytes = bytes_c;
      own = true;
    }
    GemmArgs g;
    g.a = nullptr;
    g.b = nullptr;
    g.c = C;
    g.c_ptrs = c_ptrs;
    g.m = m;
    g.n = n;
    g.k = k;
    g.ldc = ldc;
    g.stride_c = stride_c;
    g.alpha = *alpha;
    g.beta = *beta;
    g.inv_scale = p.inv_scale;
    g.batch = batch;
    g.terms = p.terms;
    g.stream = s;
    g.is_direct = true;
    g.direct = wmmae_gemm::DirectSource{A,    B,    a_ptrs,   b_ptrs,
                                        a_rs, b_rs, stride_a, stride_b, 0, k};
    plan_k_slices(g, ws, ws_bytes);
    // staggered start for launches bound by their bytes (see the kernel)
    const DirectTimes dt =
        direct_times(m, n, k, batch, fit::kDirectStagger[p.terms - 1]);
    if (g.splits <= 1 && batch >= 8 && dt.bytes > dt.tiles)
      g.direct.stagger = 1;
    int st = gemm_dispatch(policy, 0, g);
    if (own && hipFreeAsync(ws, s) != hipSuccess && st == WMMAE_STATUS_SUCCESS)
      st = WMMAE_STATUS_RUNTIME_ERROR;
    return st;
  }
  if (path == Path::Fused) {
    if (batch > (1 << 26)) // tile indices are 32-bit
      return WMMAE_STATUS_NOT_SUPPORTED;
    FusedArgs f;
    wmmae_gemm::FusedParams &q = f.p;
    q.A = A;
    q.a_ptrs = a_ptrs;
    q.a_rs = a_rs;
    q.a_ks = a_ks;
    q.a_bs = stride_a;
    q.B = B;
    q.b_ptrs = b_ptrs;
    q.b_rs = b_rs;
    q.b_ks = b_ks;
    q.b_bs = stride_b;
    q.C = C;
    q.c_ptrs = c_ptrs;
    q.ldc = ldc;
    q.c_bs = stride_c;
    q.M = m;
    q.N = n;
    q.K = k;
    q.batch = batch;
    q.vec_a = vec_a;
    q.vec_b = vec_b;
    q.vec_store = (ldc % 4 == 0) &&
                  (c_ptrs != nullptr || (aligned16(C) && stride_c % 4 == 0));
    q.rn_main = (flags & WMMAE_FLAG_RN_MAIN) != 0;
    q.alpha = *alpha;
    q.beta = *beta;
    q.inv_scale = p.inv_scale;
    f.stream = static_cast<hipStream_t>(stream);
    return fused_dispatch(policy, f);
  }

  size_t bytes_a = 0, bytes_b = 0, bytes_c = 0;
  wmmae_tcec_pack_bytes(m, k, batch, policy, &bytes_a);
  wmmae_tcec_pack_bytes(n, k, batch, policy, &bytes_b);
  wmmae_tcec_gemm_packed_workspace_bytes(policy, m, n, k, batch, &bytes_c);
  hipStream_t s = static_cast<hipStream_t>(stream);
  bool own = false;
  if (workspace == nullptr) {
    if (bytes_a + bytes_b + bytes_c > 0) {
      WMMAE_HIP_TRY(hipMallocAsync(&workspace, bytes_a + bytes_b + bytes_c, s));
      own = true;
    }
  } else {
    if (reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
      return WMMAE_STATUS_MISALIGNED;
    // the packed operands are required; the split-K slices are optional
    if (workspace_bytes < bytes_a + bytes_b)
      return WMMAE_STATUS_WORKSPACE_TOO_SMALL;
    if (workspace_bytes < bytes_a + bytes_b + bytes_c)
      bytes_c = 0;
  }
  void *const pa = workspace;
  void *const pb = static_cast<char *>(workspace) + bytes_a;
  void *const pc =
      bytes_c > 0 ? static_cast<char *>(workspace) + bytes_a + bytes_b : nullptr;

  int st = WMMAE_STATUS_SUCCESS;
  if (k > 0) {
    // op(A)(i,l): 'N' -> A[i + l*lda], 'T' -> A[l + i*lda]
    const PackSource sa{m, A, a_ptrs, is_n(transa) ? 1 : lda,
                        is_n(transa) ? lda : 1, stride_a, pa};
    // op(B)(l,j): 'N' -> B[l + j*ldb], 'T' -> B[j + l*ldb]; packed rows = j
    const PackSource sb{n, B, b_ptrs, is_n(transb) ? ldb : 1,
                        is_n(transb) ? 1 : ldb, stride_b, pb};
    bool none_a = false, none_b = false;
    st = pack_check(policy, sa.rows, k, sa.X, sa.ptrs, sa.row_stride,
                    sa.k_stride, batch, pa, bytes_a, none_a);
    if (st == WMMAE_STATUS_SUCCESS)
      st = pack_check(policy, sb.rows, k, sb.X, sb.ptrs, sb.row_stride,
                      sb.k_stride, batch, pb, bytes_b, none_b);
    // (m, n, k and batch are all positive here: both operands have work)
    if (st == WMMAE_STATUS_SUCCESS && !none_a && !none_b)
      st = pack_dispatch(policy, k, batch, sa, &sb, s); // one launch for both
  }
  if (st == WMMAE_STATUS_SUCCESS)
    st = gemm_packed_impl(policy, m, n, k, alpha, pa, pb, beta, C, c_ptrs, ldc,
                          stride_c, batch, flags & WMMAE_FLAG_RN_MAIN, pc, bytes_c,
                          stream);
  if (own) {
    if (hipFreeAsync(workspace, s) != hipSuccess &&
        st == WMMAE_STATUS_SUCCESS)
      st = WMMAE_STATUS_RUNTIME_ERROR;
  }
  return st;
}
} // namespace

extern "C" {

int wmmae_tcec_pack(const int policy, const int rows, const int k,
                    const float *const X, const long long row_stride,
                    const long long k_stride, const long long batch_stride,
                    const int batch, void *const packed,
                    const size_t packed_bytes, void *const stream) {
  return pack_impl(policy, rows, k, X, nullptr, row_stride, k_stride,
                   batch_stride, batch, packed, packed_bytes, stream);
}

int wmmae_tcec_gemm_packed(const int policy, const int m, const int n,
                           const int k, const float *const alpha,
                           const void *const packed_a,
                           const void *const packed_b, const float *const beta,
                           float *const C, const int ldc,
                           const long long stride_c, const int batch,
                           const int flags, void *const workspace,
                           const size_t workspace_bytes, void *const stream) {
  return gemm_packed_impl(policy, m, n, k, alpha, packed_a, packed_b, beta, C,
                          nullptr, ldc, stride_c, batch, flags, workspace,
                          workspace_bytes, stream);
}

int wmmae_tcec_gemm_packed_workspace_bytes(const int policy, const int m,
                                           const int n, const int k,
                                           const int batch,
                                           size_t *const bytes) {
  PolicyInfo p;
  if (bytes == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  if (!policy_info(policy, p) || m < 0 || n < 0 || k < 0 || batch < 0)
    return WMMAE_STATUS_INVALID_VALUE;
  // (room for the slices of either kernel: the one that splits the fp32
  // operands itself plans them for its own tile)
  const int splits =
      (m == 0 || n == 0 || k == 0 || batch == 0)
          ? 1
          : std::max(choose_splits(p.terms, m, n, k, batch),
                     direct_possible(k, p.terms, 0, 1, 1)
                         ? choose_splits(p.terms, m, n, k, batch, true)
                         : 1);
  if (splits > 1) {
    *bytes = static_cast<size_t>(splits) * batch * m * n * 4u;
  } else if (batch == 1 && m > 0 && n > 0) {
    // K slices of the tiles of a partly empty last round: the largest need
    // over the tile shapes and residencies the launch may choose
    const int KT = packed_k_tiles(k);
    size_t need = 0;
    const int shapes[3][2] = {{256, 128}, {128, 128}, {64, 64}};
    for (int i = 0; i < 3; i++) {
      const int *const sh = shapes[i];
      const int per_cu = per_cu_of(policy, i);
      const TailPlan t =
          plan_tail(ceil_div(m, sh[0]) * ceil_div(n, sh[1]),
                    static_cast<long long>(device_cus()) * per_cu, KT);
      if (t.slices >= 2)
        need = std::max<size_t>(need, static_cast<size_t>(t.slices) *
                                          static_cast<size_t>(t.tail) * sh[0] *
                                          sh[1] * 4u);
    }
    *bytes = need;
  } else {
    *bytes = 0;
  }
  return WMMAE_STATUS_SUCCESS;
}

int wmmae_tcec_sgemm_path(const int m, const int n, const int k,
                          const int batch, const int policy, const int flags,
                          int *const path) {
  PolicyInfo p;
  if (path == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  if (m < 0 || n < 0 || k < 0 || batch < 0 || !policy_info(policy, p) ||
      (flags & ~WMMAE_FLAG_RN_MAIN) != 0)
    return WMMAE_STATUS_INVALID_VALUE;
  const bool any = m > 0 && n > 0 && k > 0 && batch > 0;
  const bool slices = any && choose_splits(p.terms, m, n, k, batch) > 1;
  switch (choose_path(m, n, k, batch, flags, p.terms, policy, k % 4 == 0,
                      direct_possible(k, p.terms, flags, 1, 1))) {
  case Path::Fused:
    *path = 0;
    break;
  case Path::Direct:
    *path = any && choose_splits(p.terms, m, n, k, batch, true) > 1 ? 4 : 3;
    break;
  default:
    *path = slices ? 2 : 1;
  }
  return WMMAE_STATUS_SUCCESS;
}

int wmmae_tcec_path_estimates(const int m, const int n, const int k,
                              const int batch, const int policy,
                              double *const seconds) {
  PolicyInfo p;
  if (seconds == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  if (m <= 0 || n <= 0 || k <= 0 || batch <= 0 || !policy_info(policy, p))
    return WMMAE_STATUS_INVALID_VALUE;
  const PathEstimates e = estimate_paths(m, n, k, batch, p.terms, k % 4 == 0,
                                         direct_possible(k, p.terms, 0, 1, 1));
  seconds[0] = e.fused;
  seconds[1] = e.packed;
  seconds[2] = e.direct;
  return WMMAE_STATUS_SUCCESS;
}

int wmmae_tcec_time_gemm_kernel(void *const begin_event,
                                void *const end_event) {
  if ((begin_event == nullptr) != (end_event == nullptr))
    return WMMAE_STATUS_NULL_POINTER;
  t_gemm_begin = static_cast<hipEvent_t>(begin_event);
  t_gemm_end = static_cast<hipEvent_t>(end_event);
  return WMMAE_STATUS_SUCCESS;
}

int wmmae_tcec_force_k_slices(const int slices) {
  if (slices < 0)
    return WMMAE_STATUS_INVALID_VALUE;
  t_forced_k_slices = slices;
  return WMMAE_STATUS_SUCCESS;
}

int wmmae_tcec_sgemm_k_slices(const int m, const int n, const int k,
                              const int batch, const int policy,
                              const int flags, int *const slices) {
  PolicyInfo p;
  if (slices == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  constexpr int kPathFlags = WMMAE_FLAG_PATH_PACKED | WMMAE_FLAG_PATH_FUSED |
                             WMMAE_FLAG_PATH_DIRECT;
  if (m < 0 || n < 0 || k < 0 || batch < 0 || !policy_info(policy, p) ||
      (flags & ~(WMMAE_FLAG_RN_MAIN | kPathFlags)) != 0)
    return WMMAE_STATUS_INVALID_VALUE;
  *slices = 1;
  if (m == 0 || n == 0 || k == 0 || batch == 0)
    return WMMAE_STATUS_SUCCESS;
  const bool direct_ok = direct_possible(k, p.terms, flags, 1, 1);
  Path path = choose_path(m, n, k, batch, flags & WMMAE_FLAG_RN_MAIN, p.terms,
                          policy, k % 4 == 0, direct_ok);
  if ((flags & WMMAE_FLAG_PATH_DIRECT) != 0) {
    if (!direct_ok)
      return WMMAE_STATUS_NOT_SUPPORTED;
    path = Path::Direct;
  } else if ((flags & WMMAE_FLAG_PATH_FUSED) != 0) {
    path = Path::Fused;
  } else if ((flags & WMMAE_FLAG_PATH_PACKED) != 0) {
    path = Path::Packed;
  }
  if (path != Path::Fused)
    *slices = choose_splits(p.terms, m, n, k, batch, path == Path::Direct);
  return WMMAE_STATUS_SUCCESS;
}

int wmmae_tcec_sgemm_workspace_bytes(const int m, const int n, const int k,
                                     const int batch, const int policy,
                                     size_t *const bytes) {
  size_t a = 0, b = 0, c = 0;
  if (bytes == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  if (m < 0 || n < 0)
    return WMMAE_STATUS_INVALID_VALUE;
  int s = wmmae_tcec_pack_bytes(m, k, batch, policy, &a);
  if (s != WMMAE_STATUS_SUCCESS)
    return s;
  s = wmmae_tcec_pack_bytes(n, k, batch, policy, &b);
  if (s != WMMAE_STATUS_SUCCESS)
    return s;
  s = wmmae_tcec_gemm_packed_workspace_bytes(policy, m, n, k, batch, &c);
  if (s != WMMAE_STATUS_SUCCESS)
    return s;
  *bytes = a + b + c;
  return WMMAE_STATUS_SUCCESS;
}

int wmmae_tcec_sgemm_strided_batched(
    const char transa, const char transb, const int m, const int n, const int k,
    const float *const alpha, const float *const A, const int lda,
    const long long stride_a, const float *const B, const int ldb,
    const long long stride_b, const float *const beta, float *const C,
    const int ldc, const long long stride_c, const int batch, const int policy,
    const int flags, void *const workspace, const size_t workspace_bytes,
    void *const stream) {
  return sgemm_impl(transa, transb, m, n, k, alpha, A, nullptr, lda, stride_a,
                    B, nullptr, ldb, stride_b, beta, C, nullptr, ldc, stride_c,
                    batch, policy, flags, workspace, workspace_bytes, stream);
}

int wmmae_tcec_sgemm_batched(const char transa, const char transb, const int m,
                             const int n, const int k, const float *const alpha,
                             const float *const *const A_array, const int lda,
                             const float *const *const B_array, const int ldb,
                             const float *const beta,
                             float *const *const C_array, const int ldc,
                             const int batch, const int policy, const int flags,
                             void *const workspace,
                             const size_t workspace_bytes,
                             void *const stream) {
  return sgemm_impl(transa, transb, m, n, k, alpha, nullptr, A_array, lda, 0,
                    nullptr, B_array, ldb, 0, beta, nullptr, C_array, ldc, 0,
                    batch, policy, flags, workspace, workspace_bytes, stream);
}

int wmmae_direct_read_first(const int tail, const int k, const int stage,
                            const int lane, long long *const first) {
  if (first == nullptr)
    return WMMAE_STATUS_NULL_POINTER;
  if (k < 4 || stage < 0 || stage >= ceil_div(k, 32) || lane < 0 || lane > 63 ||
      (tail == 0 && k % 32 != 0))
    return WMMAE_STATUS_INVALID_VALUE;
  *first = wmmae_gemm::direct_read_first(tail != 0, k, stage,
                                         static_cast<unsigned>(lane));
  return WMMAE_STATUS_SUCCESS;
}

// ---------------------------------------------- entry point that allocates
// nothing: the workspace is a device array that is part of the library image.
// Each GPU holds its own copy at its own address; in host code the array's
// name is only a handle for hipGetSymbolAddress, never a device address.
} // extern "C"

namespace {
constexpr size_t kStaticScratchBytes = WMMAE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on the current device, looked up once per
// device (with that device current) and kept.
int static_scratch(void **const out) {
  static std::atomic<void *> ptrs[64];
  int dev = 0;
  WMMAE_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64)
    return WMMAE_STATUS_NOT_SUPPORTED;
  void *p = ptrs[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    WMMAE_HIP_TRY(
        hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch)));
    if (p == nullptr)
      return WMMAE_STATUS_RUNTIME_ERROR;
    ptrs[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return WMMAE_STATUS_SUCCESS;
}
} // namespace

extern "C" {

int wmmae_tcec_sgemm_static(const char transa, const char transb, const int m,
                            const int n, const int k, const float *const alpha,
                            const float *const A, const int lda,
                            const float *const B, const int ldb,
                            const float *const beta, float *const C,
                            const int ldc, const int policy, const int flags,
                            void *const stream) {
  void *ws = nullptr;
  const int st = static_scratch(&ws);
  if (st != WMMAE_STATUS_SUCCESS)
    return st;
  // sgemm_impl allocates only when it is handed no workspace; with one it
  // returns WMMAE_STATUS_WORKSPACE_TOO_SMALL when the split operands do not
  // fit, and makes K slices only if they fit as well
  return sgemm_impl(transa, transb, m, n, k, alpha, A, nullptr, lda, 0, B,
                    nullptr, ldb, 0, beta, C, nullptr, ldc, 0, 1, policy, flags,
                    ws, kStaticScratchBytes, stream);
}

int wmmae_tcec_sgemm(const char transa, const char transb, const int m,
                     const int n, const int k, const float *const alpha,
                     const float *const A, const int lda, const float *const B,
                     const int ldb, const float *const beta, float *const C,
                     const int ldc, const int policy, const int flags,
                     void *const workspace, const size_t workspace_bytes,
                     void *const stream) {
  return sgemm_impl(transa, transb, m, n, k, alpha, A, nullptr, lda, 0, B,
                    nullptr, ldb, 0, beta, C, nullptr, ldc, 0, 1, policy, flags,
                    workspace, workspace_bytes, stream);
}

} // extern "C"
