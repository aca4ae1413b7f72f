// Utilities next to the fragment API: element cast and asynchronous
// global -> LDS copies (reference: include/wmma_extension/utils.hpp:21-64,
// where the copies are cp.async on sm_80 and plain loads elsewhere).
//
// gfx950 has a direct global -> LDS load (global_load_lds_dword / _dwordx4):
// the data bypasses the registers, the wave goes on, and completion is
// tracked by the wave's vector-memory counter.  Its LDS address is not per
// lane: lane l of the wave writes `base + l*Size`.  cp_async<Size>(smem, gmem)
// keeps the reference's per-lane signature and uses the direct load whenever
// the destinations of the active lanes have exactly that shape (the usual
// `smem + threadIdx.x`), which it checks at run time with one ballot; any other
// destination pattern, and Size == 8 (no such direct load), is served by a
// load through registers, which is complete when cp_async returns.
#pragma once
#include "detail/common.hpp"
#include <cstdint>

namespace mtk {
namespace wmma {
namespace utils {

// cast<DST_T>(v): v converted to the storage type of tag DST_T, round to
// nearest even (reference: utils.hpp:21-26).
template <class DST_T, class SRC_T>
WMMAE_HD typename mtk::wmma::detail::common::storage_t<DST_T>::type
cast(const SRC_T v) {
  return mtk::wmma::detail::common::cast<DST_T>(v);
}

namespace cp_async {

namespace detail {
// Group bookkeeping of one wave, kept in LDS (wave w of the workgroup owns
// row w): [0] direct global -> LDS loads issued so far, [1] commits so far,
// [2 + c % kGroupRing] the value of [0] at commit c.  The hardware counts the
// wave's outstanding vector-memory instructions, oldest first, so "at most N
// groups pending" is "at most ([0] now) - ([0] at the N-th last commit)
// instructions outstanding".  Only differences of these words are ever used,
// so the LDS need not be initialised: with fewer than N commits behind it,
// wait_group<N> reads a stale word and waits for more than it has to or for
// nothing, and both are correct then.
// The words are read and written with LDS instructions the compiler does not
// see as such (inline assembly): before an LDS read it knows of, it waits for
// every direct global -> LDS load in flight, and the bookkeeping of a copy must
// not wait for the copy.
constexpr unsigned kGroupRing = 8;
// LDS byte address of the calling wave's words
WMMAE_D uint32_t group_state() {
  __shared__ uint32_t state[16][2 + kGroupRing];
  const unsigned tid =
      threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z);
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) void *)state[(tid >> 6) & 15u]));
}
// [0] += 1, by the first active lane
WMMAE_D void count_issue() {
  const uint32_t s = group_state();
  const uint32_t lane = mtk::wmma::detail::common::get_lane_id();
  if (lane == __builtin_amdgcn_readfirstlane(lane))
    asm volatile("ds_add_u32 %0, %1" ::"v"(s), "v"(1u) : "memory");
}
// words [0] and [1]; every active lane reads the same
WMMAE_D void read_counts(const uint32_t s, uint32_t &issued,
                         uint32_t &commits) {
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  u32x2 v;
  asm volatile("ds_read2_b32 %0, %1 offset1:1\n\ts_waitcnt lgkmcnt(0)"
               : "=v"(v)
               : "v"(s)
               : "memory");
  issued = v[0];
  commits = v[1];
}
// s_waitcnt vmcnt(t) for a wave-uniform t in [LO, HI]
template <int LO, int HI> WMMAE_D void wait_vmcnt(const uint32_t t) {
  if constexpr (LO == HI) {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LO) : "memory");
  } else {
    constexpr int MID = (LO + HI) / 2;
    if (t <= static_cast<uint32_t>(MID))
      wait_vmcnt<LO, MID>(t);
    else
      wait_vmcnt<MID + 1, HI>(t);
  }
}
} // namespace detail

// Copy Size bytes (4, 8 or 16) per lane from global memory to LDS.  `smem` and
// `gmem` must be Size-aligned.  The data is visible to the calling wave after
// wait_all() / wait_group<N>() / wait_pending<N>(), to the workgroup after a
// barrier that follows it.
template <unsigned Size>
WMMAE_D void cp_async(void *const smem, const void *const gmem) {
  static_assert(Size == 4 || Size == 8 || Size == 16,
                "Size must be one of 4, 8 and 16");
  if constexpr (Size == 4 || Size == 16) {
    // LDS byte address of this lane's destination, and the base it implies
    const uint32_t dst = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (__attribute__((address_space(3))) void *)smem));
    const uint32_t lane = mtk::wmma::detail::common::get_lane_id();
    const uint32_t base = dst - lane * Size;
    const uint32_t base0 = __builtin_amdgcn_readfirstlane(base);
    // every active lane agrees on the base <=> destinations are lane-linear
    const bool linear =
        __builtin_amdgcn_ballot_w64(base != base0) == 0 && (base0 % Size) == 0;
    if (linear) {
      const auto g = (const __attribute__((address_space(1))) void *)gmem;
      const auto l = (__attribute__((address_space(3))) void *)(uintptr_t)base0;
      if constexpr (Size == 4)
        __builtin_amdgcn_global_load_lds(g, l, 4, 0, 0);
      else
        __builtin_amdgcn_global_load_lds(g, l, 16, 0, 0);
      detail::count_issue();
      return;
    }
  }
#pragma unroll
  for (unsigned i = 0; i < Size / 4; i++)
    reinterpret_cast<uint32_t *>(smem)[i] =
        reinterpret_cast<const uint32_t *>(gmem)[i];
}

// The same copy for callers whose destinations are lane-linear by
// construction: lane l of the wave passes smem = (wave's base) + l*Size, with
// a Size-aligned base - e.g. `tile + Size/4 * threadIdx.x` for a float tile.
// This is the native shape of the gfx950 instruction; nothing is checked, so
// the wave issues the load at once (cp_async spends about fifteen scalar and
// vector instructions and a branch per call on finding this out at run time,
// measured at 15 % of a GEMM that stages its tiles with it).  No counterpart
// in the reference.  Size 4 or 16.
template <unsigned Size>
WMMAE_D void cp_async_lane_linear(void *const smem, const void *const gmem) {
  static_assert(Size == 4 || Size == 16, "Size must be 4 or 16");
  const uint32_t dst = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) void *)smem));
  // the first active lane's destination names the wave's base
  const uint32_t lane = mtk::wmma::detail::common::get_lane_id();
  const uint32_t base0 = __builtin_amdgcn_readfirstlane(dst - lane * Size);
  const auto g = (const __attribute__((address_space(1))) void *)gmem;
  const auto l = (__attribute__((address_space(3))) void *)(uintptr_t)base0;
  if constexpr (Size == 4)
    __builtin_amdgcn_global_load_lds(g, l, 4, 0, 0);
  else
    __builtin_amdgcn_global_load_lds(g, l, 16, 0, 0);
}

// Close the group of the copies issued since the last commit()
// (reference: utils.hpp:46-50, cp.async.commit_group).
WMMAE_D void commit() {
  const uint32_t s = detail::group_state();
  uint32_t issued, commits;
  detail::read_counts(s, issued, commits);
  commits += 1u;
  // (every active lane writes the same two words)
  asm volatile("ds_write_b32 %0, %1 offset:8\n\tds_write_b32 %2, %3 offset:4" ::"v"(
                   s + 4u * (commits % detail::kGroupRing)),
               "v"(issued), "v"(s), "v"(commits)
               : "memory");
}

// All copies issued by this wave have landed in LDS.  The compiler may not
// move instructions across the wait in either direction: arithmetic that
// touches registers only (the MFMAs of the stage being multiplied while the
// next one is copied) would otherwise be free to sink below it, which turns
// "copy while computing" into "copy, then compute".
WMMAE_D void wait_all() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

// At most the N most recently committed groups of cp_async copies are still
// pending (reference: utils.hpp:58-62, cp.async.wait_group N; N <= 7 here).
// Copies issued after the last commit() stay pending as well.  The hardware
// counter also holds the wave's other vector-memory instructions (ordinary
// loads and stores issued since), so with those in between the wait can be
// longer than needed, never shorter.  The copies made by cp_async_lane_linear
// are not counted: code that uses them knows its group sizes and waits with
// wait_pending.
template <int N> WMMAE_D void wait_group() {
  static_assert(N >= 0 && N < static_cast<int>(detail::kGroupRing),
                "at most 7 groups can be left pending");
  if constexpr (N == 0) {
    wait_all();
  } else {
    const uint32_t s = detail::group_state();
    uint32_t issued, commits, then;
    detail::read_counts(s, issued, commits);
    asm volatile("ds_read_b32 %0, %1 offset:8\n\ts_waitcnt lgkmcnt(0)"
                 : "=v"(then)
                 : "v"(s + 4u * ((commits - N) % detail::kGroupRing))
                 : "memory");
    const uint32_t allowed = __builtin_amdgcn_readfirstlane(issued - then);
    __builtin_amdgcn_sched_barrier(0);
    // (more than 63 instructions are never outstanding)
    if (allowed < 64u)
      detail::wait_vmcnt<0, 63>(allowed);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// At most N of this wave's copies (vector-memory instructions, oldest first)
// are still in flight: wait_group<N / G> for code that knows it issues G copies
// per group, without the bookkeeping.
template <int N> WMMAE_D void wait_pending() {
  static_assert(N >= 0 && N <= 63, "the counter has 6 bits");
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
  __builtin_amdgcn_sched_barrier(0);
}

} // namespace cp_async
} // namespace utils
} // namespace wmma
} // namespace mtk
