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

// Group bookkeeping is done by the hardware counter; nothing to do here.
WMMAE_D void commit() {}

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

// The reference waits until at most N committed groups are pending.  The
// hardware counts instructions, not groups, and a group may hold any number
// of copies, so the only bound that is always safe is zero.  Code that knows
// its group size uses wait_pending instead.
template <int N> WMMAE_D void wait_group() { wait_all(); }

// At most N of this wave's cp_async calls (vector-memory instructions, oldest
// first) are still in flight.  With G calls per group this is the reference's
// wait_group<N / G>.
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
