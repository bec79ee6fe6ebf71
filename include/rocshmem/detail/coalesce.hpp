// Wavefront message coalescing: neighbouring lanes whose messages continue
// one another (same PE, same size, source and destination each advanced by
// exactly that size) are merged into the lowest lane of the run.
//
// Result-compatible with the reference's WfCoalOn::coalesce
// (src/wf_coal_policy.cpp:57-172): a lane is absorbed iff it is not lane 0,
// the lane below is active, and that lane's (pe, size, src+size, dst+size)
// match; every other active lane is a sender whose size grows by one message
// per absorbed lane directly above it.  As there, the neighbour's size is
// compared through 32 bits.  Neighbour values travel by DPP wave_shr:1
// instead of ds_bpermute-based shuffles, and the run length comes from the
// ballot of absorbed lanes.
//
// Merging a run into the lowest lane's serial copy would slow a load/store
// path down; what the thread-level put does with a run instead is move it with
// the whole wavefront (detail/rma.hpp::put_as_one_run).
#ifndef ROCSHMEM_AMD_DETAIL_COALESCE_HPP_
#define ROCSHMEM_AMD_DETAIL_COALESCE_HPP_

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace rocshmem {
namespace detail {

#if defined(__HIPCC__)

// Value of `v` in the next lower lane of the wavefront; lane 0 and lanes whose
// lower neighbour is inactive get their own value back.
__device__ __forceinline__ uint32_t from_lower_lane(uint32_t v) {
  constexpr int kWaveShr1 = 0x138;
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(
      static_cast<int>(v), static_cast<int>(v), kWaveShr1, 0xf, 0xf, false));
}
__device__ __forceinline__ uint64_t from_lower_lane64(uint64_t v) {
  const uint32_t lo = from_lower_lane(static_cast<uint32_t>(v));
  const uint32_t hi = from_lower_lane(static_cast<uint32_t>(v >> 32));
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// Returns true when the calling lane must send; *size is then the merged size.
__device__ __forceinline__ bool wf_coalesce(int pe, const void *source, const void *dest,
                                            size_t *size) {
  const uint64_t src = reinterpret_cast<uint64_t>(source);
  const uint64_t dst = reinterpret_cast<uint64_t>(dest);
  const uint64_t my_size = *size;

  const uint64_t lower_src = from_lower_lane64(src);
  const uint64_t lower_dst = from_lower_lane64(dst);
  const int lower_pe = static_cast<int>(from_lower_lane(static_cast<uint32_t>(pe)));
  const uint64_t lower_size = from_lower_lane(static_cast<uint32_t>(my_size));

  const uint64_t active = __ballot(1);
  const unsigned lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));

  const bool absorbed = lane != 0 && ((active >> (lane - 1)) & 1ull) &&
                        lower_size == my_size && lower_src + my_size == src &&
                        lower_dst + my_size == dst && lower_pe == pe;
  const uint64_t absorbed_mask = __ballot(absorbed);
  if (!absorbed) {
    // Count the unbroken run of absorbed lanes directly above this one.
    const uint64_t above = lane == 63 ? 0ull : (absorbed_mask >> (lane + 1));
    const unsigned run = static_cast<unsigned>(__ffsll(static_cast<long long>(~above))) - 1u;
    *size = my_size + my_size * run;
  }
  return !absorbed;
}

#endif  // __HIPCC__

}  // namespace detail
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_DETAIL_COALESCE_HPP_
