// Byte-copy engine behind putmem/getmem at thread, wavefront, work-group and
// grid granularity.
//
// Replaces the reference's memcpy / memcpy_wg / memcpy_wave
// (src/util.hpp:170-262), which move 8 bytes per lane per iteration through
// cache-bypassing flat stores and make three strided passes (8/4/2 bytes) plus
// a one-byte tail.  Here a cooperating group of lanes peels the destination to
// 16-byte alignment, streams 16 bytes per lane per step with several loads in
// flight (the source may sit at any byte offset — gfx950 global loads need no
// alignment), and finishes the sub-16-byte tail with byte moves.  All stores
// are write-through buffer stores (see below); bulk copies add the
// non-temporal hint on both sides.
//
// The result is a byte-exact copy of [src, src+n) to [dst, dst+n) for every n
// and every pair of alignments.  The reference's work-group and wavefront
// loops leave the last byte of an odd-sized message (n >= 3) uncopied because
// the tail move reuses a stale pointer (src/util.hpp:203-223); that defect is
// not reproduced.
#ifndef ROCSHMEM_AMD_DETAIL_COPY_ENGINE_HPP_
#define ROCSHMEM_AMD_DETAIL_COPY_ENGINE_HPP_

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace rocshmem {
namespace detail {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_any __attribute__((aligned(1)));
typedef uint64_t u64_any __attribute__((aligned(1)));
typedef uint32_t u32_any __attribute__((aligned(1)));
typedef uint16_t u16_any __attribute__((aligned(1)));

// Messages at least this large are moved with the non-temporal hint.
constexpr size_t kNonTemporalBytes = size_t{4} << 10;

// ---- write-through stores ---------------------------------------------------
// Every store of a cooperative copy or fold goes out as a buffer store with
// the sc1 (agent scope, write-through) bit.  The L2 of the issuing XCD then
// holds no dirty lines for the message, so the release that follows a put
// (quiet, fence, the signal of put_signal, a barrier) has nothing to write
// back: measured on MI355X, 16384 work-groups each ending in a release cost
// 0.48 ms extra after plain or non-temporal stores and 0.03 ms after sc1
// stores, at the same store bandwidth.  (8-byte atomic stores, the other way
// to get sc1 from the compiler, run 4.6x slower.)
//
// A buffer resource covers at most 4 GiB and must be wave-uniform; callers
// pass the same destination in every lane (the _wg/_wave calling convention).
constexpr int kAuxWriteThrough = 16;             // sc1
constexpr int kAuxWriteThroughStreaming = 16 | 2;  // sc1 nt
constexpr size_t kWindowBytes = size_t{1} << 30;   // bytes addressed per resource

__device__ __forceinline__ __amdgpu_buffer_rsrc_t window_of(const void *base, size_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(a));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(a >> 32));
  void *uniform = reinterpret_cast<void *>((static_cast<uint64_t>(hi) << 32) | lo);
  const uint32_t range = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bytes));
  return __builtin_amdgcn_make_buffer_rsrc(uniform, 0, static_cast<int>(range), 0x00020000);
}

template <bool kNonTemporal>
__device__ __forceinline__ void store16(__amdgpu_buffer_rsrc_t w, uint32_t off, u32x4 v) {
  __builtin_amdgcn_raw_buffer_store_b128(
      v, w, static_cast<int>(off), 0, kNonTemporal ? kAuxWriteThroughStreaming : kAuxWriteThrough);
}
__device__ __forceinline__ void store1(__amdgpu_buffer_rsrc_t w, uint32_t off, uint8_t v) {
  __builtin_amdgcn_raw_buffer_store_b8(v, w, static_cast<int>(off), 0, kAuxWriteThrough);
}

template <bool kNonTemporal>
__device__ __forceinline__ u32x4 load16(const char *p) {
  if constexpr (kNonTemporal) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4_any *>(p));
  } else {
    return *reinterpret_cast<const u32x4_any *>(p);
  }
}

// Copy n <= kWindowBytes bytes with `nlanes` cooperating lanes; this lane is
// number `lane` (0-based, dense).  Lanes need not belong to one wavefront or
// work-group: a whole grid can call this with global thread ids.
template <int kUnroll, bool kNonTemporal>
__device__ __forceinline__ void copy_window(char *dst, const char *src, size_t n, size_t lane,
                                            size_t nlanes) {
  const __amdgpu_buffer_rsrc_t w = window_of(dst, n);
  size_t head = (16u - (reinterpret_cast<uintptr_t>(dst) & 15u)) & 15u;
  if (head > n) head = n;
  for (size_t k = lane; k < head; k += nlanes) store1(w, static_cast<uint32_t>(k), src[k]);
  src += head;
  const size_t body = n - head;
  const uint32_t base = static_cast<uint32_t>(head);

  const size_t nvec = body >> 4;
  size_t i = lane;
  if constexpr (kUnroll > 1) {
    // Two batches of kUnroll vectors: the loads of the next batch are issued
    // before the stores of the current one, so a lane always has loads in
    // flight while it waits.
    const size_t span = static_cast<size_t>(kUnroll) * nlanes;
    if (i + span - nlanes < nvec) {
      u32x4 v[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        v[u] = load16<kNonTemporal>(src + ((i + u * nlanes) << 4));
      for (i += span; i + span - nlanes < nvec; i += span) {
        u32x4 next[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
          next[u] = load16<kNonTemporal>(src + ((i + u * nlanes) << 4));
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
          store16<kNonTemporal>(w, base + static_cast<uint32_t>((i - span + u * nlanes) << 4), v[u]);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) v[u] = next[u];
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u)
        store16<kNonTemporal>(w, base + static_cast<uint32_t>((i - span + u * nlanes) << 4), v[u]);
    }
  }
  for (; i < nvec; i += nlanes)
    store16<kNonTemporal>(w, base + static_cast<uint32_t>(i << 4),
                          load16<kNonTemporal>(src + (i << 4)));

  const size_t done = nvec << 4;
  const size_t tail = body - done;
  for (size_t k = lane; k < tail; k += nlanes)
    store1(w, base + static_cast<uint32_t>(done + k), src[done + k]);
}

// Any size: 1 GiB windows, one buffer resource each.
template <int kUnroll, bool kNonTemporal>
__device__ __forceinline__ void copy_lanes_impl(char *dst, const char *src, size_t n, size_t lane,
                                                size_t nlanes) {
  while (n > kWindowBytes) {
    copy_window<kUnroll, kNonTemporal>(dst, src, kWindowBytes, lane, nlanes);
    dst += kWindowBytes;
    src += kWindowBytes;
    n -= kWindowBytes;
  }
  copy_window<kUnroll, kNonTemporal>(dst, src, n, lane, nlanes);
}

// kLoads: 16-byte vectors per batch; the loop keeps two batches per lane (the
// next one loading while the current one is stored), which measured 3 % more
// for a put_signal dispatch of 900 KB messages and 17 % more for a lone
// wavefront than one batch at a time.  Batches of 4 saturate a CU when a full
// work-group copies (batches of 2 lose 10-40 %); a lone wavefront needs 8 to
// cover the memory latency.  The register count of a kernel is that of its
// widest path (about 100 VGPRs with batches of 4, the limit of 128 for a
// 1024-lane work-group with batches of 8), so the deeper variant is chosen
// per call site, not at run time.
template <int kLoads = 4>
__device__ __forceinline__ void copy_lanes(void *dst, const void *src, size_t n, size_t lane,
                                           size_t nlanes,
                                           size_t nt_bytes = kNonTemporalBytes) {
  char *d = static_cast<char *>(dst);
  const char *s = static_cast<const char *>(src);
  if (n >= nt_bytes) {
    copy_lanes_impl<kLoads, true>(d, s, n, lane, nlanes);
  } else {
    copy_lanes_impl<kLoads, false>(d, s, n, lane, nlanes);
  }
}

// One lane copies n bytes on its own: 16-byte moves, then 8/4/2/1.  A lone
// lane is bound by memory latency, so large messages keep eight loads in
// flight (measured: 1 MiB from one thread in 7 ms with one load at a time).
__device__ __forceinline__ void copy_thread(void *dst, const void *src,
                                            size_t n) {
  char *d = static_cast<char *>(dst);
  const char *s = static_cast<const char *>(src);
  while (n >= 128) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const u32x4_any *>(s + 16 * u);
#pragma unroll
    for (int u = 0; u < 8; ++u) *reinterpret_cast<u32x4_any *>(d + 16 * u) = v[u];
    d += 128; s += 128; n -= 128;
  }
  while (n >= 16) {
    *reinterpret_cast<u32x4_any *>(d) = *reinterpret_cast<const u32x4_any *>(s);
    d += 16; s += 16; n -= 16;
  }
  if (n & 8) {
    *reinterpret_cast<u64_any *>(d) = *reinterpret_cast<const u64_any *>(s);
    d += 8; s += 8;
  }
  if (n & 4) {
    *reinterpret_cast<u32_any *>(d) = *reinterpret_cast<const u32_any *>(s);
    d += 4; s += 4;
  }
  if (n & 2) {
    *reinterpret_cast<u16_any *>(d) = *reinterpret_cast<const u16_any *>(s);
    d += 2; s += 2;
  }
  if (n & 1) *d = *s;
}

// Rank of this lane among the currently active lanes of its wavefront, and
// the number of active lanes.  The reference strides by the active-lane count
// but indexes by the raw lane id (src/util.hpp:226-262), which skips data when
// the active lanes are not the lowest ones; ranking the active lanes is
// correct for any mask.
__device__ __forceinline__ unsigned active_lane_rank(unsigned *count) {
  const unsigned long long mask = __ballot(1);
  const unsigned lo = static_cast<unsigned>(mask);
  const unsigned hi = static_cast<unsigned>(mask >> 32);
  *count = __popcll(mask);
  return __builtin_amdgcn_mbcnt_hi(hi, __builtin_amdgcn_mbcnt_lo(lo, 0u));
}

__device__ __forceinline__ void copy_wave(void *dst, const void *src, size_t n,
                                          size_t nt_bytes = kNonTemporalBytes) {
  unsigned count;
  const unsigned rank = active_lane_rank(&count);
  copy_lanes<8>(dst, src, n, rank, count, nt_bytes);
}

}  // namespace detail
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_DETAIL_COPY_ENGINE_HPP_
