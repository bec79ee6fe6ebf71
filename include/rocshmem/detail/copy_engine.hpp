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
// The same from a pointer known to name device (global) memory, split into a
// wave-uniform base and a 32-bit byte offset per lane: a global_load with the
// base in scalar registers and one address register.  A load through a
// generic pointer is a flat instruction, which the hardware may also route to
// LDS or scratch; the compiler then has to wait for all outstanding memory
// operations before it uses the result, and the pipelining below is lost.
typedef const __attribute__((address_space(1))) char *GlobalBytes;
typedef const __attribute__((address_space(1))) u32x4_any *GlobalVec;
template <bool kNonTemporal>
__device__ __forceinline__ u32x4 load16(GlobalBytes base, uint32_t off) {
  if constexpr (kNonTemporal) {
    return __builtin_nontemporal_load((GlobalVec)(base + off));  // NOLINT
  } else {
    return *(GlobalVec)(base + off);  // NOLINT
  }
}
__device__ __forceinline__ GlobalBytes wave_uniform_global(const char *p) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(a));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(a >> 32));
  return (GlobalBytes)((static_cast<uint64_t>(hi) << 32) | lo);  // NOLINT
}
// True when a generic pointer names LDS or private (scratch) memory.
__device__ __forceinline__ bool in_lds_or_scratch(const void *p) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_is_shared(p) || __builtin_amdgcn_is_private(p);
#else
  (void)p;  // the host pass only parses device functions
  return false;
#endif
}

// The local side of a put or get may be a __shared__ array or a stack
// variable (the reference copies through generic pointers, so it accepts
// them).  Global loads cannot reach those, so such a copy reads through flat
// accesses, 16 bytes per lane per step and bytes at the end.  A destination in
// device memory (a put from a local buffer) is still written with write-through
// buffer stores, like every other store of a cooperative copy: completion on a
// ROCSHMEM_CTX_NOSTORE context counts on that.  n <= kWindowBytes.
__device__ __forceinline__ void copy_generic(char *dst, const char *src, size_t n, size_t lane,
                                             size_t nlanes) {
  const size_t nvec = n >> 4;
  if (in_lds_or_scratch(dst)) {
    for (size_t i = lane; i < nvec; i += nlanes)
      *reinterpret_cast<u32x4_any *>(dst + (i << 4)) =
          *reinterpret_cast<const u32x4_any *>(src + (i << 4));
    for (size_t k = (nvec << 4) + lane; k < n; k += nlanes) dst[k] = src[k];
    return;
  }
  const __amdgpu_buffer_rsrc_t w = window_of(dst, n);
  size_t head = (16u - (reinterpret_cast<uintptr_t>(dst) & 15u)) & 15u;
  if (head > n) head = n;
  for (size_t k = lane; k < head; k += nlanes)
    store1(w, static_cast<uint32_t>(k), static_cast<uint8_t>(src[k]));
  const size_t body_vec = (n - head) >> 4;
  for (size_t i = lane; i < body_vec; i += nlanes)
    store16<false>(w, static_cast<uint32_t>(head + (i << 4)),
                   *reinterpret_cast<const u32x4_any *>(src + head + (i << 4)));
  for (size_t k = head + (body_vec << 4) + lane; k < n; k += nlanes)
    store1(w, static_cast<uint32_t>(k), static_cast<uint8_t>(src[k]));
}

// Copy n <= kWindowBytes bytes with `nlanes` cooperating lanes; this lane is
// number `lane` (0-based, dense).  Lanes need not belong to one wavefront or
// work-group: a whole grid can call this with global thread ids.  dst, src
// and n are the same in every lane of a wavefront.
template <int kUnroll, bool kNonTemporal>
__device__ __forceinline__ void copy_window(char *dst, const char *src_any, size_t n, size_t lane,
                                            size_t nlanes) {
  if (__builtin_expect(in_lds_or_scratch(dst) || in_lds_or_scratch(src_any), 0)) {
    copy_generic(dst, src_any, n, lane, nlanes);
    return;
  }
  const __amdgpu_buffer_rsrc_t w = window_of(dst, n);
  if (n <= 64 && n <= nlanes) {
    // A byte per lane of the first wavefront (flags, counters, small control
    // messages): no peeling and no loops.  A lone wavefront issues an
    // instruction every few cycles, so what a small message pays for beyond
    // its one load and one store is the number of instructions on its path.
    if (lane < n) store1(w, static_cast<uint32_t>(lane), wave_uniform_global(src_any)[lane]);
    return;
  }
  if (((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src_any) | n) & 15u) == 0 &&
      n <= (nlanes << 4)) {
    // Aligned and at most one vector per lane: the same kind of short path
    // (1.7 -> 1.4 us one way for a 128-byte to 1 KiB ping-pong).  Extending it
    // to a whole burst per lane costs 25 registers and more than it gains.
    if (lane < (n >> 4)) {
      const uint32_t off = static_cast<uint32_t>(lane << 4);
      store16<kNonTemporal>(w, off, load16<kNonTemporal>(wave_uniform_global(src_any), off));
    }
    return;
  }
  size_t head = (16u - (reinterpret_cast<uintptr_t>(dst) & 15u)) & 15u;
  if (head > n) head = n;
  for (size_t k = lane; k < head; k += nlanes) store1(w, static_cast<uint32_t>(k), src_any[k]);
  const GlobalBytes src = wave_uniform_global(src_any + head);
  const size_t body = n - head;
  const uint32_t base = static_cast<uint32_t>(head);

  const size_t nvec = body >> 4;
  const size_t span = static_cast<size_t>(kUnroll) * nlanes;
  auto load_batch = [&](u32x4 (&v)[kUnroll], size_t first) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      v[u] = load16<kNonTemporal>(src, static_cast<uint32_t>((first + lane + u * nlanes) << 4));
  };
  auto store_batch = [&](const u32x4 (&v)[kUnroll], size_t first) {
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      store16<kNonTemporal>(w, base + static_cast<uint32_t>((first + lane + u * nlanes) << 4), v[u]);
  };
  // Whole batches of kUnroll vectors per lane: all loads of a batch, then all
  // its stores; the stores are not waited for, so they overlap the next
  // batch's loads.  Measured on MI355X with 256 work-groups of 1024 lanes
  // streaming 900 KB messages each: batches of 8 give 6.15 TB/s, of 4 6.0, of 2
  // 5.4; keeping a second batch loading while the first is stored (two
  // register sets taking turns) loses 2-7 % against the plain alternation.
  size_t done_vec = 0;  // vectors [0, done_vec) are on their way; uniform
  if constexpr (kUnroll > 1) {
    u32x4 v[kUnroll];
    for (; done_vec + span <= nvec; done_vec += span) {
      load_batch(v, done_vec);
      store_batch(v, done_vec);
    }
  }
  // Fewer than kUnroll vectors per lane are left (any number when kUnroll is
  // 1): all of a lane's are loaded before the first is stored, so a message of
  // up to kUnroll vectors per lane costs one memory round trip, not one per
  // vector.
  for (size_t i = done_vec + lane; i < nvec; i += span) {
    u32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      if (i + u * nlanes < nvec)
        v[u] = load16<kNonTemporal>(src, static_cast<uint32_t>((i + u * nlanes) << 4));
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      if (i + u * nlanes < nvec)
        store16<kNonTemporal>(w, base + static_cast<uint32_t>((i + u * nlanes) << 4), v[u]);
  }

  const uint32_t done = static_cast<uint32_t>(nvec << 4);
  const size_t tail = body - done;
  for (size_t k = lane; k < tail; k += nlanes)
    store1(w, base + done + static_cast<uint32_t>(k), src[done + k]);
}

// Any size: 1 GiB windows, one buffer resource each.
template <int kUnroll, bool kNonTemporal>
__device__ __forceinline__ void copy_lanes_impl(char *dst, const char *src, size_t n, size_t lane,
                                                size_t nlanes) {
  do {
    const size_t chunk = n < kWindowBytes ? n : kWindowBytes;
    copy_window<kUnroll, kNonTemporal>(dst, src, chunk, lane, nlanes);
    dst += chunk;
    src += chunk;
    n -= chunk;
  } while (n);
}

// kLoads: 16-byte vectors a lane loads before it stores them.  A message of up
// to kLoads vectors per lane costs one memory round trip; longer ones alternate
// bursts of kLoads loads and kLoads stores.  Eight covers the memory latency
// for a lone wavefront and is the best burst length for full work-groups that
// stream long messages (see copy_window); the loop needs 4 * kLoads data
// registers.
template <int kLoads = 8>
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
// Plain loads and stores through generic pointers: either side may be LDS or
// a stack variable.  Used where the destination is the caller's own buffer
// (gets); a put goes through copy_thread_through.
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

// ---- write-through stores of a single lane -----------------------------------
// A lane's own stores cannot be buffer stores (the resource is wave-uniform,
// the lanes of a thread-level put go to different places), and global stores
// carry the sc1 bit only as atomic stores: naturally aligned pieces of 1, 2, 4
// or 8 bytes.  `d` names device memory.
typedef __attribute__((address_space(1))) uint64_t *GlobalU64;
typedef __attribute__((address_space(1))) uint32_t *GlobalU32;
typedef __attribute__((address_space(1))) uint16_t *GlobalU16;
typedef __attribute__((address_space(1))) uint8_t *GlobalU8;
__device__ __forceinline__ void store_through8(char *d, uint64_t v) {
  __hip_atomic_store((GlobalU64)d, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // NOLINT
}
__device__ __forceinline__ void store_through4(char *d, uint32_t v) {
  __hip_atomic_store((GlobalU32)d, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // NOLINT
}
__device__ __forceinline__ void store_through2(char *d, uint16_t v) {
  __hip_atomic_store((GlobalU16)d, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // NOLINT
}
__device__ __forceinline__ void store_through1(char *d, uint8_t v) {
  __hip_atomic_store((GlobalU8)d, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // NOLINT
}
// Sixteen bytes at a 16-byte aligned device address.  No builtin gives a
// global store of this width the sc1 bit, so the instruction is written out;
// the compiler does not count it among the outstanding memory operations,
// which only makes its own waits stricter, and callers wait for the lane's
// stores themselves (drain_own_stores).  The s_nop keeps a following write to
// the data registers one wait state away, as a store of more than 8 bytes
// needs on this family.
__device__ __forceinline__ void store_through16(char *d, u32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 0"
               :
               : "v"(reinterpret_cast<unsigned long long>(d)), "v"(v)
               : "memory");
}

// One lane copies n bytes to device memory with write-through stores, so that
// the payload of a thread-level put is visible at agent scope once the lane's
// stores are acknowledged (s_waitcnt) — no L2 write-back.  The destination is
// peeled to 16-byte alignment with the largest pieces its address allows, then
// moved eight 16-byte vectors at a time (all loads of a batch before its
// stores), then finished the same way.  The source may sit anywhere (device
// memory, LDS, a stack variable) at any alignment.
__device__ __forceinline__ void copy_thread_through(void *dst, const void *src, size_t n) {
  char *d = static_cast<char *>(dst);
  const char *s = static_cast<const char *>(src);
  // One piece: the largest power of two up to 16 that the address is aligned
  // to and that fits.
  auto piece = [&]() {
    size_t a = reinterpret_cast<uintptr_t>(d) & 15u;
    a = a ? (a & (~a + 1)) : 16;
    while (a > n) a >>= 1;
    if (a == 16) store_through16(d, *reinterpret_cast<const u32x4_any *>(s));
    else if (a == 8) store_through8(d, *reinterpret_cast<const u64_any *>(s));
    else if (a == 4) store_through4(d, *reinterpret_cast<const u32_any *>(s));
    else if (a == 2) store_through2(d, *reinterpret_cast<const u16_any *>(s));
    else store_through1(d, static_cast<uint8_t>(*s));
    d += a; s += a; n -= a;
  };
  while (n && (reinterpret_cast<uintptr_t>(d) & 15u)) piece();
  while (n >= 128) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const u32x4_any *>(s + 16 * u);
#pragma unroll
    for (int u = 0; u < 8; ++u) store_through16(d + 16 * u, v[u]);
    d += 128; s += 128; n -= 128;
  }
  while (n) piece();
}

// A single value of 1, 2, 4 or 8 bytes (or a multiple of 8) at a naturally
// aligned device address, written through: rocshmem_<T>_p.
template <typename T>
__device__ __forceinline__ void store_value_through(T *dst, T value) {
  char *d = reinterpret_cast<char *>(dst);
  if constexpr (sizeof(T) == 8) {
    uint64_t b;
    __builtin_memcpy(&b, &value, 8);
    store_through8(d, b);
  } else if constexpr (sizeof(T) == 4) {
    uint32_t b;
    __builtin_memcpy(&b, &value, 4);
    store_through4(d, b);
  } else if constexpr (sizeof(T) == 2) {
    uint16_t b;
    __builtin_memcpy(&b, &value, 2);
    store_through2(d, b);
  } else if constexpr (sizeof(T) == 1) {
    uint8_t b;
    __builtin_memcpy(&b, &value, 1);
    store_through1(d, b);
  } else {
    copy_thread_through(d, &value, sizeof(T));
  }
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
  copy_lanes(dst, src, n, rank, count, nt_bytes);
}

}  // namespace detail
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_DETAIL_COPY_ENGINE_HPP_
