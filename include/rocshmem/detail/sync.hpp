// Ordering, atomic memory operations, point-to-point waits and the PE barrier.
//
// The reference issues every atomic and fence at system scope, sequentially
// consistent (src/ipc_policy.hpp:56-99, src/atomic.hpp:59-139) and polls with
// a cache-bypassing load followed by s_waitcnt (src/assembly.hpp:115-162).
// All PEs of this build live on one GPU, so agent scope is the widest scope
// that exists: release = write back this XCD's L2 (buffer_wbl2 sc1),
// acquire = invalidate it (buffer_inv sc1), polls and flag stores go through
// to memory (sc1) so work-groups on different XCDs see each other.
#ifndef ROCSHMEM_AMD_DETAIL_SYNC_HPP_
#define ROCSHMEM_AMD_DETAIL_SYNC_HPP_

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <type_traits>

#include "state.hpp"

namespace rocshmem {
namespace detail {

#if defined(__HIPCC__)

__device__ __forceinline__ void fence_release() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
}
__device__ __forceinline__ void fence_acquire() {
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}
// Wait until every memory operation this wavefront has issued is acknowledged.
// A write-through (sc1) store is acknowledged once it is visible at agent
// scope, so after this the wavefront's cooperative-copy stores are complete
// without an L2 write-back.  Plain stores may still sit dirty in the L2.
__device__ __forceinline__ void drain_own_stores() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
}

// Integer type of the same width, used to move float/double through atomics.
template <size_t N> struct BitsOf;
template <> struct BitsOf<1> { using type = uint8_t; };
template <> struct BitsOf<2> { using type = uint16_t; };
template <> struct BitsOf<4> { using type = uint32_t; };
template <> struct BitsOf<8> { using type = uint64_t; };

template <typename T>
__device__ __forceinline__ T load_through(const T *p) {
  using B = typename BitsOf<sizeof(T)>::type;
  B b = __hip_atomic_load(reinterpret_cast<const B *>(p), __ATOMIC_RELAXED,
                          __HIP_MEMORY_SCOPE_AGENT);
  T out;
  __builtin_memcpy(&out, &b, sizeof(T));
  return out;
}

template <typename T>
__device__ __forceinline__ void store_through(T *p, T v) {
  using B = typename BitsOf<sizeof(T)>::type;
  B b;
  __builtin_memcpy(&b, &v, sizeof(T));
  __hip_atomic_store(reinterpret_cast<B *>(p), b, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

// ---- atomic memory operations on an already-translated address -----------
// Each is one device-wide RMW.  By default the memory order is
// acquire-release, so an AMO can publish or consume data the way the
// reference's seq_cst ones do (src/ipc_policy.hpp:69-99).  With `relaxed`
// (contexts created with ROCSHMEM_CTX_NOSTORE) only the word itself is
// atomic, which is all OpenSHMEM asks of an AMO, and the L2 write-back and
// invalidate that an agent-scope release / acquire costs are left to the
// caller's quiet / fence / wait_until.
// One RMW per lane, straight to memory.
template <typename T>
__device__ __forceinline__ T amo_fetch_add_each(T *p, T v, bool relaxed = false) {
  if (relaxed) return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return __hip_atomic_fetch_add(p, v, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
__device__ __forceinline__ void amo_add_each(T *p, T v, bool relaxed = false) {
  if (relaxed) (void)__hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else (void)__hip_atomic_fetch_add(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ unsigned lane_index() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}
template <typename T>
__device__ __forceinline__ T read_lane(T v, int lane) {
  if constexpr (sizeof(T) == 8) {
    unsigned long long b;
    __builtin_memcpy(&b, &v, 8);
    const unsigned lo = __builtin_amdgcn_readlane(static_cast<unsigned>(b), lane);
    const unsigned hi = __builtin_amdgcn_readlane(static_cast<unsigned>(b >> 32), lane);
    b = (static_cast<unsigned long long>(hi) << 32) | lo;
    T out;
    __builtin_memcpy(&out, &b, 8);
    return out;
  } else {
    unsigned b;
    __builtin_memcpy(&b, &v, 4);
    b = __builtin_amdgcn_readlane(b, lane);
    T out;
    __builtin_memcpy(&out, &b, 4);
    return out;
  }
}
// Value of `v` in lane `lane` (which must be active), lane index per lane.
template <typename T>
__device__ __forceinline__ T from_lane(T v, int lane) {
  if constexpr (sizeof(T) == 8) {
    unsigned long long b;
    __builtin_memcpy(&b, &v, 8);
    const unsigned lo = __builtin_amdgcn_ds_bpermute(lane << 2, static_cast<int>(b));
    const unsigned hi = __builtin_amdgcn_ds_bpermute(lane << 2, static_cast<int>(b >> 32));
    b = (static_cast<unsigned long long>(hi) << 32) | lo;
    T out;
    __builtin_memcpy(&out, &b, 8);
    return out;
  } else {
    int b;
    __builtin_memcpy(&b, &v, 4);
    b = __builtin_amdgcn_ds_bpermute(lane << 2, b);
    T out;
    __builtin_memcpy(&out, &b, 4);
    return out;
  }
}

// One step of a wavefront-wide inclusive sum over all 64 lanes with DPP moves:
// every lane adds the value `ctrl` brings it (0 where there is no source lane).
template <typename T, int kCtrl, int kRowMask>
__device__ __forceinline__ T dpp_add_step(T x) {
  if constexpr (sizeof(T) == 8) {
    unsigned long long b;
    __builtin_memcpy(&b, &x, 8);
    const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_update_dpp(
        0, static_cast<int>(static_cast<unsigned>(b)), kCtrl, kRowMask, 0xf, false));
    const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_update_dpp(
        0, static_cast<int>(static_cast<unsigned>(b >> 32)), kCtrl, kRowMask, 0xf, false));
    const unsigned long long moved = (static_cast<unsigned long long>(hi) << 32) | lo;
    T add;
    __builtin_memcpy(&add, &moved, 8);
    return static_cast<T>(x + add);
  } else {
    unsigned b;
    __builtin_memcpy(&b, &x, 4);
    const unsigned moved =
        static_cast<unsigned>(__builtin_amdgcn_update_dpp(0, static_cast<int>(b), kCtrl, kRowMask, 0xf, false));
    T add;
    __builtin_memcpy(&add, &moved, 4);
    return static_cast<T>(x + add);
  }
}
// Inclusive prefix sum of x over lanes 0..63 in six DPP steps (shifts by 1, 2,
// 4, 8 within rows of 16 lanes, then the last lane of row 0/2 and of rows 0-1
// broadcast to the rows after them).  Every lane of the wavefront must be
// active: a partial sum travels through the lanes between its source and its
// destination.
template <typename T>
__device__ __forceinline__ T wave_inclusive_sum(T x) {
  x = dpp_add_step<T, 0x111, 0xf>(x);  // row_shr:1
  x = dpp_add_step<T, 0x112, 0xf>(x);  // row_shr:2
  x = dpp_add_step<T, 0x114, 0xf>(x);  // row_shr:4
  x = dpp_add_step<T, 0x118, 0xf>(x);  // row_shr:8
  x = dpp_add_step<T, 0x142, 0xa>(x);  // row_bcast:15 into rows 1 and 3
  x = dpp_add_step<T, 0x143, 0xc>(x);  // row_bcast:31 into rows 2 and 3
  return x;
}

// Wavefront-aggregated add.  Lanes of the calling wavefront that target the
// same word are merged: the lowest such lane issues ONE RMW with the sum, and
// every lane of the group receives base + (sum of the group's lower lanes) —
// exactly what it would have fetched had the group's operations run back to
// back in lane order, so the fetched values remain a valid serialisation.
// A hot word (skewed address streams) then costs one memory-side atomic per
// wavefront instead of one per lane.  Groups are found by peeling: take the
// first unassigned lane, ballot for its address, repeat; the search stops once
// a number of lanes in a row turned out to be alone (six, plus four for every
// group found so far: a stream that has shown one hot word tends to have
// more), which keeps the cost flat for address streams without collisions.
// The lower-lane sums of a group come from the lane count when all its addends
// are equal (fetch_inc, add of a constant), from a six-step DPP prefix sum over
// the wavefront when the group is large and the wavefront full, and from a walk
// over the group's lanes otherwise.
template <typename T, bool kFetch>
__device__ __forceinline__ T amo_add_wave(T *p, T v, bool relaxed) {
  constexpr int kMissBudget = 6, kMissBudgetPerGroup = 4, kScanFrom = 5;
  const unsigned lane = lane_index();
  const unsigned long long addr = reinterpret_cast<unsigned long long>(p);
  const unsigned long long active = __ballot(1);
  unsigned long long rem = active;
  int leader = static_cast<int>(lane);
  T prefix = static_cast<T>(0);
  T total = v;
  int misses = 0, budget = kMissBudget;
  while (rem && misses < budget) {
    const int l = __ffsll(static_cast<long long>(rem)) - 1;
    const unsigned long long a = read_lane(addr, l);
    const bool mine = addr == a;
    const unsigned long long same = __ballot(mine);
    if (same & (same - 1)) {  // two or more lanes share this word
      misses = 0;
      budget += kMissBudgetPerGroup;
      const int members = __popcll(same);
      const T v_first = read_lane(v, l);
      T before, sum;  // of this lane's group: addends of its lower lanes, all addends
      if (__ballot(mine && v != v_first) == 0) {
        const unsigned below = __builtin_amdgcn_mbcnt_hi(
            static_cast<unsigned>(same >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(same), 0u));
        before = static_cast<T>(v_first * static_cast<T>(below));
        sum = static_cast<T>(v_first * static_cast<T>(members));
      } else if (members >= kScanFrom && active == ~0ull) {
        const T mine_v = mine ? v : static_cast<T>(0);
        const T upto = wave_inclusive_sum<T>(mine_v);
        before = static_cast<T>(upto - mine_v);
        sum = read_lane(upto, 63);
      } else {
        T run = static_cast<T>(0);
        before = run;
        unsigned long long m = same;
        while (m) {
          const int j = __ffsll(static_cast<long long>(m)) - 1;
          const T vj = read_lane(v, j);
          if (static_cast<int>(lane) == j) before = run;
          run = static_cast<T>(run + vj);
          m &= m - 1;
        }
        sum = run;
      }
      if (mine) {
        leader = l;
        prefix = before;
        total = sum;
      }
    } else {
      ++misses;
    }
    rem &= ~same;
  }
  T base = static_cast<T>(0);
  if (leader == static_cast<int>(lane)) {
    if constexpr (kFetch) base = amo_fetch_add_each(p, total, relaxed);
    else amo_add_each(p, total, relaxed);
  }
  if constexpr (kFetch) {
    base = from_lane(base, leader);
    return static_cast<T>(base + prefix);
  }
  return base;
}

template <typename T>
__device__ __forceinline__ T amo_fetch_add(T *p, T v, bool relaxed = false) {
  return amo_add_wave<T, true>(p, v, relaxed);
}
template <typename T>
__device__ __forceinline__ void amo_add(T *p, T v, bool relaxed = false) {
  (void)amo_add_wave<T, false>(p, v, relaxed);
}
template <typename T>
__device__ __forceinline__ T amo_fetch_cas(T *p, T cond, T v, bool relaxed = false) {
  using B = typename BitsOf<sizeof(T)>::type;
  B expected, desired;
  __builtin_memcpy(&expected, &cond, sizeof(T));
  __builtin_memcpy(&desired, &v, sizeof(T));
  if (relaxed)
    __hip_atomic_compare_exchange_strong(reinterpret_cast<B *>(p), &expected, desired,
                                         __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
  else
    __hip_atomic_compare_exchange_strong(reinterpret_cast<B *>(p), &expected, desired,
                                         __ATOMIC_ACQ_REL, __ATOMIC_ACQUIRE,
                                         __HIP_MEMORY_SCOPE_AGENT);
  T out;
  __builtin_memcpy(&out, &expected, sizeof(T));
  return out;
}
template <typename T>
__device__ __forceinline__ void amo_set(T *p, T v, bool relaxed = false) {
  using B = typename BitsOf<sizeof(T)>::type;
  B b;
  __builtin_memcpy(&b, &v, sizeof(T));
  if (relaxed)
    __hip_atomic_store(reinterpret_cast<B *>(p), b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else
    __hip_atomic_store(reinterpret_cast<B *>(p), b, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
__device__ __forceinline__ T amo_fetch(T *p, bool relaxed = false) {
  using B = typename BitsOf<sizeof(T)>::type;
  B b = relaxed ? __hip_atomic_load(reinterpret_cast<const B *>(p), __ATOMIC_RELAXED,
                                    __HIP_MEMORY_SCOPE_AGENT)
                : __hip_atomic_load(reinterpret_cast<const B *>(p), __ATOMIC_ACQUIRE,
                                    __HIP_MEMORY_SCOPE_AGENT);
  T out;
  __builtin_memcpy(&out, &b, sizeof(T));
  return out;
}
template <typename T>
__device__ __forceinline__ T amo_swap(T *p, T v, bool relaxed = false) {
  using B = typename BitsOf<sizeof(T)>::type;
  B b;
  __builtin_memcpy(&b, &v, sizeof(T));
  B old = relaxed ? __hip_atomic_exchange(reinterpret_cast<B *>(p), b, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT)
                  : __hip_atomic_exchange(reinterpret_cast<B *>(p), b, __ATOMIC_ACQ_REL,
                                          __HIP_MEMORY_SCOPE_AGENT);
  T out;
  __builtin_memcpy(&out, &old, sizeof(T));
  return out;
}
template <typename T>
__device__ __forceinline__ T amo_fetch_and(T *p, T v, bool relaxed = false) {
  if (relaxed) return __hip_atomic_fetch_and(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return __hip_atomic_fetch_and(p, v, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
__device__ __forceinline__ T amo_fetch_or(T *p, T v, bool relaxed = false) {
  if (relaxed) return __hip_atomic_fetch_or(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return __hip_atomic_fetch_or(p, v, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename T>
__device__ __forceinline__ T amo_fetch_xor(T *p, T v, bool relaxed = false) {
  if (relaxed) return __hip_atomic_fetch_xor(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return __hip_atomic_fetch_xor(p, v, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- point-to-point synchronisation ---------------------------------------
// Comparator table of the reference's Context::test
// (src/context_tmpl_device.hpp:337-377); an unknown comparator never holds.
template <typename T>
__device__ __forceinline__ bool compare(T x, int cmp, T val) {
  switch (cmp) {
    case ROCSHMEM_CMP_EQ: return x == val;
    case ROCSHMEM_CMP_NE: return x != val;
    case ROCSHMEM_CMP_GT: return x > val;
    case ROCSHMEM_CMP_GE: return x >= val;
    case ROCSHMEM_CMP_LT: return x < val;
    case ROCSHMEM_CMP_LE: return x <= val;
    default: return false;
  }
}

// Between two polls of a wait.  The reference's waits spin without bound
// (src/context_tmpl_device.hpp:201-218); so do these unless the runtime has
// been given a limit (ROCSHMEM_EMU_SPIN_LIMIT): then a wait that has polled
// that often records the fact (DeviceState::gave_up, which the host reads) and
// returns, so that a kernel whose partner never comes ends instead of holding
// the GPU.  Returns false when the caller should stop waiting.
__device__ __forceinline__ bool keep_waiting(uint64_t *polls) {
  __builtin_amdgcn_s_sleep(1);
  const uint64_t limit = g_state.spin_limit;
  if (limit == 0 || ++*polls < limit) return true;
  __hip_atomic_fetch_add(g_state.gave_up, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return false;
}

// One poll.  A successful poll acquires, so data published before the value
// was written (put_signal payloads) is visible afterwards.
template <typename T>
__device__ __forceinline__ int test(T *ivar, int cmp, T val) {
  if (compare(load_through(ivar), cmp, val)) {
    fence_acquire();
    return 1;
  }
  return 0;
}

template <typename T>
__device__ __forceinline__ void wait_until(T *ivar, int cmp, T val) {
  uint64_t polls = 0;
  while (!compare(load_through(ivar), cmp, val))
    if (!keep_waiting(&polls)) break;
  fence_acquire();
}

__device__ __forceinline__ size_t first_unmasked(size_t nelems, const int *status) {
  size_t i = 0;
  if (status) {
    while (i < nelems && status[i] != 0) ++i;
  }
  return i;
}

// src/context_tmpl_device.hpp:220-250
template <typename T>
__device__ __forceinline__ size_t wait_until_any(T *ivars, size_t nelems,
                                                 const int *status, int cmp, T val) {
  if (!nelems) return SIZE_MAX;
  const size_t pos = first_unmasked(nelems, status);
  if (pos == nelems) return SIZE_MAX;
  uint64_t polls = 0;
  for (;;) {
    for (size_t i = pos; i < nelems; ++i) {
      if (status && status[i]) continue;
      if (test(ivars + i, cmp, val)) return i;
    }
    if (!keep_waiting(&polls)) return SIZE_MAX;
  }
}

// src/context_tmpl_device.hpp:252-275
template <typename T>
__device__ __forceinline__ void wait_until_all(T *ivars, size_t nelems,
                                               const int *status, int cmp, T val) {
  if (!nelems) return;
  const size_t pos = first_unmasked(nelems, status);
  if (pos == nelems) return;
  for (size_t i = pos; i < nelems; ++i) {
    if (status && status[i]) continue;
    wait_until(ivars + i, cmp, val);
  }
}

// src/context_tmpl_device.hpp:277-310: sweeps until one sweep finds at least
// one satisfied entry and reports every entry that sweep found.
template <typename T>
__device__ __forceinline__ size_t wait_until_some(T *ivars, size_t nelems,
                                                  size_t *indices, const int *status,
                                                  int cmp, T val) {
  if (!nelems) return 0;
  const size_t pos = first_unmasked(nelems, status);
  if (pos == nelems) return 0;
  size_t ncompleted = 0;
  uint64_t polls = 0;
  while (ncompleted == 0) {
    for (size_t i = pos; i < nelems; ++i) {
      if (status && status[i]) continue;
      if (test(ivars + i, cmp, val)) indices[ncompleted++] = i;
    }
    if (ncompleted == 0 && !keep_waiting(&polls)) break;
  }
  return ncompleted;
}

// ---- barrier between the work-groups that act for the PEs of a team --------
// Called by every thread of exactly one work-group per team member.  The
// first wavefront does the work with its lanes in parallel: lane j announces
// this round's epoch in member j's pad and polls member j's announcement in
// the local pad.  (The reference's thread 0 walks the flags one by one and
// resets them: src/ipc/context_ipc_device_coll.cpp:31-99.)
//
// What the arrival publishes:
//   PUBLISH_ALL     everything the work-group has stored, plain stores
//                   included: an agent-scope release, i.e. an L2 write-back.
//                   On MI355X one write-back stalls its XCD's L2 for about
//                   0.3 us whenever the kernel has loads in flight, whether or
//                   not a line is dirty (measured: a P = 8 team reduce with a
//                   write-back in both of its barriers loses 3 % with 32
//                   teams on the GPU and 11 % with 128).
//   PUBLISH_LIBRARY what the library itself has stored for the work-group
//                   (cooperative copies and folds are write-through stores):
//                   every wavefront waits for its own stores, no write-back.
//                   Right for the barrier that ends a collective, whose
//                   payload the library wrote, and for contexts created with
//                   ROCSHMEM_CTX_NOSTORE.
enum PublishKind : int { PUBLISH_ALL = 0, PUBLISH_LIBRARY = 1 };

__device__ __forceinline__ void sync_pes(const Context *c, SyncPad *pad,
                                         int pe_start, int stride, int size,
                                         int my_index, int publish = PUBLISH_ALL) {
  if (publish == PUBLISH_LIBRARY) drain_own_stores();
  __syncthreads();
  const unsigned tid = flat_thread_id();
  if (tid < 64u) {
    unsigned nl = flat_block_size();
    if (nl > 64u) nl = 64u;
    // A load that goes to memory (385 ns), although the counter is private to
    // this work-group: read through the caches (an L2 hit, 115 ns) it leaves a
    // line in the L2, and an L2 that holds lines makes every write-back on its
    // XCD slow (a many-teams reduce lost 4 % that way).
    const unsigned long long round = load_through(&pad->epoch) + 1ull;
    if (publish == PUBLISH_ALL) fence_release();
    for (unsigned j = tid; j < static_cast<unsigned>(size); j += nl) {
      SyncPad *peer = remote_ws(c, pad, pe_start + static_cast<int>(j) * stride);
      store_through(&peer->slots[my_index], round);
    }
    for (unsigned j = tid; j < static_cast<unsigned>(size); j += nl) {
      uint64_t polls = 0;
      while (load_through(&pad->slots[j]) < round)
        if (!keep_waiting(&polls)) break;
    }
    fence_acquire();
    // All lanes of this wavefront have left their polling loops here.
    if (tid == 0) store_through(&pad->epoch, round);
  }
  __syncthreads();
}

#endif  // __HIPCC__

}  // namespace detail
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_DETAIL_SYNC_HPP_
