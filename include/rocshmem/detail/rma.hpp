// Remote memory access, put-with-signal and context lifecycle of one PE.
#ifndef ROCSHMEM_AMD_DETAIL_RMA_HPP_
#define ROCSHMEM_AMD_DETAIL_RMA_HPP_

#include "coalesce.hpp"
#include "copy_engine.hpp"
#include "state.hpp"
#include "sync.hpp"

namespace rocshmem {
namespace detail {

#if defined(__HIPCC__)

// Team-relative PE -> world PE for the calls that translate
// (src/rocshmem_gpu.cpp:267-274: a null team_opaque passes pe through).
__device__ __forceinline__ int translate_pe(rocshmem_ctx_t ctx, int pe) {
  const TeamInfo *ti = reinterpret_cast<const TeamInfo *>(ctx.team_opaque);
  return ti ? ti->pe_start + ti->stride * pe : pe;
}

// ---- what completes a put, and what quiet / fence add -------------------------
// Every store the library makes to the symmetric heap is a write-through store
// (sc1): buffer stores in the cooperative copies and folds, atomic stores in
// the single-lane copy.  Such a store is acknowledged once it is visible at
// agent scope, so a wavefront completes its own puts by waiting for its own
// memory operations (drain_own_stores) — no L2 write-back.  That is how the
// blocking thread- and wavefront-level puts return with their payload
// delivered on every kind of context, as the reference's do through a fence
// after each copy (src/ipc/context_ipc_device.cpp:62-69,137-144), at a
// fortieth of the cost: an agent-scope fence is an L2 write-back plus
// invalidate, which an XCD's L2 serves one after another (measured on MI355X,
// 2 Mi putmem_wave calls of 512 bytes from every CU: 70 M calls/s with a fence
// per call, 2.7 G calls/s with the wait).
//
// What a put does NOT publish is the caller's own plain stores.  That is the
// job of quiet and fence: on a default context a full agent-scope release
// (L2 write-back; cumulative, so it also covers stores that other wavefronts
// of the work-group made before a barrier).  A context created with
// ROCSHMEM_CTX_NOSTORE promises that quiet / fence need not order the caller's
// plain stores (the reference turns its flush off for such contexts,
// src/fence_policy.hpp:45-63): there they are the wait alone.  The work-group
// put ends in a barrier, not in a completion (as in the reference, :109-116);
// on a NOSTORE context every wavefront also waits for its own share first, so
// that a quiet by any one thread covers the whole work-group's put.
__device__ __forceinline__ bool no_store_order(const Context *c) {
  return (ctx_options(c) & static_cast<unsigned>(ROCSHMEM_CTX_NOSTORE)) != 0;
}
// A get reads what memory holds now: the L1 of the CU and the L2 of the XCD may
// keep a line of the heap that another XCD has since written through to
// memory (measured with the L2's hit counters: reads of the heap are cached in
// the L2 whether the heap was allocated cached or uncached), and a loop that
// polls with gets must not be served that line for ever.  So a thread- or
// wavefront-level get invalidates first (an agent-scope acquire), as every
// successful wait does.
__device__ __forceinline__ void fresh_reads() { fence_acquire(); }
// quiet / fence on context c.
__device__ __forceinline__ void ctx_release(const Context *c) {
  if (no_store_order(c)) drain_own_stores();
  else fence_release();
}

// ---- thread granularity (context_ipc_device.cpp:62-88) ----------------------
// The reference puts a coalescing step in front of its per-thread messages
// (src/wf_coal_policy.cpp:57-172).  Here, when the runtime asks for it
// (DeviceState::coalesce_puts), a thread-level put first looks whether the
// messages of all active lanes continue one another to the same PE; such a
// run is one message, moved by the whole wavefront with the cooperative copy
// (16 bytes per lane and step, whatever the size of a lane's own message).
// Returns false, having done nothing, for anything else.
__device__ __forceinline__ bool put_as_one_run(Context *c, void *dest, const void *source,
                                               size_t n, int pe) {
  size_t merged = n;
  const bool sender = wf_coalesce(pe, source, dest, &merged);
  const unsigned long long senders = __ballot(sender);
  // One sender means every other active lane was absorbed, which needs the
  // lane below it to be active: the run starts at the lowest active lane.
  if (senders & (senders - 1)) return false;
  // From here on everything is taken from the sender's lane, so that all
  // lanes decide and address alike.
  const int leader = __ffsll(static_cast<long long>(senders)) - 1;
  const size_t total = read_lane(static_cast<unsigned long long>(merged), leader);
  const size_t own = read_lane(static_cast<unsigned long long>(n), leader);
  if (total == own) return false;  // a lone lane: nothing to share
  char *d = reinterpret_cast<char *>(read_lane(reinterpret_cast<unsigned long long>(dest), leader));
  const char *s = reinterpret_cast<const char *>(
      read_lane(reinterpret_cast<unsigned long long>(source), leader));
  const int to = read_lane(pe, leader);
  const size_t nt = g_state.nt_bytes;  // (asked for before remote_addr's branch, see putmem_wg)
  copy_wave(remote_addr(c, d, to), s, total, nt);
  drain_own_stores();
  return true;
}

__device__ __forceinline__ void putmem(Context *c, void *dest, const void *source,
                                       size_t n, int pe) {
  if (g_state.coalesce_puts && put_as_one_run(c, dest, source, n, pe)) return;
  copy_thread_through(remote_addr(c, static_cast<char *>(dest), pe), source, n);
  drain_own_stores();
}
__device__ __forceinline__ void getmem(Context *c, void *dest, const void *source,
                                       size_t n, int pe) {
  fresh_reads();
  copy_thread(dest, remote_addr(c, static_cast<const char *>(source), pe), n);
}
// rocshmem_<T>_p / _g: one naturally aligned value.
template <typename T>
__device__ __forceinline__ void put_value(Context *c, T *dest, T value, int pe) {
  store_value_through(remote_addr(c, dest, pe), value);
  drain_own_stores();
}

// One value of 1, 2, 4 or 8 bytes comes as a single load that goes to memory
// (what a loop that polls with rocshmem_<T>_g needs, at no invalidate);
// anything wider as a get.
template <typename T>
__device__ __forceinline__ T get_value(Context *c, const T *source, int pe) {
  const T *from = remote_addr(c, source, pe);
  if constexpr (sizeof(T) == 1 || sizeof(T) == 2 || sizeof(T) == 4 || sizeof(T) == 8) {
    return load_through(from);
  } else {
    T value;
    fresh_reads();
    copy_thread(&value, from, sizeof(T));
    return value;
  }
}

// Non-blocking forms: the call only issues the copy; rocshmem_ctx_quiet (or
// fence) by the same thread completes it.  The reference's _nbi calls are its
// blocking ones; here a thread or wavefront that issues many small messages
// pays for one completion instead of one per message.
__device__ __forceinline__ void putmem_nbi(Context *c, void *dest, const void *source,
                                           size_t n, int pe) {
  copy_thread_through(remote_addr(c, static_cast<char *>(dest), pe), source, n);
}
__device__ __forceinline__ void getmem_nbi(Context *c, void *dest, const void *source,
                                           size_t n, int pe) {
  fresh_reads();
  copy_thread(dest, remote_addr(c, static_cast<const char *>(source), pe), n);
}

// ---- wavefront granularity (context_ipc_device.cpp:137-164) ---------------
__device__ __forceinline__ void putmem_wave(Context *c, void *dest, const void *source,
                                            size_t n, int pe) {
  const size_t nt = g_state.nt_bytes;
  copy_wave(remote_addr(c, static_cast<char *>(dest), pe), source, n, nt);
  drain_own_stores();
}
// A get's stores go to the caller's own buffer; the wait makes them complete
// for whoever reads it after a barrier.
__device__ __forceinline__ void getmem_wave(Context *c, void *dest, const void *source,
                                            size_t n, int pe) {
  fresh_reads();
  const size_t nt = g_state.nt_bytes;
  copy_wave(dest, remote_addr(c, static_cast<const char *>(source), pe), n, nt);
  drain_own_stores();
}

// Non-blocking wavefront forms: complete at the calling wavefront's quiet on
// either kind of context.
__device__ __forceinline__ void putmem_nbi_wave(Context *c, void *dest, const void *source,
                                                size_t n, int pe) {
  const size_t nt = g_state.nt_bytes;
  copy_wave(remote_addr(c, static_cast<char *>(dest), pe), source, n, nt);
}
__device__ __forceinline__ void getmem_nbi_wave(Context *c, void *dest, const void *source,
                                                size_t n, int pe) {
  fresh_reads();
  const size_t nt = g_state.nt_bytes;
  copy_wave(dest, remote_addr(c, static_cast<const char *>(source), pe), n, nt);
}

// ---- work-group granularity: copy, then __syncthreads (:109-125) ----------
// The ordering option is looked at before the copy although it is only needed
// after it: the context's hot fields share one scalar load, and a call then
// waits for the scalar data path once, not once per field (a scalar load that
// hits costs about 100 ns, which a small message feels).
__device__ __forceinline__ void putmem_wg(Context *c, void *dest, const void *source,
                                          size_t n, int pe) {
  const bool relaxed = no_store_order(c);
  // (everything that comes from scalar loads is asked for before remote_addr,
  // whose rare table path is a branch that later loads would queue behind)
  const unsigned tid = flat_thread_id(), bs = flat_block_size();
  const size_t nt = g_state.nt_bytes;
  copy_lanes(remote_addr(c, static_cast<char *>(dest), pe), source, n, tid, bs, nt);
  // Each wavefront completes its own share, so that after the barrier a quiet
  // by any one thread covers the whole work-group's put.
  if (relaxed) drain_own_stores();
  __syncthreads();
}
// The work-group get is the reference's: copy, then barrier, and no fence
// (:118-125) — it reads through whatever the caches hold, which is right
// after any synchronisation (waits and barriers invalidate) and keeps a bulk
// get from every CU at the rate of the put (an invalidate per call costs an
// XCD's L2 as much as a write-back: 65536 calls of 4 KiB took 0.97 ms with it
// against 0.083 ms without).  A loop that polls uses rocshmem_<T>_g, a thread-
// or wavefront-level get, or a wait.
__device__ __forceinline__ void getmem_wg(Context *c, void *dest, const void *source,
                                          size_t n, int pe) {
  const unsigned tid = flat_thread_id(), bs = flat_block_size();
  const size_t nt = g_state.nt_bytes;
  copy_lanes(dest, remote_addr(c, static_cast<const char *>(source), pe), n, tid, bs, nt);
  __syncthreads();
}

// ---- signal update by the one lane that leads the call (:221-298) ---------
// On a default context the store / add is a release at agent scope, which
// orders it after the payload and after everything else the caller's group
// wrote before it.  On a ROCSHMEM_CTX_NOSTORE context the payload is already
// complete when the leader gets here (write-through stores, waited for by
// each wavefront or thread), so a relaxed update suffices.
__device__ __forceinline__ void signal_update(Context *c, uint64_t *sig_addr,
                                              uint64_t signal, int sig_op, int pe,
                                              bool relaxed = false) {
  unsigned long long *target =
      reinterpret_cast<unsigned long long *>(remote_addr(c, sig_addr, pe));
  switch (sig_op) {
    case ROCSHMEM_SIGNAL_SET:
      amo_set<unsigned long long>(target, signal, relaxed);
      break;
    case ROCSHMEM_SIGNAL_ADD:
      amo_add<unsigned long long>(target, signal, relaxed);
      break;
    default:
      break;  // unknown op: payload delivered, signal untouched
  }
}

__device__ __forceinline__ void putmem_signal(Context *c, void *dest, const void *source,
                                              size_t n, uint64_t *sig_addr,
                                              uint64_t signal, int sig_op, int pe) {
  putmem(c, dest, source, n, pe);
  signal_update(c, sig_addr, signal, sig_op, pe, no_store_order(c));
}
__device__ __forceinline__ void putmem_signal_wave(Context *c, void *dest,
                                                   const void *source, size_t n,
                                                   uint64_t *sig_addr, uint64_t signal,
                                                   int sig_op, int pe) {
  putmem_wave(c, dest, source, n, pe);
  // The leader is the lowest active lane, which exists for any active mask.
  const unsigned long long mask = __ballot(1);
  const unsigned lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  if (lane == static_cast<unsigned>(__ffsll(static_cast<long long>(mask)) - 1))
    signal_update(c, sig_addr, signal, sig_op, pe, no_store_order(c));
}
__device__ __forceinline__ void putmem_signal_wg(Context *c, void *dest,
                                                 const void *source, size_t n,
                                                 uint64_t *sig_addr, uint64_t signal,
                                                 int sig_op, int pe) {
  putmem_wg(c, dest, source, n, pe);
  if (is_block_leader()) signal_update(c, sig_addr, signal, sig_op, pe, no_store_order(c));
}

// signal_fetch: atomic read of the caller's own word (:300-324).
__device__ __forceinline__ uint64_t signal_fetch(const uint64_t *sig_addr) {
  return amo_fetch(const_cast<unsigned long long *>(
      reinterpret_cast<const unsigned long long *>(sig_addr)));
}
__device__ __forceinline__ uint64_t signal_fetch_wave(const uint64_t *sig_addr) {
  const unsigned long long mask = __ballot(1);
  const int leader = __ffsll(static_cast<long long>(mask)) - 1;
  const unsigned lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
  unsigned long long v = 0;
  if (static_cast<int>(lane) == leader) v = signal_fetch(sig_addr);
  const unsigned lo = __builtin_amdgcn_readlane(static_cast<unsigned>(v), leader);
  const unsigned hi = __builtin_amdgcn_readlane(static_cast<unsigned>(v >> 32), leader);
  return (static_cast<uint64_t>(hi) << 32) | lo;
}
__device__ __forceinline__ uint64_t signal_fetch_wg(const uint64_t *sig_addr) {
  __shared__ unsigned long long wg_value;
  __syncthreads();
  if (is_block_leader()) wg_value = signal_fetch(sig_addr);
  __syncthreads();
  return wg_value;
}

// ---- context lifecycle (src/rocshmem_gpu.cpp:286-325) ----------------------
__device__ __forceinline__ Context *pool_claim(CtxPool *pool) {
  const int words = (pool->capacity + 63) / 64;
  for (int w = 0; w < words; ++w) {
    unsigned long long m = __hip_atomic_load(&pool->free_mask[w], __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
    while (m) {
      const int b = __ffsll(static_cast<long long>(m)) - 1;
      const unsigned long long bit = 1ull << b;
      const unsigned long long old = __hip_atomic_fetch_and(
          &pool->free_mask[w], ~bit, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
      if (old & bit) return pool->slots + (w * 64 + b);
      m = old & ~bit;
    }
  }
  return nullptr;
}
__device__ __forceinline__ void pool_release(CtxPool *pool, Context *c) {
  const int s = ctx_view(c)->pool_slot;
  __hip_atomic_fetch_or(&pool->free_mask[s >> 6], 1ull << (s & 63), __ATOMIC_RELEASE,
                        __HIP_MEMORY_SCOPE_AGENT);
}

// Thread 0 claims a context of PE `pe` bound to `tinfo`; every thread learns
// the outcome through *ctx (which lives in the caller's shared memory).  Each
// pool slot holds one prebuilt object per ordering option, so nothing is
// written into a context here; the team travels in the handle.
__device__ __forceinline__ int wg_ctx_create_for(int pe, TeamInfo *tinfo, long options,
                                                 rocshmem_ctx_t *ctx) {
  if (is_block_leader()) {
    CtxPool *pool = g_state.ctx_pool + pe;
    Context *c = pool_claim(pool);
    if (c && (options & ROCSHMEM_CTX_NOSTORE)) c += pool->capacity;
    ctx->ctx_opaque = c;
    ctx->team_opaque = tinfo;
  }
  __syncthreads();
  return ctx->ctx_opaque ? 0 : -1;
}

__device__ __forceinline__ void wg_ctx_destroy(rocshmem_ctx_t *ctx) {
  if (is_block_leader()) {
    Context *c = reinterpret_cast<Context *>(ctx->ctx_opaque);
    if (c && ctx_view(c)->pool_slot >= 0) pool_release(g_state.ctx_pool + ctx_view(c)->my_pe, c);
  }
}

#endif  // __HIPCC__

}  // namespace detail
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_DETAIL_RMA_HPP_
