// Work-group collectives of one PE: all-reduce, broadcast, alltoall, fcollect,
// barrier_all / sync_all / team_sync.
//
// Calling convention (same as the reference, include/rocshmem/rocshmem_COLL.hpp:33):
// every thread of exactly one work-group per team member calls with identical
// arguments; a team serves one collective at a time.
#ifndef ROCSHMEM_AMD_DETAIL_COLLECTIVES_HPP_
#define ROCSHMEM_AMD_DETAIL_COLLECTIVES_HPP_

#include "copy_engine.hpp"
#include "reduce_engine.hpp"
#include "state.hpp"
#include "sync.hpp"

namespace rocshmem {
namespace detail {

#if defined(__HIPCC__)

// What a synchronisation the user asked for publishes on context c: all of
// the work-group's stores, unless the context was created with
// ROCSHMEM_CTX_NOSTORE (include/rocshmem/rocshmem_common.hpp; the reference
// switches its flush off for that option, src/fence_policy.hpp:45-63).
__device__ __forceinline__ int publish_of(const Context *c) {
  return (ctx_options(c) & static_cast<unsigned>(ROCSHMEM_CTX_NOSTORE)) ? PUBLISH_LIBRARY : PUBLISH_ALL;
}

__device__ __forceinline__ void team_pad_sync(const Context *c, Team *t, int kind, int publish) {
  sync_pes(c, &t->sync[kind], t->wrt_world.pe_start, t->wrt_world.stride,
           t->num_pes, t->my_pe, publish);
}

// src/ipc/context_ipc_device_coll.cpp:101-123
__device__ __forceinline__ void sync_all(Context *c) {
  sync_pes(c, ctx_view(c)->world_sync, 0, 1, ctx_view(c)->num_pes, ctx_view(c)->my_pe, publish_of(c));
}
__device__ __forceinline__ void barrier_all(Context *c) {
  // quiet() of the calling PE is the release half of the barrier's first step.
  sync_all(c);
}

// All-reduce over the team.  Replaces the reference's direct / ring selector
// and its two algorithms (src/ipc/context_ipc_tmpl_device.hpp:166-418) by a
// direct reduce-scatter + all-gather in one pass: after every member has
// arrived, the members fold the index range between them — blocks drawn in
// index order from a counter for large arrays, every P-th block of
// kShareVectors vectors for small ones, either way whatever the sizes of their
// work-groups — from all P sources in ascending member order and store the
// result into all P destinations; a second barrier ends the operation.  Each element is computed
// once, so all members hold bit-identical results.
//
// The reference's selector (:361-418) takes its direct path when P * nreduce
// elements fit max(nreduce / 2 + 1, ROCSHMEM_REDUCE_MIN_WRKDATA_SIZE) and
// P <= ROCSHMEM_REDUCE_SYNC_SIZE, otherwise its ring when
// 2 * P <= ROCSHMEM_REDUCE_SYNC_SIZE, and otherwise returns ROCSHMEM_ERROR.
// Nothing here needs those buffers, but the same calls are refused so that a
// program sees the same status on either library.
// Arrays of at least this many bytes per member are shared out through the
// counter (tens of draws per wavefront; below that the draw's round trip is
// not worth it).
constexpr size_t kTicketBytesFrom = size_t{1} << 20;

__device__ __forceinline__ bool reduce_accepted(int P, int nreduce) {
  const size_t direct_wrk = static_cast<size_t>(P) * static_cast<size_t>(nreduce);
  size_t provided_wrk = static_cast<size_t>(nreduce / 2 + 1);
  if (provided_wrk < ROCSHMEM_REDUCE_MIN_WRKDATA_SIZE) provided_wrk = ROCSHMEM_REDUCE_MIN_WRKDATA_SIZE;
  if (provided_wrk >= direct_wrk && static_cast<size_t>(P) <= ROCSHMEM_REDUCE_SYNC_SIZE) return true;
  return static_cast<size_t>(2 * P) <= ROCSHMEM_REDUCE_SYNC_SIZE;
}

// The fold when the members' slices do not sit a fixed distance apart (one
// process per PE: every peer slice is mapped wherever HIP put it, and found
// through the context's table).  Element by element, members combined in team
// order like the strided fold; blocks of 1024 elements go round the members so
// that the split does not depend on anybody's work-group size.
template <typename E, ROCSHMEM_OP Op>
__device__ __forceinline__ void fold_by_table(Context *c, Team *t,
                                              typename ElemTraits<E>::storage *dest,
                                              const typename ElemTraits<E>::storage *source,
                                              size_t n, unsigned tid, unsigned bs) {
  using Tr = ElemTraits<E>;
  using S = typename Tr::storage;
  using A = typename Tr::accum;
  constexpr size_t kBlock = 1024;
  const int P = t->num_pes, start = t->wrt_world.pe_start, stride = t->wrt_world.stride;
  for (size_t b = static_cast<size_t>(t->my_pe) * kBlock; b < n; b += static_cast<size_t>(P) * kBlock) {
    const size_t bend = b + kBlock < n ? b + kBlock : n;
    for (size_t i = b + tid; i < bend; i += bs) {
      A acc = Tr::widen(*remote_addr(c, source + i, start));
      for (int p = 1; p < P; ++p)
        acc = combine<A, Op>(acc, Tr::widen(*remote_addr(c, source + i, start + p * stride)));
      const S out = Tr::narrow(acc);
      for (int p = 0; p < P; ++p) store_value_through(remote_addr(c, dest + i, start + p * stride), out);
    }
  }
}

template <typename E, ROCSHMEM_OP Op>
__device__ __forceinline__ int wg_reduce(Context *c, Team *t,
                                         typename ElemTraits<E>::storage *dest,
                                         const typename ElemTraits<E>::storage *source,
                                         int nreduce) {
  using S = typename ElemTraits<E>::storage;
  const int P = t->num_pes;
  if (!reduce_accepted(P, nreduce)) return ROCSHMEM_ERROR;

  const size_t n = static_cast<size_t>(nreduce);
  // Large arrays are handed out block by block from a counter on the team's
  // first member (see fold_window), which that member zeroes before it
  // arrives: nobody draws before the entry barrier has seen every member, and
  // every draw of the call before has been answered by its exit barrier.
  // Small ones are split by rule, which costs no round trip to the counter.
  const bool by_table = peers_by_table(c);
  const bool by_tickets = !by_table && n * sizeof(S) >= kTicketBytesFrom && n * sizeof(S) <= kWindowBytes;
  SyncPad *const first_pad = remote_ws(c, &t->sync[SYNC_REDUCE], t->wrt_world.pe_start);
  unsigned long long *const tickets = &first_pad->tickets;
  if (by_tickets && t->my_pe == 0 && is_block_leader()) store_through(tickets, 0ull);

  // Entry: every member's source, which its caller may have written with plain
  // stores, is final.
  team_pad_sync(c, t, SYNC_REDUCE, publish_of(c));

  if (by_table) {
    fold_by_table<E, Op>(c, t, dest, source, n, flat_thread_id(), flat_block_size());
    team_pad_sync(c, t, SYNC_REDUCE, PUBLISH_LIBRARY);
    return ROCSHMEM_SUCCESS;
  }
  const int64_t to_first = static_cast<int64_t>(t->wrt_world.pe_start - ctx_view(c)->my_pe) *
                           static_cast<int64_t>(ctx_view(c)->pe_stride);
  const int64_t hop = static_cast<int64_t>(t->wrt_world.stride) *
                      static_cast<int64_t>(ctx_view(c)->pe_stride);
  S *dst0 = reinterpret_cast<S *>(reinterpret_cast<char *>(dest) + to_first);
  const S *src0 = reinterpret_cast<const S *>(reinterpret_cast<const char *>(source) + to_first);
  // Arrays that are streamed once are read and written with the non-temporal
  // hint, as the bulk copy does.
  const size_t part = static_cast<size_t>(t->my_pe), nparts = static_cast<size_t>(P);
  const unsigned tid = flat_thread_id(), bs = flat_block_size();
  if (by_tickets)
    fold_span_any<E, Op, true, SHARE_TICKETS>(dst0, src0, hop, P, 0, n, tid, bs, part, nparts, tickets);
  else if (n * sizeof(S) >= g_state.nt_bytes)
    fold_span_any<E, Op, true, SHARE_BLOCKS>(dst0, src0, hop, P, 0, n, tid, bs, part, nparts);
  else
    fold_span_any<E, Op, false, SHARE_BLOCKS>(dst0, src0, hop, P, 0, n, tid, bs, part, nparts);

  // Exit: the results were written by the fold, through to memory.
  team_pad_sync(c, t, SYNC_REDUCE, PUBLISH_LIBRARY);
  return ROCSHMEM_SUCCESS;
}

// dest on every member except the root becomes the root's source; the root's
// dest is left alone (src/ipc/context_ipc_tmpl_device.hpp:420-472).  Members
// pull after an entry barrier, so P-1 work-groups copy in parallel and the
// root's source is known to be final; the exit barrier tells the root when
// its source may change.
__device__ __forceinline__ void wg_broadcast(Context *c, Team *t, void *dest,
                                             const void *source, size_t bytes,
                                             int pe_root) {
  team_pad_sync(c, t, SYNC_BCAST, publish_of(c));
  if (t->my_pe != pe_root) {
    const int root_world = t->wrt_world.pe_start + t->wrt_world.stride * pe_root;
    copy_lanes(dest, remote_addr(c, static_cast<const char *>(source), root_world),
               bytes, flat_thread_id(), flat_block_size(), g_state.nt_bytes);
  }
  team_pad_sync(c, t, SYNC_BCAST, PUBLISH_LIBRARY);
}

// dst_j[me*n + k] = src_me[j*n + k] for every member j, self included
// (src/ipc/context_ipc_tmpl_device.hpp:480-501).
__device__ __forceinline__ void wg_alltoall(Context *c, Team *t, void *dest,
                                            const void *source, size_t block_bytes) {
  char *d = static_cast<char *>(dest) + static_cast<size_t>(t->my_pe) * block_bytes;
  const char *s = static_cast<const char *>(source);
  const unsigned tid = flat_thread_id(), bs = flat_block_size();
  for (int j = 0; j < t->num_pes; ++j) {
    const int pe = t->wrt_world.pe_start + t->wrt_world.stride * j;
    copy_lanes(remote_addr(c, d, pe), s + static_cast<size_t>(j) * block_bytes,
               block_bytes, tid, bs, g_state.nt_bytes);
  }
  team_pad_sync(c, t, SYNC_ALLTOALL, PUBLISH_LIBRARY);
}

// dst_j[me*n + k] = src_me[k] (src/ipc/context_ipc_tmpl_device.hpp:509-531).
__device__ __forceinline__ void wg_fcollect(Context *c, Team *t, void *dest,
                                            const void *source, size_t block_bytes) {
  char *d = static_cast<char *>(dest) + static_cast<size_t>(t->my_pe) * block_bytes;
  const unsigned tid = flat_thread_id(), bs = flat_block_size();
  for (int j = 0; j < t->num_pes; ++j) {
    const int pe = t->wrt_world.pe_start + t->wrt_world.stride * j;
    copy_lanes(remote_addr(c, d, pe), source, block_bytes, tid, bs, g_state.nt_bytes);
  }
  team_pad_sync(c, t, SYNC_ALLTOALL, PUBLISH_LIBRARY);
}

#endif  // __HIPCC__

}  // namespace detail
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_DETAIL_COLLECTIVES_HPP_
