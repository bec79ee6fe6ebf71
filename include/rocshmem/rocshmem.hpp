// Public header of the symmetric-heap data-movement library for MI355X.
//
// Host interface: runtime bring-up, symmetric allocation, teams.
// Device interface: everything a kernel calls — context lifecycle, ordering,
// PE queries, barriers — plus, through the family headers included below, RMA,
// atomics, signals, collectives and point-to-point waits.
//
// Declarations match include/rocshmem/rocshmem.hpp:62-530 of the reference.
// Device functions are defined inline so user kernels need no relocatable
// device code.  All P processing elements are hosted by one process on one
// GPU (see rocshmem_emu.hpp for the controls that choose P and the acting PE).
#ifndef ROCSHMEM_AMD_ROCSHMEM_HPP_
#define ROCSHMEM_AMD_ROCSHMEM_HPP_

#include <hip/hip_runtime.h>

#include <cassert>
#include <cstdlib>

// No MPI is used by this library; MPI_Comm only keeps rocshmem_init's
// signature source-compatible.  Without a real mpi.h the names come from
// compat/mpi.h.
#if __has_include(<mpi.h>) && !defined(ROCSHMEM_AMD_NO_MPI_HEADER)
#include <mpi.h>
#else
#include "compat/mpi.h"
#endif

#include "rocshmem_config.h"
#include "rocshmem_common.hpp"
#include "rocshmem_RMA.hpp"
#include "rocshmem_AMO.hpp"
#include "rocshmem_SIG_OP.hpp"
#include "rocshmem_COLL.hpp"
#include "rocshmem_P2P_SYNC.hpp"
#include "rocshmem_RMA_X.hpp"
#include "rocshmem_emu.hpp"
#include "rocshmem_HOST.hpp"

namespace rocshmem {

// ============================ host interface ================================
__host__ void rocshmem_init(MPI_Comm comm = MPI_COMM_WORLD);
__host__ void rocshmem_init_thread(int requested, int *provided,
                                   MPI_Comm comm = MPI_COMM_WORLD);
__host__ void rocshmem_query_thread(int *provided);
__host__ void rocshmem_dump_stats();
__host__ void rocshmem_reset_stats();
__host__ void rocshmem_finalize();
__host__ void *rocshmem_malloc(size_t size);
__host__ void rocshmem_free(void *ptr);
__host__ int rocshmem_n_pes();
__host__ int rocshmem_my_pe();
__host__ int rocshmem_ctx_create(int64_t options, rocshmem_ctx_t *ctx);
__host__ void rocshmem_ctx_destroy(rocshmem_ctx_t ctx);
__host__ int rocshmem_team_translate_pe(rocshmem_team_t src_team, int src_pe,
                                        rocshmem_team_t dest_team);
__host__ int rocshmem_team_n_pes(rocshmem_team_t team);
__host__ int rocshmem_team_my_pe(rocshmem_team_t team);
__host__ int rocshmem_team_split_strided(rocshmem_team_t parent_team, int start,
                                         int stride, int size,
                                         const rocshmem_team_config_t *config,
                                         long config_mask, rocshmem_team_t *new_team);
__host__ void rocshmem_team_destroy(rocshmem_team_t team);
__host__ void rocshmem_ctx_fence(rocshmem_ctx_t ctx);
__host__ void rocshmem_fence();
__host__ void rocshmem_ctx_quiet(rocshmem_ctx_t ctx);
__host__ void rocshmem_quiet();
__host__ void rocshmem_barrier_all();
__host__ void rocshmem_sync_all();
__host__ void rocshmem_global_exit(int status);

#if defined(__HIPCC__)

// Default context: a null handle, resolved on the device to the default
// context of the acting PE.
__attribute__((used)) static __constant__ rocshmem_ctx_t ROCSHMEM_CTX_DEFAULT = {nullptr, nullptr};

// =========================== device interface ===============================
__device__ inline void rocshmem_query_thread(int *provided) {
  *provided = ROCSHMEM_THREAD_WG_FUNNELED;
}
__device__ inline void rocshmem_wg_init_thread(int, int *provided) {
  rocshmem_query_thread(provided);
}
__device__ inline void rocshmem_wg_init() {}
__device__ inline void rocshmem_wg_finalize() {}

// Context bound to the world team of the acting PE.
__device__ ATTR_NO_INLINE inline int rocshmem_wg_ctx_create(int64_t options,
                                                            rocshmem_ctx_t *ctx) {
  const int pe = detail::acting_pe();
  return detail::wg_ctx_create_for(pe, &detail::g_state.world_team[pe].wrt_world,
                                   options, ctx);
}
// Context bound to `team`; the PE is the one the team object belongs to.
__device__ ATTR_NO_INLINE inline int rocshmem_wg_team_create_ctx(rocshmem_team_t team,
                                                                 long options,
                                                                 rocshmem_ctx_t *ctx) {
  detail::Team *t = detail::team_of(team);
  if (!t) {  // ROCSHMEM_TEAM_INVALID, or the acting PE is not a member
    if (detail::is_block_leader()) *ctx = rocshmem_ctx_t{nullptr, nullptr};
    __syncthreads();
    return -1;
  }
  return detail::wg_ctx_create_for(t->my_pe_in_world, &t->wrt_world, options, ctx);
}
__device__ ATTR_NO_INLINE inline void rocshmem_wg_ctx_destroy(rocshmem_ctx_t *ctx) {
  detail::wg_ctx_destroy(ctx);
}

// fence / quiet are ordering points, not completion waits
// (src/ipc/context_ipc_device.cpp:90-102, where both are a sequentially
// consistent store per PE).  Every operation of this library has already
// performed its loads and stores when it returns, so what is left to do is to
// publish them: a release at agent scope.
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_fence(rocshmem_ctx_t ctx) {
  detail::ctx_release(detail::ctx_of(ctx));
}
__device__ ATTR_NO_INLINE inline void rocshmem_fence() { detail::fence_release(); }
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_fence(rocshmem_ctx_t ctx, int) {
  detail::ctx_release(detail::ctx_of(ctx));
}
__device__ ATTR_NO_INLINE inline void rocshmem_fence(int) { detail::fence_release(); }
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_quiet(rocshmem_ctx_t ctx) {
  detail::ctx_release(detail::ctx_of(ctx));
}
__device__ ATTR_NO_INLINE inline void rocshmem_quiet() { detail::fence_release(); }
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_threadfence_system(rocshmem_ctx_t) {
  __threadfence_system();
}
__device__ ATTR_NO_INLINE inline void rocshmem_threadfence_system() { __threadfence_system(); }

// src/rocshmem_gpu.cpp:606-635
__device__ inline int rocshmem_ctx_n_pes(rocshmem_ctx_t ctx) {
  const detail::TeamInfo *ti = reinterpret_cast<const detail::TeamInfo *>(ctx.team_opaque);
  return ti ? ti->size : detail::g_state.n_pes;
}
__device__ inline int rocshmem_n_pes() { return detail::g_state.n_pes; }
__device__ inline int rocshmem_ctx_my_pe(rocshmem_ctx_t ctx) {
  const int me = detail::ctx_of(ctx)->my_pe;
  const detail::TeamInfo *ti = reinterpret_cast<const detail::TeamInfo *>(ctx.team_opaque);
  if (!ti) return me;
  const int rel = (me - ti->pe_start) / ti->stride;
  if (me < ti->pe_start || (me - ti->pe_start) % ti->stride || rel >= ti->size) return -1;
  return rel;
}
__device__ inline int rocshmem_my_pe() { return detail::acting_pe(); }

// src/team.cpp:51-111
__device__ inline int rocshmem_team_translate_pe(rocshmem_team_t src_team, int src_pe,
                                                 rocshmem_team_t dest_team) {
  if (src_team == ROCSHMEM_TEAM_INVALID || dest_team == ROCSHMEM_TEAM_INVALID) return -1;
  const detail::Team *s = detail::team_of(src_team);
  const detail::Team *d = detail::team_of(dest_team);
  if (!s || !d) return -1;
  const int world = s->wrt_world.pe_start + s->wrt_world.stride * src_pe;
  const int off = world - d->wrt_world.pe_start;
  if (off < 0 || off % d->wrt_world.stride) return -1;
  const int rel = off / d->wrt_world.stride;
  return rel >= d->num_pes ? -1 : rel;
}

__device__ ATTR_NO_INLINE inline void rocshmem_ctx_wg_barrier_all(rocshmem_ctx_t ctx) {
  detail::barrier_all(detail::ctx_of(ctx));
}
__device__ ATTR_NO_INLINE inline void rocshmem_wg_barrier_all() {
  rocshmem_ctx_wg_barrier_all(rocshmem_ctx_t{nullptr, nullptr});
}
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_wg_sync_all(rocshmem_ctx_t ctx) {
  detail::sync_all(detail::ctx_of(ctx));
}
__device__ ATTR_NO_INLINE inline void rocshmem_wg_sync_all() {
  rocshmem_ctx_wg_sync_all(rocshmem_ctx_t{nullptr, nullptr});
}
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_wg_team_sync(rocshmem_ctx_t ctx,
                                                                rocshmem_team_t team) {
  detail::Team *t = detail::team_of(team);
  if (t) {
    detail::Context *c = detail::ctx_of(ctx);
    detail::team_pad_sync(c, t, detail::SYNC_BARRIER, detail::publish_of(c));
  }
}
__device__ ATTR_NO_INLINE inline void rocshmem_wg_team_sync(rocshmem_team_t team) {
  rocshmem_ctx_wg_team_sync(rocshmem_ctx_t{nullptr, nullptr}, team);
}

// Address of `dest` on PE `pe` for direct loads and stores.  The reference's
// load/store path returns nullptr here (src/ipc/context_ipc_device.cpp:104-107);
// with every slice in one address space the real address is available.
__device__ ATTR_NO_INLINE inline void *rocshmem_ptr(const void *dest, int pe) {
  return detail::remote_addr(detail::ctx_of(rocshmem_ctx_t{nullptr, nullptr}),
                             static_cast<char *>(const_cast<void *>(dest)), pe);
}

#endif  // __HIPCC__

}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_ROCSHMEM_HPP_
