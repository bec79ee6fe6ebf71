// Work-group collectives: all-reduce, alltoall, broadcast, fcollect.
//
// Names and arguments follow include/rocshmem/rocshmem_COLL.hpp of the
// reference.  Every thread of one work-group per team member calls with
// identical arguments.  A call with zero elements returns at once without
// synchronising (src/context_tmpl_device.hpp:82-87,142-147,170-175).
//
// Additions that have no counterpart in the reference: bf16 sums with fp32
// accumulation (rocshmem_ctx_bf16_sum_wg_reduce) and the OpenSHMEM-style
// aliases rocshmem_ctx_<T>_<op>_wg_to_all, rocshmem_ctx_alltoallmem[_wg],
// rocshmem_ctx_broadcastmem[_wg] and rocshmem_ctx_broadcast (bytes).
#ifndef ROCSHMEM_AMD_COLL_HPP_
#define ROCSHMEM_AMD_COLL_HPP_

#include "detail/collectives.hpp"
#include "detail/type_lists.hpp"

namespace rocshmem {

#if defined(__HIPCC__)

#define ROCSHMEM_AMD_REDUCE1(T, TN, OPN, OP)                                              \
  __device__ ATTR_NO_INLINE inline int rocshmem_ctx_##TN##_##OPN##_wg_reduce(             \
      rocshmem_ctx_t ctx, rocshmem_team_t team, T *dest, const T *source, int nreduce) {  \
    if (nreduce == 0) return ROCSHMEM_SUCCESS;                                            \
    detail::Team *t = detail::team_of(team);                                              \
    if (!t) return ROCSHMEM_ERROR;                                                        \
    return detail::wg_reduce<T, OP>(detail::ctx_of(ctx), t, dest, source, nreduce);       \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline int rocshmem_ctx_##TN##_##OPN##_wg_to_all(             \
      rocshmem_ctx_t ctx, rocshmem_team_t team, T *dest, const T *source, int nreduce) {  \
    return rocshmem_ctx_##TN##_##OPN##_wg_reduce(ctx, team, dest, source, nreduce);       \
  }

#define ROCSHMEM_AMD_REDUCE_ARITH(T, TN)          \
  ROCSHMEM_AMD_REDUCE1(T, TN, sum, ROCSHMEM_SUM)  \
  ROCSHMEM_AMD_REDUCE1(T, TN, min, ROCSHMEM_MIN)  \
  ROCSHMEM_AMD_REDUCE1(T, TN, max, ROCSHMEM_MAX)  \
  ROCSHMEM_AMD_REDUCE1(T, TN, prod, ROCSHMEM_PROD)
#define ROCSHMEM_AMD_REDUCE_INT(T, TN)            \
  ROCSHMEM_AMD_REDUCE_ARITH(T, TN)                \
  ROCSHMEM_AMD_REDUCE1(T, TN, or, ROCSHMEM_OR)    \
  ROCSHMEM_AMD_REDUCE1(T, TN, and, ROCSHMEM_AND)  \
  ROCSHMEM_AMD_REDUCE1(T, TN, xor, ROCSHMEM_XOR)

ROCSHMEM_AMD_INT_REDUCE_TYPES(ROCSHMEM_AMD_REDUCE_INT)
ROCSHMEM_AMD_FLOAT_REDUCE_TYPES(ROCSHMEM_AMD_REDUCE_ARITH)
#undef ROCSHMEM_AMD_REDUCE_INT
#undef ROCSHMEM_AMD_REDUCE_ARITH
#undef ROCSHMEM_AMD_REDUCE1

__device__ ATTR_NO_INLINE inline int rocshmem_ctx_bf16_sum_wg_reduce(
    rocshmem_ctx_t ctx, rocshmem_team_t team, rocshmem_bf16 *dest,
    const rocshmem_bf16 *source, int nreduce) {
  if (nreduce == 0) return ROCSHMEM_SUCCESS;
  detail::Team *t = detail::team_of(team);
  if (!t) return ROCSHMEM_ERROR;
  return detail::wg_reduce<detail::Bf16Tag, ROCSHMEM_SUM>(
      detail::ctx_of(ctx), t, reinterpret_cast<uint16_t *>(dest),
      reinterpret_cast<const uint16_t *>(source), nreduce);
}
__device__ ATTR_NO_INLINE inline int rocshmem_ctx_bf16_sum_wg_to_all(
    rocshmem_ctx_t ctx, rocshmem_team_t team, rocshmem_bf16 *dest,
    const rocshmem_bf16 *source, int nreduce) {
  return rocshmem_ctx_bf16_sum_wg_reduce(ctx, team, dest, source, nreduce);
}

// Untyped forms: nelems counts bytes per team member.
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_alltoallmem_wg(
    rocshmem_ctx_t ctx, rocshmem_team_t team, void *dest, const void *source,
    size_t nelems) {
  detail::Team *t = detail::team_of(team);
  if (nelems == 0 || !t) return;  // not a member of `team`: nothing to take part in
  detail::wg_alltoall(detail::ctx_of(ctx), t, dest, source, nelems);
}
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_broadcastmem_wg(
    rocshmem_ctx_t ctx, rocshmem_team_t team, void *dest, const void *source,
    size_t nelems, int pe_root) {
  detail::Team *t = detail::team_of(team);
  if (nelems == 0 || !t) return;
  detail::wg_broadcast(detail::ctx_of(ctx), t, dest, source, nelems, pe_root);
}
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_fcollectmem_wg(
    rocshmem_ctx_t ctx, rocshmem_team_t team, void *dest, const void *source,
    size_t nelems) {
  detail::Team *t = detail::team_of(team);
  if (nelems == 0 || !t) return;
  detail::wg_fcollect(detail::ctx_of(ctx), t, dest, source, nelems);
}

// The same three under the OpenSHMEM 1.5 spellings (no granularity suffix):
// still work-group calls, every thread of the work-group with equal arguments.
__device__ inline void rocshmem_ctx_alltoallmem(rocshmem_ctx_t ctx, rocshmem_team_t team,
                                                void *dest, const void *source,
                                                size_t nelems) {
  rocshmem_ctx_alltoallmem_wg(ctx, team, dest, source, nelems);
}
__device__ inline void rocshmem_ctx_broadcastmem(rocshmem_ctx_t ctx, rocshmem_team_t team,
                                                 void *dest, const void *source, size_t nelems,
                                                 int pe_root) {
  rocshmem_ctx_broadcastmem_wg(ctx, team, dest, source, nelems, pe_root);
}
__device__ inline void rocshmem_ctx_broadcast(rocshmem_ctx_t ctx, rocshmem_team_t team,
                                              void *dest, const void *source, size_t nelems,
                                              int pe_root) {
  rocshmem_ctx_broadcastmem_wg(ctx, team, dest, source, nelems, pe_root);
}
__device__ inline void rocshmem_ctx_fcollectmem(rocshmem_ctx_t ctx, rocshmem_team_t team,
                                                void *dest, const void *source,
                                                size_t nelems) {
  rocshmem_ctx_fcollectmem_wg(ctx, team, dest, source, nelems);
}

#define ROCSHMEM_AMD_COLL(T, TN)                                                          \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_wg_alltoall(                  \
      rocshmem_ctx_t ctx, rocshmem_team_t team, T *dest, const T *source, int nelems) {   \
    rocshmem_ctx_alltoallmem_wg(ctx, team, dest, source,                                  \
                                static_cast<size_t>(nelems) * sizeof(T));                 \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_wg_broadcast(                 \
      rocshmem_ctx_t ctx, rocshmem_team_t team, T *dest, const T *source, int nelems,     \
      int pe_root) {                                                                      \
    rocshmem_ctx_broadcastmem_wg(ctx, team, dest, source,                                 \
                                 static_cast<size_t>(nelems) * sizeof(T), pe_root);       \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_wg_fcollect(                  \
      rocshmem_ctx_t ctx, rocshmem_team_t team, T *dest, const T *source, int nelems) {   \
    rocshmem_ctx_fcollectmem_wg(ctx, team, dest, source,                                  \
                                static_cast<size_t>(nelems) * sizeof(T));                 \
  }

ROCSHMEM_AMD_COLL_TYPES(ROCSHMEM_AMD_COLL)
#undef ROCSHMEM_AMD_COLL

#endif  // __HIPCC__

}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_COLL_HPP_
