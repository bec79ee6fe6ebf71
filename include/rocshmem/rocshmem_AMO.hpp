// Atomic memory operations on symmetric objects.
//
// Names and arguments follow include/rocshmem/rocshmem_AMO.hpp of the
// reference.  `pe` is a world PE (no team translation, as in
// src/rocshmem_gpu.cpp:641-748).  fetch_inc / inc / fetch are fetch_add(1) /
// add(1) / an atomic read, as there (:657-684).  swap and the bitwise
// operations, which the reference's IPC path only stubs with assert(false)
// (src/ipc/context_ipc_tmpl_device.hpp:91-128), are real atomics here.
// Returned values keep their full width.
#ifndef ROCSHMEM_AMD_AMO_HPP_
#define ROCSHMEM_AMD_AMO_HPP_

#include "detail/rma.hpp"
#include "detail/type_lists.hpp"

namespace rocshmem {

#if defined(__HIPCC__)

#define ROCSHMEM_AMD_AMO_STANDARD(T, TN)                                                  \
  __device__ ATTR_NO_INLINE inline T rocshmem_ctx_##TN##_atomic_fetch_add(                \
      rocshmem_ctx_t ctx, T *dest, T value, int pe) {                                     \
    detail::Context *c = detail::ctx_of(ctx);                                             \
    return detail::amo_fetch_add(detail::remote_addr(c, dest, pe), value,                 \
                                 detail::no_store_order(c));                              \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline T rocshmem_##TN##_atomic_fetch_add(T *dest, T value,   \
                                                                     int pe) {            \
    return rocshmem_ctx_##TN##_atomic_fetch_add(rocshmem_ctx_t{nullptr, nullptr}, dest,   \
                                                value, pe);                               \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_atomic_add(                   \
      rocshmem_ctx_t ctx, T *dest, T value, int pe) {                                     \
    detail::Context *c = detail::ctx_of(ctx);                                             \
    detail::amo_add(detail::remote_addr(c, dest, pe), value, detail::no_store_order(c));  \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_atomic_add(T *dest, T value,      \
                                                                  int pe) {               \
    rocshmem_ctx_##TN##_atomic_add(rocshmem_ctx_t{nullptr, nullptr}, dest, value, pe);    \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline T rocshmem_ctx_##TN##_atomic_fetch_inc(                \
      rocshmem_ctx_t ctx, T *dest, int pe) {                                              \
    return rocshmem_ctx_##TN##_atomic_fetch_add(ctx, dest, static_cast<T>(1), pe);        \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline T rocshmem_##TN##_atomic_fetch_inc(T *dest, int pe) {  \
    return rocshmem_##TN##_atomic_fetch_add(dest, static_cast<T>(1), pe);                 \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_atomic_inc(                   \
      rocshmem_ctx_t ctx, T *dest, int pe) {                                              \
    rocshmem_ctx_##TN##_atomic_add(ctx, dest, static_cast<T>(1), pe);                     \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_atomic_inc(T *dest, int pe) {     \
    rocshmem_##TN##_atomic_add(dest, static_cast<T>(1), pe);                              \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline T rocshmem_ctx_##TN##_atomic_compare_swap(             \
      rocshmem_ctx_t ctx, T *dest, T cond, T value, int pe) {                             \
    detail::Context *c = detail::ctx_of(ctx);                                             \
    return detail::amo_fetch_cas(detail::remote_addr(c, dest, pe), cond, value,           \
                                 detail::no_store_order(c));                              \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline T rocshmem_##TN##_atomic_compare_swap(                 \
      T *dest, T cond, T value, int pe) {                                                 \
    return rocshmem_ctx_##TN##_atomic_compare_swap(rocshmem_ctx_t{nullptr, nullptr}, dest,\
                                                   cond, value, pe);                      \
  }

#define ROCSHMEM_AMD_AMO_EXTENDED(T, TN)                                                  \
  __device__ ATTR_NO_INLINE inline T rocshmem_ctx_##TN##_atomic_fetch(                    \
      rocshmem_ctx_t ctx, T *source, int pe) {                                            \
    detail::Context *c = detail::ctx_of(ctx);                                             \
    return detail::amo_fetch(detail::remote_addr(c, source, pe),                          \
                             detail::no_store_order(c));                                  \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline T rocshmem_##TN##_atomic_fetch(T *source, int pe) {    \
    return rocshmem_ctx_##TN##_atomic_fetch(rocshmem_ctx_t{nullptr, nullptr}, source, pe);\
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_atomic_set(                   \
      rocshmem_ctx_t ctx, T *dest, T value, int pe) {                                     \
    detail::Context *c = detail::ctx_of(ctx);                                             \
    detail::amo_set(detail::remote_addr(c, dest, pe), value, detail::no_store_order(c));  \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_atomic_set(T *dest, T value,      \
                                                                  int pe) {               \
    rocshmem_ctx_##TN##_atomic_set(rocshmem_ctx_t{nullptr, nullptr}, dest, value, pe);    \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline T rocshmem_ctx_##TN##_atomic_swap(                     \
      rocshmem_ctx_t ctx, T *dest, T value, int pe) {                                     \
    detail::Context *c = detail::ctx_of(ctx);                                             \
    return detail::amo_swap(detail::remote_addr(c, dest, pe), value,                      \
                            detail::no_store_order(c));                                   \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline T rocshmem_##TN##_atomic_swap(T *dest, T value,        \
                                                                 int pe) {                \
    return rocshmem_ctx_##TN##_atomic_swap(rocshmem_ctx_t{nullptr, nullptr}, dest, value, \
                                           pe);                                           \
  }

#define ROCSHMEM_AMD_AMO_BITWISE1(T, TN, OP)                                              \
  __device__ ATTR_NO_INLINE inline T rocshmem_ctx_##TN##_atomic_fetch_##OP(               \
      rocshmem_ctx_t ctx, T *dest, T value, int pe) {                                     \
    detail::Context *c = detail::ctx_of(ctx);                                             \
    return detail::amo_fetch_##OP(detail::remote_addr(c, dest, pe), value,                \
                                  detail::no_store_order(c));                             \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline T rocshmem_##TN##_atomic_fetch_##OP(T *dest, T value,  \
                                                                      int pe) {           \
    return rocshmem_ctx_##TN##_atomic_fetch_##OP(rocshmem_ctx_t{nullptr, nullptr}, dest,  \
                                                 value, pe);                              \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_atomic_##OP(                  \
      rocshmem_ctx_t ctx, T *dest, T value, int pe) {                                     \
    (void)rocshmem_ctx_##TN##_atomic_fetch_##OP(ctx, dest, value, pe);                    \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_atomic_##OP(T *dest, T value,     \
                                                                   int pe) {              \
    (void)rocshmem_##TN##_atomic_fetch_##OP(dest, value, pe);                             \
  }

#define ROCSHMEM_AMD_AMO_BITWISE(T, TN) \
  ROCSHMEM_AMD_AMO_BITWISE1(T, TN, and) \
  ROCSHMEM_AMD_AMO_BITWISE1(T, TN, or)  \
  ROCSHMEM_AMD_AMO_BITWISE1(T, TN, xor)

ROCSHMEM_AMD_AMO_STANDARD_TYPES(ROCSHMEM_AMD_AMO_STANDARD)
ROCSHMEM_AMD_AMO_EXTENDED_TYPES(ROCSHMEM_AMD_AMO_EXTENDED)
ROCSHMEM_AMD_AMO_BITWISE_TYPES(ROCSHMEM_AMD_AMO_BITWISE)
#undef ROCSHMEM_AMD_AMO_STANDARD
#undef ROCSHMEM_AMD_AMO_EXTENDED
#undef ROCSHMEM_AMD_AMO_BITWISE
#undef ROCSHMEM_AMD_AMO_BITWISE1

#endif  // __HIPCC__

}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_AMO_HPP_
