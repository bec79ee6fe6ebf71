// Thread-granularity remote memory access: putmem/getmem, typed put/get/p/g
// and their _nbi forms, with and without an explicit context.
//
// Same names, argument order and PE-translation rule as the reference
// (include/rocshmem/rocshmem_RMA.hpp; src/rocshmem_gpu.cpp:327-451): these
// calls map a team-relative `pe` through the context's team; zero-length
// calls do nothing; the _nbi forms return once the copy is issued and complete
// at the calling thread's rocshmem_ctx_quiet / rocshmem_ctx_fence.
#ifndef ROCSHMEM_AMD_RMA_HPP_
#define ROCSHMEM_AMD_RMA_HPP_

#include "detail/rma.hpp"
#include "detail/type_lists.hpp"

namespace rocshmem {

#if defined(__HIPCC__)

__device__ ATTR_NO_INLINE inline void rocshmem_ctx_putmem(rocshmem_ctx_t ctx, void *dest,
                                                   const void *source, size_t nelems,
                                                   int pe) {
  if (nelems == 0) return;
  detail::putmem(detail::ctx_of(ctx), dest, source, nelems, detail::translate_pe(ctx, pe));
}
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_getmem(rocshmem_ctx_t ctx, void *dest,
                                                   const void *source, size_t nelems,
                                                   int pe) {
  if (nelems == 0) return;
  detail::getmem(detail::ctx_of(ctx), dest, source, nelems, detail::translate_pe(ctx, pe));
}
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_putmem_nbi(rocshmem_ctx_t ctx, void *dest,
                                                       const void *source,
                                                       size_t nelems, int pe) {
  if (nelems == 0) return;
  detail::putmem_nbi(detail::ctx_of(ctx), dest, source, nelems, detail::translate_pe(ctx, pe));
}
__device__ ATTR_NO_INLINE inline void rocshmem_ctx_getmem_nbi(rocshmem_ctx_t ctx, void *dest,
                                                       const void *source,
                                                       size_t nelems, int pe) {
  if (nelems == 0) return;
  detail::getmem_nbi(detail::ctx_of(ctx), dest, source, nelems, detail::translate_pe(ctx, pe));
}
__device__ ATTR_NO_INLINE inline void rocshmem_putmem(void *dest, const void *source,
                                               size_t nelems, int pe) {
  rocshmem_ctx_putmem(rocshmem_ctx_t{nullptr, nullptr}, dest, source, nelems, pe);
}
__device__ ATTR_NO_INLINE inline void rocshmem_getmem(void *dest, const void *source,
                                               size_t nelems, int pe) {
  rocshmem_ctx_getmem(rocshmem_ctx_t{nullptr, nullptr}, dest, source, nelems, pe);
}
__device__ ATTR_NO_INLINE inline void rocshmem_putmem_nbi(void *dest, const void *source,
                                                   size_t nelems, int pe) {
  rocshmem_ctx_putmem_nbi(rocshmem_ctx_t{nullptr, nullptr}, dest, source, nelems, pe);
}
__device__ ATTR_NO_INLINE inline void rocshmem_getmem_nbi(void *dest, const void *source,
                                                   size_t nelems, int pe) {
  rocshmem_ctx_getmem_nbi(rocshmem_ctx_t{nullptr, nullptr}, dest, source, nelems, pe);
}

#define ROCSHMEM_AMD_TYPED_RMA(T, TN)                                                    \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_put(                         \
      rocshmem_ctx_t ctx, T *dest, const T *source, size_t nelems, int pe) {             \
    rocshmem_ctx_putmem(ctx, dest, source, nelems * sizeof(T), pe);                      \
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_put(T *dest, const T *source,    \
                                                            size_t nelems, int pe) {     \
    rocshmem_putmem(dest, source, nelems * sizeof(T), pe);                               \
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_put_nbi(                     \
      rocshmem_ctx_t ctx, T *dest, const T *source, size_t nelems, int pe) {             \
    rocshmem_ctx_putmem_nbi(ctx, dest, source, nelems * sizeof(T), pe);                  \
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_put_nbi(T *dest, const T *source,\
                                                                size_t nelems, int pe) { \
    rocshmem_putmem_nbi(dest, source, nelems * sizeof(T), pe);                           \
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_p(rocshmem_ctx_t ctx,        \
                                                              T *dest, T value, int pe) {\
    detail::put_value<T>(detail::ctx_of(ctx), dest, value, detail::translate_pe(ctx, pe));\
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_p(T *dest, T value, int pe) {    \
    rocshmem_ctx_##TN##_p(rocshmem_ctx_t{nullptr, nullptr}, dest, value, pe);            \
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_get(                         \
      rocshmem_ctx_t ctx, T *dest, const T *source, size_t nelems, int pe) {             \
    rocshmem_ctx_getmem(ctx, dest, source, nelems * sizeof(T), pe);                      \
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_get(T *dest, const T *source,    \
                                                            size_t nelems, int pe) {     \
    rocshmem_getmem(dest, source, nelems * sizeof(T), pe);                               \
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_get_nbi(                     \
      rocshmem_ctx_t ctx, T *dest, const T *source, size_t nelems, int pe) {             \
    rocshmem_ctx_getmem_nbi(ctx, dest, source, nelems * sizeof(T), pe);                  \
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_get_nbi(T *dest, const T *source,\
                                                                size_t nelems, int pe) { \
    rocshmem_getmem_nbi(dest, source, nelems * sizeof(T), pe);                           \
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline T rocshmem_ctx_##TN##_g(rocshmem_ctx_t ctx,           \
                                                           const T *source, int pe) {    \
    return detail::get_value<T>(detail::ctx_of(ctx), source, detail::translate_pe(ctx, pe)); \
  }                                                                                      \
  __device__ ATTR_NO_INLINE inline T rocshmem_##TN##_g(const T *source, int pe) {        \
    return rocshmem_ctx_##TN##_g(rocshmem_ctx_t{nullptr, nullptr}, source, pe);          \
  }

ROCSHMEM_AMD_RMA_TYPES(ROCSHMEM_AMD_TYPED_RMA)
#undef ROCSHMEM_AMD_TYPED_RMA

#endif  // __HIPCC__

}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_RMA_HPP_
