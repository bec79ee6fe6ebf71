// Work-group (_wg) and wavefront (_wave) remote memory access.
//
// Same names and arguments as include/rocshmem/rocshmem_RMA_X.hpp of the
// reference.  Every thread of the work-group (or every active lane of the
// wavefront) must call with identical arguments.  As in the reference
// (src/rocshmem_gpu.cpp:753-872) `pe` is a world PE here — these calls do not
// translate through the context's team — and zero-length calls do nothing.
// The _nbi_wave forms return once the copy is issued and complete at the
// calling wavefront's quiet; the _nbi_wg forms complete like the blocking ones
// (a quiet by one thread could not answer for the other wavefronts' stores).
#ifndef ROCSHMEM_AMD_RMA_X_HPP_
#define ROCSHMEM_AMD_RMA_X_HPP_

#include "detail/rma.hpp"
#include "detail/type_lists.hpp"

namespace rocshmem {

#if defined(__HIPCC__)

#define ROCSHMEM_AMD_MEM_X(DIR, SFX, IMPL)                                                \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##DIR##mem##SFX(                     \
      rocshmem_ctx_t ctx, void *dest, const void *source, size_t nelems, int pe) {        \
    if (nelems == 0) return;                                                              \
    detail::IMPL(detail::ctx_of(ctx), dest, source, nelems, pe);                          \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_##DIR##mem##SFX(                         \
      void *dest, const void *source, size_t nelems, int pe) {                            \
    rocshmem_ctx_##DIR##mem##SFX(rocshmem_ctx_t{nullptr, nullptr}, dest, source, nelems,  \
                                 pe);                                                     \
  }

ROCSHMEM_AMD_MEM_X(put, _wg, putmem_wg)
ROCSHMEM_AMD_MEM_X(put, _nbi_wg, putmem_wg)
ROCSHMEM_AMD_MEM_X(put, _wave, putmem_wave)
ROCSHMEM_AMD_MEM_X(put, _nbi_wave, putmem_nbi_wave)
ROCSHMEM_AMD_MEM_X(get, _wg, getmem_wg)
ROCSHMEM_AMD_MEM_X(get, _nbi_wg, getmem_wg)
ROCSHMEM_AMD_MEM_X(get, _wave, getmem_wave)
ROCSHMEM_AMD_MEM_X(get, _nbi_wave, getmem_nbi_wave)
#undef ROCSHMEM_AMD_MEM_X

#define ROCSHMEM_AMD_TYPED_X1(T, TN, DIR, SFX)                                            \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_##DIR##SFX(                   \
      rocshmem_ctx_t ctx, T *dest, const T *source, size_t nelems, int pe) {              \
    rocshmem_ctx_##DIR##mem##SFX(ctx, dest, source, nelems * sizeof(T), pe);              \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_##DIR##SFX(                       \
      T *dest, const T *source, size_t nelems, int pe) {                                  \
    rocshmem_##DIR##mem##SFX(dest, source, nelems * sizeof(T), pe);                       \
  }

#define ROCSHMEM_AMD_TYPED_X(T, TN)                                                       \
  ROCSHMEM_AMD_TYPED_X1(T, TN, put, _wg)                                                  \
  ROCSHMEM_AMD_TYPED_X1(T, TN, put, _nbi_wg)                                              \
  ROCSHMEM_AMD_TYPED_X1(T, TN, put, _wave)                                                \
  ROCSHMEM_AMD_TYPED_X1(T, TN, put, _nbi_wave)                                            \
  ROCSHMEM_AMD_TYPED_X1(T, TN, get, _wg)                                                  \
  ROCSHMEM_AMD_TYPED_X1(T, TN, get, _nbi_wg)                                              \
  ROCSHMEM_AMD_TYPED_X1(T, TN, get, _wave)                                                \
  ROCSHMEM_AMD_TYPED_X1(T, TN, get, _nbi_wave)

ROCSHMEM_AMD_RMA_TYPES(ROCSHMEM_AMD_TYPED_X)
#undef ROCSHMEM_AMD_TYPED_X
#undef ROCSHMEM_AMD_TYPED_X1

#endif  // __HIPCC__

}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_RMA_X_HPP_
