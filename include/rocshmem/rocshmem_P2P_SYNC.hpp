// Point-to-point synchronisation: wait_until, its any/all/some forms, test.
//
// Names and arguments follow include/rocshmem/rocshmem_P2P_SYNC.hpp of the
// reference; behaviour follows src/context_tmpl_device.hpp:201-377, including
// the return conventions (any: SIZE_MAX when nothing can be waited on; some:
// count found by the first successful sweep) and the _vector forms, which the
// reference leaves as stubs that wait for nothing.  A successful wait or test
// also acquires, so a payload published before the awaited value is visible.
#ifndef ROCSHMEM_AMD_P2P_SYNC_HPP_
#define ROCSHMEM_AMD_P2P_SYNC_HPP_

#include "detail/sync.hpp"
#include "detail/type_lists.hpp"

namespace rocshmem {

#if defined(__HIPCC__)

#define ROCSHMEM_AMD_WAIT(T, TN)                                                          \
  __device__ inline void rocshmem_##TN##_wait_until(T *ivars, int cmp, T val) {           \
    detail::wait_until(ivars, cmp, val);                                                  \
  }                                                                                       \
  __device__ inline size_t rocshmem_##TN##_wait_until_any(                                \
      T *ivars, size_t nelems, const int *status, int cmp, T val) {                       \
    return detail::wait_until_any(ivars, nelems, status, cmp, val);                       \
  }                                                                                       \
  __device__ inline void rocshmem_##TN##_wait_until_all(                                  \
      T *ivars, size_t nelems, const int *status, int cmp, T val) {                       \
    detail::wait_until_all(ivars, nelems, status, cmp, val);                              \
  }                                                                                       \
  __device__ inline size_t rocshmem_##TN##_wait_until_some(                               \
      T *ivars, size_t nelems, size_t *indices, const int *status, int cmp, T val) {      \
    return detail::wait_until_some(ivars, nelems, indices, status, cmp, val);             \
  }                                                                                       \
  __device__ inline size_t rocshmem_##TN##_wait_until_any_vector(                         \
      T *, size_t, const int *, int, T) {                                                 \
    return 0;                                                                             \
  }                                                                                       \
  __device__ inline void rocshmem_##TN##_wait_until_all_vector(T *, size_t, const int *,  \
                                                               int, T) {}                 \
  __device__ inline size_t rocshmem_##TN##_wait_until_some_vector(                        \
      T *, size_t, size_t *, const int *, int, T) {                                       \
    return 0;                                                                             \
  }                                                                                       \
  __device__ inline int rocshmem_##TN##_test(T *ivars, int cmp, T val) {                  \
    return detail::test(ivars, cmp, val);                                                 \
  }

ROCSHMEM_AMD_WAIT_TYPES(ROCSHMEM_AMD_WAIT)
#undef ROCSHMEM_AMD_WAIT

#endif  // __HIPCC__

}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_P2P_SYNC_HPP_
