// Put-with-signal and signal_fetch.
//
// Names and arguments follow include/rocshmem/rocshmem_SIG_OP.hpp of the
// reference.  The payload is copied, ordered, and then exactly one lane (the
// calling thread / the lowest active lane of the wavefront / thread 0 of the
// work-group) updates the 64-bit signal word on the target PE: SET stores,
// ADD adds (src/ipc/context_ipc_device.cpp:221-298).  A zero-length call does
// nothing at all — the signal is not updated (src/context_device.cpp:251-262).
// `pe` is a world PE.
#ifndef ROCSHMEM_AMD_SIG_OP_HPP_
#define ROCSHMEM_AMD_SIG_OP_HPP_

#include "detail/rma.hpp"
#include "detail/type_lists.hpp"

namespace rocshmem {

#if defined(__HIPCC__)

#define ROCSHMEM_AMD_PUTMEM_SIGNAL(SFX, IMPL)                                             \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_putmem_signal##SFX(                  \
      rocshmem_ctx_t ctx, void *dest, const void *source, size_t nelems,                  \
      uint64_t *sig_addr, uint64_t signal, int sig_op, int pe) {                          \
    if (nelems == 0) return;                                                              \
    detail::IMPL(detail::ctx_of(ctx), dest, source, nelems, sig_addr, signal, sig_op,     \
                 pe);                                                                     \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_putmem_signal##SFX(                      \
      void *dest, const void *source, size_t nelems, uint64_t *sig_addr,                  \
      uint64_t signal, int sig_op, int pe) {                                              \
    rocshmem_ctx_putmem_signal##SFX(rocshmem_ctx_t{nullptr, nullptr}, dest, source,       \
                                    nelems, sig_addr, signal, sig_op, pe);                \
  }

ROCSHMEM_AMD_PUTMEM_SIGNAL(, putmem_signal)
ROCSHMEM_AMD_PUTMEM_SIGNAL(_nbi, putmem_signal)
ROCSHMEM_AMD_PUTMEM_SIGNAL(_wave, putmem_signal_wave)
ROCSHMEM_AMD_PUTMEM_SIGNAL(_nbi_wave, putmem_signal_wave)
ROCSHMEM_AMD_PUTMEM_SIGNAL(_wg, putmem_signal_wg)
ROCSHMEM_AMD_PUTMEM_SIGNAL(_nbi_wg, putmem_signal_wg)
#undef ROCSHMEM_AMD_PUTMEM_SIGNAL

#define ROCSHMEM_AMD_TYPED_SIGNAL1(T, TN, SFX)                                            \
  __device__ ATTR_NO_INLINE inline void rocshmem_ctx_##TN##_put_signal##SFX(              \
      rocshmem_ctx_t ctx, T *dest, const T *source, size_t nelems, uint64_t *sig_addr,    \
      uint64_t signal, int sig_op, int pe) {                                              \
    rocshmem_ctx_putmem_signal##SFX(ctx, dest, source, nelems * sizeof(T), sig_addr,      \
                                    signal, sig_op, pe);                                  \
  }                                                                                       \
  __device__ ATTR_NO_INLINE inline void rocshmem_##TN##_put_signal##SFX(                  \
      T *dest, const T *source, size_t nelems, uint64_t *sig_addr, uint64_t signal,       \
      int sig_op, int pe) {                                                               \
    rocshmem_putmem_signal##SFX(dest, source, nelems * sizeof(T), sig_addr, signal,       \
                                sig_op, pe);                                              \
  }

#define ROCSHMEM_AMD_TYPED_SIGNAL(T, TN)     \
  ROCSHMEM_AMD_TYPED_SIGNAL1(T, TN, )        \
  ROCSHMEM_AMD_TYPED_SIGNAL1(T, TN, _nbi)    \
  ROCSHMEM_AMD_TYPED_SIGNAL1(T, TN, _wave)   \
  ROCSHMEM_AMD_TYPED_SIGNAL1(T, TN, _nbi_wave) \
  ROCSHMEM_AMD_TYPED_SIGNAL1(T, TN, _wg)     \
  ROCSHMEM_AMD_TYPED_SIGNAL1(T, TN, _nbi_wg)

ROCSHMEM_AMD_RMA_TYPES(ROCSHMEM_AMD_TYPED_SIGNAL)
#undef ROCSHMEM_AMD_TYPED_SIGNAL
#undef ROCSHMEM_AMD_TYPED_SIGNAL1

__device__ ATTR_NO_INLINE inline uint64_t rocshmem_signal_fetch(const uint64_t *sig_addr) {
  return detail::signal_fetch(sig_addr);
}
__device__ ATTR_NO_INLINE inline uint64_t rocshmem_signal_fetch_wg(const uint64_t *sig_addr) {
  return detail::signal_fetch_wg(sig_addr);
}
__device__ ATTR_NO_INLINE inline uint64_t rocshmem_signal_fetch_wave(const uint64_t *sig_addr) {
  return detail::signal_fetch_wave(sig_addr);
}

#endif  // __HIPCC__

}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_SIG_OP_HPP_
