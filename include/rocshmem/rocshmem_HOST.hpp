// Host-side data movement, atomics, point-to-point synchronisation and
// collectives: the __host__ halves of include/rocshmem/rocshmem_RMA.hpp,
// rocshmem_AMO.hpp, rocshmem_P2P_SYNC.hpp and rocshmem_COLL.hpp of the
// reference, with the same names and argument lists.
//
// The reference forwards these calls to MPI one-sided operations on a window
// over the symmetric heap (src/host/host.cpp:162-249,
// src/host/host_helpers.hpp:52-88, src/host/host_templates.hpp:40-645).  Here
// every PE is a slice of one device allocation, so a host put/get is a copy
// between the caller's buffer (host or device memory) and a slice, an atomic
// is a one-thread kernel that runs the device atomic, a wait polls the word
// with device-to-host copies on a stream of its own, and collectives are the
// whole-GPU kernels.
//
// Which PE the host acts as: the PE of the context passed in (contexts made
// by rocshmem_ctx_create belong to the PE that was acting then); calls
// without a context act as the current acting PE (rocshmem_emu_set_pe), or,
// in a PE thread (rocshmem_emu_run_pes), as that thread's PE.  Outside PE
// threads a collective is ONE call for the whole team, not one per member; PE
// threads call it once each, as the processes of the reference do.
#ifndef ROCSHMEM_AMD_HOST_HPP_
#define ROCSHMEM_AMD_HOST_HPP_

#include <hip/hip_runtime.h>

#include <chrono>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <type_traits>
#include <vector>

#include "../rocshmem_amd.h"
#include "detail/type_lists.hpp"
#include "rocshmem_common.hpp"

namespace rocshmem {
namespace detail {

// The reference's host calls return void and die inside MPI on a bad
// argument; here a refused call names itself and aborts.
inline void host_require(int rc, const char *what) {
  if (rc != 0) {
    fprintf(stderr, "rocshmem: host call %s refused its arguments (code %d)\n", what, rc);
    abort();
  }
}

// Host collectives return when the data is in place (the reference's
// MPI_Bcast / MPI_Allreduce block): launch, then wait for the null stream.
// The callers are the PEs start, start + stride, ... (size of them, world
// numbering).  Outside PE threads there is one caller and it does the work;
// in PE threads (rocshmem_emu_run_pes) every member calls and the last one to
// arrive does the work for all while the others wait.
template <typename Launch>
inline void host_collective(int start, int stride, int size, Launch &&launch, const char *what) {
  if (!rocshmem_amd_pe_threads_enter(start, stride, size)) return;
  int rc = launch();
  if (rc == 0) rc = rocshmem_amd_stream_sync(nullptr);
  rocshmem_amd_pe_threads_leave(start, stride, size);
  host_require(rc, what);
}
template <typename Launch>
inline void host_team_collective(rocshmem_team_t team, Launch &&launch, const char *what) {
  int start = 0, stride = 1, size = 1;
  host_require(rocshmem_amd_team_active_set(team, &start, &stride, &size), what);
  host_collective(start, stride, size, launch, what);
}

inline int host_pe_of(rocshmem_ctx_t ctx) { return rocshmem_amd_ctx_pe(ctx.ctx_opaque); }

// Element type -> rocshmem_amd_dtype.  Fixed-width names are aliases of the
// basic types on this platform, so they arrive here as those.
template <typename T>
constexpr int host_dtype() {
  if (std::is_same<T, float>::value) return ROCSHMEM_AMD_FLOAT;
  if (std::is_same<T, double>::value) return ROCSHMEM_AMD_DOUBLE;
  if (std::is_same<T, char>::value) return ROCSHMEM_AMD_CHAR;
  if (std::is_same<T, signed char>::value) return ROCSHMEM_AMD_SCHAR;
  if (std::is_same<T, unsigned char>::value) return ROCSHMEM_AMD_UCHAR;
  if (std::is_same<T, short>::value) return ROCSHMEM_AMD_SHORT;
  if (std::is_same<T, unsigned short>::value) return ROCSHMEM_AMD_USHORT;
  if (std::is_same<T, int>::value) return ROCSHMEM_AMD_INT;
  if (std::is_same<T, unsigned int>::value) return ROCSHMEM_AMD_UINT;
  if (std::is_same<T, long>::value) return ROCSHMEM_AMD_LONG;
  if (std::is_same<T, unsigned long>::value) return ROCSHMEM_AMD_ULONG;
  if (std::is_same<T, long long>::value) return ROCSHMEM_AMD_LONGLONG;
  if (std::is_same<T, unsigned long long>::value) return ROCSHMEM_AMD_ULONGLONG;
  return -1;
}

// Comparator table of the reference (src/host/host_templates.hpp:395-424); an
// unknown comparator never holds.
template <typename T>
inline bool host_compare(int cmp, T x, T val) {
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

// Deadline for the bounded forms; a negative limit never expires.
struct HostDeadline {
  std::chrono::steady_clock::time_point end;
  bool bounded;
  explicit HostDeadline(long timeout_ms)
      : end(std::chrono::steady_clock::now() +
            std::chrono::milliseconds(timeout_ms < 0 ? 0 : timeout_ms)),
        bounded(timeout_ms >= 0) {}
  bool passed() const { return bounded && std::chrono::steady_clock::now() >= end; }
};

template <typename T>
inline T host_peek_one(const T *ivar) {
  T v;
  host_require(rocshmem_amd_host_peek(&v, ivar, sizeof(T)), "peek");
  return v;
}

// test (src/host/host_templates.hpp:627-641): one read, one comparison.
template <typename T>
inline int host_test(const T *ivar, int cmp, T val) {
  return host_compare(cmp, host_peek_one(ivar), val) ? 1 : 0;
}

// wait_until (:448-471).  Returns false if the limit ran out first.
template <typename T>
inline bool host_wait_until(const T *ivar, int cmp, T val, long timeout_ms = -1) {
  const HostDeadline limit(timeout_ms);
  while (!host_test(ivar, cmp, val)) {
    if (limit.passed()) return false;
  }
  return true;
}

// First index the status array leaves unmasked; nelems if there is none.  A
// null status masks nothing (the reference's host path dereferences it,
// :486-498; the device path treats null as all zeros).
inline size_t host_first_unmasked(size_t nelems, const int *status) {
  size_t i = 0;
  if (status) {
    while (i < nelems && status[i] != 0) ++i;
  }
  return i;
}

// wait_until_any (:502-531): sweeps from the first unmasked element and
// returns the first index that satisfies; SIZE_MAX for an empty or fully
// masked set (and when the limit runs out, with *timed_out set).
template <typename T>
inline size_t host_wait_until_any(const T *ivars, size_t nelems, const int *status, int cmp, T val,
                                  long timeout_ms = -1, bool *timed_out = nullptr) {
  if (timed_out) *timed_out = false;
  if (!nelems) return SIZE_MAX;
  const size_t pos = host_first_unmasked(nelems, status);
  if (pos == nelems) return SIZE_MAX;
  const HostDeadline limit(timeout_ms);
  std::vector<T> seen(nelems);
  for (;;) {
    host_require(rocshmem_amd_host_peek(seen.data() + pos, ivars + pos, (nelems - pos) * sizeof(T)),
                 "peek");
    for (size_t i = pos; i < nelems; ++i) {
      if (status && status[i]) continue;
      if (host_compare(cmp, seen[i], val)) return i;
    }
    if (limit.passed()) {
      if (timed_out) *timed_out = true;
      return SIZE_MAX;
    }
  }
}

// wait_until_all (:534-560): each unmasked element in turn is waited for; an
// element that held once is not looked at again.
template <typename T>
inline bool host_wait_until_all(const T *ivars, size_t nelems, const int *status, int cmp, T val,
                                long timeout_ms = -1) {
  if (!nelems) return true;
  const size_t pos = host_first_unmasked(nelems, status);
  if (pos == nelems) return true;
  const HostDeadline limit(timeout_ms);
  for (size_t i = pos; i < nelems; ++i) {
    if (status && status[i]) continue;
    while (!host_test(ivars + i, cmp, val)) {
      if (limit.passed()) return false;
    }
  }
  return true;
}

// wait_until_some (:562-598): repeats whole sweeps until one finds at least
// one satisfied element; returns how many that sweep found, their indices in
// ascending order in `indices`.
template <typename T>
inline size_t host_wait_until_some(const T *ivars, size_t nelems, size_t *indices,
                                   const int *status, int cmp, T val, long timeout_ms = -1,
                                   bool *timed_out = nullptr) {
  if (timed_out) *timed_out = false;
  if (!nelems) return 0;
  const size_t pos = host_first_unmasked(nelems, status);
  if (pos == nelems) return 0;
  const HostDeadline limit(timeout_ms);
  std::vector<T> seen(nelems);
  for (;;) {
    host_require(rocshmem_amd_host_peek(seen.data() + pos, ivars + pos, (nelems - pos) * sizeof(T)),
                 "peek");
    size_t n = 0;
    for (size_t i = pos; i < nelems; ++i) {
      if (status && status[i]) continue;
      if (host_compare(cmp, seen[i], val)) indices[n++] = i;
    }
    if (n) return n;
    if (limit.passed()) {
      if (timed_out) *timed_out = true;
      return 0;
    }
  }
}

// Value-initialised T; spelled as a function because T may be a two-word type
// name inside the stamping macros.
template <typename T>
inline T host_zero() {
  return T();
}

template <typename T>
inline T host_amo(int amo_op, rocshmem_ctx_t ctx, T *dest, T value, T cond, int pe,
                  const char *what) {
  T out = T();
  const int me = host_pe_of(ctx);
  host_require(rocshmem_amd_host_amo(amo_op, host_dtype<T>(), rocshmem_amd_pe_ptr(dest, me), &value,
                                     &cond, me, pe, &out),
               what);
  return out;
}

// Forms without a comparison value / without any operand.
template <typename T>
inline T host_amo(int amo_op, rocshmem_ctx_t ctx, T *dest, T value, int pe, const char *what) {
  return host_amo<T>(amo_op, ctx, dest, value, host_zero<T>(), pe, what);
}
template <typename T>
inline T host_amo(int amo_op, rocshmem_ctx_t ctx, T *dest, int pe, const char *what) {
  return host_amo<T>(amo_op, ctx, dest, host_zero<T>(), host_zero<T>(), pe, what);
}

}  // namespace detail

constexpr rocshmem_ctx_t ROCSHMEM_AMD_HOST_DEFAULT_CTX{nullptr, nullptr};

// ---------------------------------------------------------------------------
// RMA (include/rocshmem/rocshmem_RMA.hpp; src/host/host_helpers.hpp:52-88).
// The local buffer may be host memory or device memory.  The _nbi forms are
// complete on return as well (permitted: they may complete at any time up to
// the next quiet).
// ---------------------------------------------------------------------------
// The symmetric side may be given as any PE's address of the object; it is
// taken as the calling PE's.
__host__ inline void rocshmem_ctx_putmem(rocshmem_ctx_t ctx, void *dest, const void *source,
                                         size_t nelems, int pe) {
  const int me = detail::host_pe_of(ctx);
  detail::host_require(rocshmem_amd_host_putmem(nelems ? rocshmem_amd_pe_ptr(dest, me) : dest,
                                                source, nelems, me, pe),
                       "putmem");
}
__host__ inline void rocshmem_putmem(void *dest, const void *source, size_t nelems, int pe) {
  rocshmem_ctx_putmem(ROCSHMEM_AMD_HOST_DEFAULT_CTX, dest, source, nelems, pe);
}
__host__ inline void rocshmem_ctx_getmem(rocshmem_ctx_t ctx, void *dest, const void *source,
                                         size_t nelems, int pe) {
  const int me = detail::host_pe_of(ctx);
  detail::host_require(
      rocshmem_amd_host_getmem(dest, nelems ? rocshmem_amd_pe_ptr(source, me) : source, nelems, me,
                               pe),
      "getmem");
}
__host__ inline void rocshmem_getmem(void *dest, const void *source, size_t nelems, int pe) {
  rocshmem_ctx_getmem(ROCSHMEM_AMD_HOST_DEFAULT_CTX, dest, source, nelems, pe);
}
__host__ inline void rocshmem_ctx_putmem_nbi(rocshmem_ctx_t ctx, void *dest, const void *source,
                                             size_t nelems, int pe) {
  rocshmem_ctx_putmem(ctx, dest, source, nelems, pe);
}
__host__ inline void rocshmem_putmem_nbi(void *dest, const void *source, size_t nelems, int pe) {
  rocshmem_putmem(dest, source, nelems, pe);
}
__host__ inline void rocshmem_ctx_getmem_nbi(rocshmem_ctx_t ctx, void *dest, const void *source,
                                             size_t nelems, int pe) {
  rocshmem_ctx_getmem(ctx, dest, source, nelems, pe);
}
__host__ inline void rocshmem_getmem_nbi(void *dest, const void *source, size_t nelems, int pe) {
  rocshmem_getmem(dest, source, nelems, pe);
}

#define ROCSHMEM_AMD_HOST_RMA(T, TN)                                                              \
  __host__ inline void rocshmem_ctx_##TN##_put(rocshmem_ctx_t ctx, T *dest, const T *source,      \
                                               size_t nelems, int pe) {                           \
    rocshmem_ctx_putmem(ctx, dest, source, nelems * sizeof(T), pe);                               \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_put(T *dest, const T *source, size_t nelems, int pe) {     \
    rocshmem_putmem(dest, source, nelems * sizeof(T), pe);                                        \
  }                                                                                               \
  __host__ inline void rocshmem_ctx_##TN##_put_nbi(rocshmem_ctx_t ctx, T *dest, const T *source,  \
                                                   size_t nelems, int pe) {                       \
    rocshmem_ctx_putmem(ctx, dest, source, nelems * sizeof(T), pe);                               \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_put_nbi(T *dest, const T *source, size_t nelems, int pe) { \
    rocshmem_putmem(dest, source, nelems * sizeof(T), pe);                                        \
  }                                                                                               \
  __host__ inline void rocshmem_ctx_##TN##_p(rocshmem_ctx_t ctx, T *dest, T value, int pe) {      \
    rocshmem_ctx_putmem(ctx, dest, &value, sizeof(T), pe);                                        \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_p(T *dest, T value, int pe) {                              \
    rocshmem_putmem(dest, &value, sizeof(T), pe);                                                 \
  }                                                                                               \
  __host__ inline void rocshmem_ctx_##TN##_get(rocshmem_ctx_t ctx, T *dest, const T *source,      \
                                               size_t nelems, int pe) {                           \
    rocshmem_ctx_getmem(ctx, dest, source, nelems * sizeof(T), pe);                               \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_get(T *dest, const T *source, size_t nelems, int pe) {     \
    rocshmem_getmem(dest, source, nelems * sizeof(T), pe);                                        \
  }                                                                                               \
  __host__ inline void rocshmem_ctx_##TN##_get_nbi(rocshmem_ctx_t ctx, T *dest, const T *source,  \
                                                   size_t nelems, int pe) {                       \
    rocshmem_ctx_getmem(ctx, dest, source, nelems * sizeof(T), pe);                               \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_get_nbi(T *dest, const T *source, size_t nelems, int pe) { \
    rocshmem_getmem(dest, source, nelems * sizeof(T), pe);                                        \
  }                                                                                               \
  __host__ inline T rocshmem_ctx_##TN##_g(rocshmem_ctx_t ctx, const T *source, int pe) {          \
    T value;                                                                                      \
    rocshmem_ctx_getmem(ctx, &value, source, sizeof(T), pe);                                      \
    return value;                                                                                 \
  }                                                                                               \
  __host__ inline T rocshmem_##TN##_g(const T *source, int pe) {                                  \
    T value;                                                                                      \
    rocshmem_getmem(&value, source, sizeof(T), pe);                                               \
    return value;                                                                                 \
  }
ROCSHMEM_AMD_RMA_TYPES(ROCSHMEM_AMD_HOST_RMA)
#undef ROCSHMEM_AMD_HOST_RMA

// ---------------------------------------------------------------------------
// Atomics (include/rocshmem/rocshmem_AMO.hpp; src/host/host_templates.hpp:
// 254-330, where they are MPI_Fetch_and_op / MPI_Compare_and_swap).
// ---------------------------------------------------------------------------
#define ROCSHMEM_AMD_HOST_AMO_STANDARD(T, TN)                                                     \
  __host__ inline T rocshmem_ctx_##TN##_atomic_fetch_add(rocshmem_ctx_t ctx, T *dest, T value,    \
                                                         int pe) {                                \
    return detail::host_amo<T>(ROCSHMEM_AMD_AMO_FETCH_ADD, ctx, dest, value, pe,                  \
                               "atomic_fetch_add");                                               \
  }                                                                                               \
  __host__ inline T rocshmem_##TN##_atomic_fetch_add(T *dest, T value, int pe) {                  \
    return rocshmem_ctx_##TN##_atomic_fetch_add(ROCSHMEM_AMD_HOST_DEFAULT_CTX, dest, value, pe);  \
  }                                                                                               \
  __host__ inline void rocshmem_ctx_##TN##_atomic_add(rocshmem_ctx_t ctx, T *dest, T value,       \
                                                      int pe) {                                   \
    (void)detail::host_amo<T>(ROCSHMEM_AMD_AMO_ADD, ctx, dest, value, pe, "atomic_add");          \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_atomic_add(T *dest, T value, int pe) {                     \
    rocshmem_ctx_##TN##_atomic_add(ROCSHMEM_AMD_HOST_DEFAULT_CTX, dest, value, pe);               \
  }                                                                                               \
  __host__ inline T rocshmem_ctx_##TN##_atomic_fetch_inc(rocshmem_ctx_t ctx, T *dest, int pe) {   \
    return detail::host_amo<T>(ROCSHMEM_AMD_AMO_FETCH_INC, ctx, dest, pe,                         \
                               "atomic_fetch_inc");                                               \
  }                                                                                               \
  __host__ inline T rocshmem_##TN##_atomic_fetch_inc(T *dest, int pe) {                           \
    return rocshmem_ctx_##TN##_atomic_fetch_inc(ROCSHMEM_AMD_HOST_DEFAULT_CTX, dest, pe);         \
  }                                                                                               \
  __host__ inline void rocshmem_ctx_##TN##_atomic_inc(rocshmem_ctx_t ctx, T *dest, int pe) {      \
    (void)detail::host_amo<T>(ROCSHMEM_AMD_AMO_INC, ctx, dest, pe, "atomic_inc");                 \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_atomic_inc(T *dest, int pe) {                              \
    rocshmem_ctx_##TN##_atomic_inc(ROCSHMEM_AMD_HOST_DEFAULT_CTX, dest, pe);                      \
  }                                                                                               \
  __host__ inline T rocshmem_ctx_##TN##_atomic_compare_swap(rocshmem_ctx_t ctx, T *dest, T cond,  \
                                                            T value, int pe) {                    \
    return detail::host_amo<T>(ROCSHMEM_AMD_AMO_COMPARE_SWAP, ctx, dest, value, cond, pe,         \
                               "atomic_compare_swap");                                            \
  }                                                                                               \
  __host__ inline T rocshmem_##TN##_atomic_compare_swap(T *dest, T cond, T value, int pe) {       \
    return rocshmem_ctx_##TN##_atomic_compare_swap(ROCSHMEM_AMD_HOST_DEFAULT_CTX, dest, cond,     \
                                                   value, pe);                                    \
  }

#define ROCSHMEM_AMD_HOST_AMO_EXTENDED(T, TN)                                                     \
  __host__ inline T rocshmem_ctx_##TN##_atomic_fetch(rocshmem_ctx_t ctx, T *source, int pe) {     \
    return detail::host_amo<T>(ROCSHMEM_AMD_AMO_FETCH, ctx, source, pe, "atomic_fetch");          \
  }                                                                                               \
  __host__ inline T rocshmem_##TN##_atomic_fetch(T *source, int pe) {                             \
    return rocshmem_ctx_##TN##_atomic_fetch(ROCSHMEM_AMD_HOST_DEFAULT_CTX, source, pe);           \
  }                                                                                               \
  __host__ inline void rocshmem_ctx_##TN##_atomic_set(rocshmem_ctx_t ctx, T *dest, T value,       \
                                                      int pe) {                                   \
    (void)detail::host_amo<T>(ROCSHMEM_AMD_AMO_SET, ctx, dest, value, pe, "atomic_set");          \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_atomic_set(T *dest, T value, int pe) {                     \
    rocshmem_ctx_##TN##_atomic_set(ROCSHMEM_AMD_HOST_DEFAULT_CTX, dest, value, pe);               \
  }                                                                                               \
  __host__ inline T rocshmem_ctx_##TN##_atomic_swap(rocshmem_ctx_t ctx, T *dest, T value,         \
                                                    int pe) {                                     \
    return detail::host_amo<T>(ROCSHMEM_AMD_AMO_SWAP, ctx, dest, value, pe, "atomic_swap");       \
  }                                                                                               \
  __host__ inline T rocshmem_##TN##_atomic_swap(T *dest, T value, int pe) {                       \
    return rocshmem_ctx_##TN##_atomic_swap(ROCSHMEM_AMD_HOST_DEFAULT_CTX, dest, value, pe);       \
  }

#define ROCSHMEM_AMD_HOST_AMO_BITWISE1(T, TN, OP, CODE)                                           \
  __host__ inline T rocshmem_ctx_##TN##_atomic_fetch_##OP(rocshmem_ctx_t ctx, T *dest, T value,   \
                                                          int pe) {                               \
    return detail::host_amo<T>(CODE, ctx, dest, value, pe, "atomic_fetch_" #OP);                  \
  }                                                                                               \
  __host__ inline T rocshmem_##TN##_atomic_fetch_##OP(T *dest, T value, int pe) {                 \
    return rocshmem_ctx_##TN##_atomic_fetch_##OP(ROCSHMEM_AMD_HOST_DEFAULT_CTX, dest, value, pe); \
  }                                                                                               \
  __host__ inline void rocshmem_ctx_##TN##_atomic_##OP(rocshmem_ctx_t ctx, T *dest, T value,      \
                                                       int pe) {                                  \
    (void)rocshmem_ctx_##TN##_atomic_fetch_##OP(ctx, dest, value, pe);                            \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_atomic_##OP(T *dest, T value, int pe) {                    \
    (void)rocshmem_##TN##_atomic_fetch_##OP(dest, value, pe);                                     \
  }
#define ROCSHMEM_AMD_HOST_AMO_BITWISE(T, TN)                                                      \
  ROCSHMEM_AMD_HOST_AMO_BITWISE1(T, TN, and, ROCSHMEM_AMD_AMO_FETCH_AND)                          \
  ROCSHMEM_AMD_HOST_AMO_BITWISE1(T, TN, or, ROCSHMEM_AMD_AMO_FETCH_OR)                            \
  ROCSHMEM_AMD_HOST_AMO_BITWISE1(T, TN, xor, ROCSHMEM_AMD_AMO_FETCH_XOR)

ROCSHMEM_AMD_AMO_STANDARD_TYPES(ROCSHMEM_AMD_HOST_AMO_STANDARD)
ROCSHMEM_AMD_AMO_EXTENDED_TYPES(ROCSHMEM_AMD_HOST_AMO_EXTENDED)
ROCSHMEM_AMD_AMO_BITWISE_TYPES(ROCSHMEM_AMD_HOST_AMO_BITWISE)
#undef ROCSHMEM_AMD_HOST_AMO_STANDARD
#undef ROCSHMEM_AMD_HOST_AMO_EXTENDED
#undef ROCSHMEM_AMD_HOST_AMO_BITWISE
#undef ROCSHMEM_AMD_HOST_AMO_BITWISE1

// ---------------------------------------------------------------------------
// Point-to-point synchronisation (include/rocshmem/rocshmem_P2P_SYNC.hpp).
// The _vector forms take one comparison value, as declared there; the
// reference's host implementation of them is empty
// (src/host/host_templates.hpp:600-625) — here they behave as the plain forms.
// ---------------------------------------------------------------------------
#define ROCSHMEM_AMD_HOST_WAIT(T, TN)                                                             \
  __host__ inline void rocshmem_##TN##_wait_until(T *ivars, int cmp, T val) {                     \
    (void)detail::host_wait_until<T>(ivars, cmp, val);                                            \
  }                                                                                               \
  __host__ inline size_t rocshmem_##TN##_wait_until_any(T *ivars, size_t nelems,                  \
                                                        const int *status, int cmp, T val) {      \
    return detail::host_wait_until_any<T>(ivars, nelems, status, cmp, val);                       \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_wait_until_all(T *ivars, size_t nelems, const int *status, \
                                                      int cmp, T val) {                           \
    (void)detail::host_wait_until_all<T>(ivars, nelems, status, cmp, val);                        \
  }                                                                                               \
  __host__ inline size_t rocshmem_##TN##_wait_until_some(T *ivars, size_t nelems,                 \
                                                         size_t *indices, const int *status,      \
                                                         int cmp, T val) {                        \
    return detail::host_wait_until_some<T>(ivars, nelems, indices, status, cmp, val);             \
  }                                                                                               \
  __host__ inline size_t rocshmem_##TN##_wait_until_any_vector(T *ivars, size_t nelems,           \
                                                               const int *status, int cmp,        \
                                                               T val) {                           \
    return detail::host_wait_until_any<T>(ivars, nelems, status, cmp, val);                       \
  }                                                                                               \
  __host__ inline void rocshmem_##TN##_wait_until_all_vector(T *ivars, size_t nelems,             \
                                                             const int *status, int cmp, T val) { \
    (void)detail::host_wait_until_all<T>(ivars, nelems, status, cmp, val);                        \
  }                                                                                               \
  __host__ inline size_t rocshmem_##TN##_wait_until_some_vector(T *ivars, size_t nelems,          \
                                                                size_t *indices,                  \
                                                                const int *status, int cmp,       \
                                                                T val) {                          \
    return detail::host_wait_until_some<T>(ivars, nelems, indices, status, cmp, val);             \
  }                                                                                               \
  __host__ inline int rocshmem_##TN##_test(T *ivars, int cmp, T val) {                            \
    return detail::host_test<T>(ivars, cmp, val);                                                 \
  }
ROCSHMEM_AMD_WAIT_TYPES(ROCSHMEM_AMD_HOST_WAIT)
#undef ROCSHMEM_AMD_HOST_WAIT

// ---------------------------------------------------------------------------
// Collectives (include/rocshmem/rocshmem_COLL.hpp; the reference calls
// MPI_Bcast / MPI_Allreduce, src/host/host_templates.hpp:128-200,333-390).
// ---------------------------------------------------------------------------
#define ROCSHMEM_AMD_HOST_BROADCAST(T, TN)                                                        \
  __host__ inline void rocshmem_ctx_##TN##_broadcast(rocshmem_ctx_t, T *dest, const T *source,    \
                                                     int nelems, int pe_root, int pe_start,       \
                                                     int log_pe_stride, int pe_size, long *) {    \
    detail::host_collective(                                                                      \
        pe_start, 1 << log_pe_stride, pe_size,                                                    \
        [&] {                                                                                     \
          return nelems < 0 ? -1                                                                  \
                            : rocshmem_amd_broadcast_active_set(                                  \
                                  rocshmem_amd_pe_ptr(dest, pe_start),                            \
                                  rocshmem_amd_pe_ptr(source, pe_start),                          \
                                  static_cast<size_t>(nelems) * sizeof(T), pe_root, pe_start,     \
                                  log_pe_stride, pe_size, nullptr);                               \
        },                                                                                        \
        "broadcast");                                                                             \
  }                                                                                               \
  __host__ inline void rocshmem_ctx_##TN##_broadcast(rocshmem_ctx_t, rocshmem_team_t team,        \
                                                     T *dest, const T *source, int nelems,        \
                                                     int pe_root) {                               \
    detail::host_team_collective(                                                                 \
        team,                                                                                     \
        [&] {                                                                                     \
          return nelems < 0 ? -1                                                                  \
                            : rocshmem_amd_broadcastmem(team, dest, source,                       \
                                                        static_cast<size_t>(nelems) * sizeof(T),  \
                                                        pe_root, nullptr);                        \
        },                                                                                        \
        "broadcast");                                                                             \
  }
ROCSHMEM_AMD_COLL_TYPES(ROCSHMEM_AMD_HOST_BROADCAST)
#undef ROCSHMEM_AMD_HOST_BROADCAST

// The active-set form rocshmem_ctx_<T>_<op>_to_all is defined by the reference
// library (src/rocshmem.cpp:974-980) and used by its tests
// (tests/sos_tests/to_all.cpp) although its public headers do not declare it.
// The team form under the to_all name is what two more of its tests call
// (tests/sos_tests/shmem_team_reduce.cpp:128) though the library has no such
// overload; it is the same as _reduce.
#define ROCSHMEM_AMD_HOST_REDUCE1(T, TN, OPN, OPCODE)                                             \
  __host__ inline void rocshmem_ctx_##TN##_##OPN##_to_all(rocshmem_ctx_t, T *dest,                \
                                                          const T *source, int nreduce,           \
                                                          int PE_start, int logPE_stride,         \
                                                          int PE_size, T *, long *) {             \
    detail::host_collective(                                                                      \
        PE_start, 1 << logPE_stride, PE_size,                                                     \
        [&] {                                                                                     \
          return rocshmem_amd_to_all(detail::host_dtype<T>(), OPCODE,                             \
                                     rocshmem_amd_pe_ptr(dest, PE_start),                         \
                                     rocshmem_amd_pe_ptr(source, PE_start), nreduce, PE_start,    \
                                     logPE_stride, PE_size, nullptr);                             \
        },                                                                                        \
        #OPN "_to_all");                                                                          \
  }                                                                                               \
  __host__ inline int rocshmem_ctx_##TN##_##OPN##_reduce(rocshmem_ctx_t, rocshmem_team_t team,    \
                                                         T *dest, const T *source, int nreduce) { \
    detail::host_team_collective(                                                                 \
        team,                                                                                     \
        [&] {                                                                                     \
          return rocshmem_amd_reduce(detail::host_dtype<T>(), OPCODE, team, dest, source,         \
                                     nreduce, nullptr);                                           \
        },                                                                                        \
        #OPN "_reduce");                                                                          \
    return ROCSHMEM_SUCCESS;                                                                      \
  }                                                                                               \
  __host__ inline int rocshmem_ctx_##TN##_##OPN##_to_all(rocshmem_ctx_t ctx, rocshmem_team_t team, \
                                                         T *dest, const T *source, int nreduce) { \
    return rocshmem_ctx_##TN##_##OPN##_reduce(ctx, team, dest, source, nreduce);                  \
  }
#define ROCSHMEM_AMD_HOST_REDUCE_ARITH(T, TN)                   \
  ROCSHMEM_AMD_HOST_REDUCE1(T, TN, sum, ROCSHMEM_AMD_SUM)       \
  ROCSHMEM_AMD_HOST_REDUCE1(T, TN, min, ROCSHMEM_AMD_MIN)       \
  ROCSHMEM_AMD_HOST_REDUCE1(T, TN, max, ROCSHMEM_AMD_MAX)       \
  ROCSHMEM_AMD_HOST_REDUCE1(T, TN, prod, ROCSHMEM_AMD_PROD)
#define ROCSHMEM_AMD_HOST_REDUCE_BITWISE(T, TN)                 \
  ROCSHMEM_AMD_HOST_REDUCE1(T, TN, or, ROCSHMEM_AMD_OR)         \
  ROCSHMEM_AMD_HOST_REDUCE1(T, TN, and, ROCSHMEM_AMD_AND)       \
  ROCSHMEM_AMD_HOST_REDUCE1(T, TN, xor, ROCSHMEM_AMD_XOR)
ROCSHMEM_AMD_INT_REDUCE_TYPES(ROCSHMEM_AMD_HOST_REDUCE_ARITH)
ROCSHMEM_AMD_INT_REDUCE_TYPES(ROCSHMEM_AMD_HOST_REDUCE_BITWISE)
ROCSHMEM_AMD_FLOAT_REDUCE_TYPES(ROCSHMEM_AMD_HOST_REDUCE_ARITH)
#undef ROCSHMEM_AMD_HOST_REDUCE1
#undef ROCSHMEM_AMD_HOST_REDUCE_ARITH
#undef ROCSHMEM_AMD_HOST_REDUCE_BITWISE

}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_HOST_HPP_
