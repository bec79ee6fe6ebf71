// Type-name tables the typed API is stamped out from.  Each entry is
// X(C type, name fragment).  The tables restate the instantiation lists of the
// reference (src/rocshmem_gpu.cpp:1528-1673).
#ifndef ROCSHMEM_AMD_DETAIL_TYPE_LISTS_HPP_
#define ROCSHMEM_AMD_DETAIL_TYPE_LISTS_HPP_

// put/get/p/g, put_signal and their _nbi/_wg/_wave forms.
#define ROCSHMEM_AMD_RMA_TYPES(X)                                            \
  X(float, float) X(double, double) X(char, char) X(signed char, schar)      \
  X(short, short) X(int, int) X(long, long) X(long long, longlong)           \
  X(unsigned char, uchar) X(unsigned short, ushort) X(unsigned int, uint)    \
  X(unsigned long, ulong) X(unsigned long long, ulonglong)                   \
  X(int8_t, int8) X(int16_t, int16) X(int32_t, int32) X(int64_t, int64)      \
  X(uint8_t, uint8) X(uint16_t, uint16) X(uint32_t, uint32)                  \
  X(uint64_t, uint64) X(size_t, size) X(ptrdiff_t, ptrdiff)

// fetch_inc / inc / fetch_add / add / compare_swap.
#define ROCSHMEM_AMD_AMO_STANDARD_TYPES(X)                                   \
  X(int, int) X(long, long) X(long long, longlong) X(unsigned int, uint)     \
  X(unsigned long, ulong) X(unsigned long long, ulonglong)                   \
  X(int32_t, int32) X(int64_t, int64) X(uint32_t, uint32)                    \
  X(uint64_t, uint64) X(size_t, size) X(ptrdiff_t, ptrdiff)

// fetch / set / swap.
#define ROCSHMEM_AMD_AMO_EXTENDED_TYPES(X)                                   \
  X(float, float) X(double, double) ROCSHMEM_AMD_AMO_STANDARD_TYPES(X)

// fetch_and / and / fetch_or / or / fetch_xor / xor.
#define ROCSHMEM_AMD_AMO_BITWISE_TYPES(X)                                    \
  X(unsigned int, uint) X(unsigned long, ulong)                              \
  X(unsigned long long, ulonglong) X(int32_t, int32) X(int64_t, int64)       \
  X(uint32_t, uint32) X(uint64_t, uint64)

// wait_until / test families.
#define ROCSHMEM_AMD_WAIT_TYPES(X)                                           \
  X(float, float) X(double, double) X(char, char) X(signed char, schar)      \
  X(short, short) X(int, int) X(long, long) X(long long, longlong)           \
  X(unsigned char, uchar) X(unsigned short, ushort) X(unsigned int, uint)    \
  X(unsigned long, ulong) X(unsigned long long, ulonglong)

// Reductions: integer types take all seven ops, floating types four.
#define ROCSHMEM_AMD_INT_REDUCE_TYPES(X)                                     \
  X(short, short) X(int, int) X(long, long) X(long long, longlong)
#define ROCSHMEM_AMD_FLOAT_REDUCE_TYPES(X) X(float, float) X(double, double)

// alltoall / broadcast / fcollect (the RMA table minus the fixed-width and
// size/ptrdiff aliases, as in include/rocshmem/rocshmem_COLL.hpp).
#define ROCSHMEM_AMD_COLL_TYPES(X)                                           \
  X(float, float) X(double, double) X(char, char) X(signed char, schar)      \
  X(short, short) X(int, int) X(long, long) X(long long, longlong)           \
  X(unsigned char, uchar) X(unsigned short, ushort) X(unsigned int, uint)    \
  X(unsigned long, ulong) X(unsigned long long, ulonglong)

#endif  // ROCSHMEM_AMD_DETAIL_TYPE_LISTS_HPP_
