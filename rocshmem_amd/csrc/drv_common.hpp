// Shared by the driver translation units: error check, context handles for a
// given PE, and the tiling rule the RMA and signal drivers use.
#ifndef ROCSHMEM_AMD_DRV_COMMON_HPP_
#define ROCSHMEM_AMD_DRV_COMMON_HPP_

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#include "rocshmem/rocshmem.hpp"
#include "runtime.hpp"

#define DRV_CHECK_HIP(expr)                                                       \
  do {                                                                            \
    hipError_t drv_err_ = (expr);                                                 \
    if (drv_err_ != hipSuccess) {                                                 \
      fprintf(stderr, "rocshmem: HIP error %d (%s) at %s:%d\n", (int)drv_err_,    \
              hipGetErrorString(drv_err_), __FILE__, __LINE__);                   \
      exit(EXIT_FAILURE);                                                         \
    }                                                                             \
  } while (0)

namespace rocshmem {
namespace drv {

inline bool valid_launch(int n_wgs, int wg_size) {
  return n_wgs >= 1 && wg_size >= 1 && wg_size <= 1024;
}
inline bool valid_pe(int pe) {
  return runtime::rt().live && pe >= 0 && pe < runtime::rt().npes;
}
// The PE a driver is asked to act for: with one process per PE, only this
// process's own.
inline bool valid_actor(int pe) {
  return valid_pe(pe) && (!runtime::rt().nprocs || pe == runtime::rt().acting_pe);
}
// Drivers that host several PEs in one launch belong to the one-process
// harness; a process that is one PE of a job refuses them.
#define DRV_ONE_PROCESS_ONLY()                 \
  do {                                         \
    if (::rocshmem::runtime::rt().nprocs) return -1; \
  } while (0)
inline hipStream_t as_stream(void *s) { return static_cast<hipStream_t>(s); }

// [p, p+bytes) lies inside the usable part of one PE's slice.
inline bool sym_ok(const void *p, size_t bytes) {
  auto &r = runtime::rt();
  if (!r.live || !p) return false;
  const uint64_t off = r.offset_of(p);
  return off != runtime::Pow2Allocator::kNoBlock && off <= r.heap_size &&
         bytes <= r.heap_size - off;
}
// As sym_ok, and the address belongs to PE `pe`.
inline bool sym_ok_on(const void *p, size_t bytes, int pe) {
  return sym_ok(p, bytes) && runtime::rt().pe_of(p) == pe;
}
// A caller-local buffer: any non-null device address outside the heap is taken
// on trust; one inside the heap must stay inside its slice.
inline bool local_ok(const void *p, size_t bytes) {
  auto &r = runtime::rt();
  if (!p) return bytes == 0;
  const char *c = static_cast<const char *>(p);
  (void)c;
  if (r.live && r.pe_of(p) >= 0) return sym_ok(p, bytes);
  return true;
}

// ---- co-residency of grids whose work-groups wait for each other --------------
// A barrier, a ping-pong or a reduce between work-groups only ends if all of
// them are on the GPU at the same time: a work-group that has not been
// scheduled cannot answer, and the ones that wait for it never leave.  The
// drivers of such kernels therefore refuse (return -1, nothing launched) a
// grid larger than what the device holds resident for that kernel and
// work-group size.  The bound is for a GPU that runs nothing else.
inline bool coresident(long n_wgs, int wgs_per_cu, int n_cus) {
  return n_wgs >= 0 && wgs_per_cu > 0 && n_cus > 0 &&
         n_wgs <= static_cast<long>(wgs_per_cu) * static_cast<long>(n_cus);
}
inline int device_cu_count() {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return cus;
}
template <typename Kernel>
inline bool grid_fits(Kernel kernel, long n_wgs, int wg_size, size_t dynamic_lds = 0) {
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, wg_size, dynamic_lds) !=
      hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  const bool ok = coresident(n_wgs, per_cu, device_cu_count());
  if (!ok)
    fprintf(stderr,
            "rocshmem: refused a launch of %ld work-groups of %d threads that wait for each "
            "other: the GPU holds %d per CU on %d CUs at once\n",
            n_wgs, wg_size, per_cu, device_cu_count());
  return ok;
}

// Bytes per tile when the caller leaves the choice to the driver: an equal
// share per group, rounded up to 16 bytes.
inline size_t auto_tile(size_t nbytes, size_t groups) {
  size_t t = (nbytes + groups - 1) / groups;
  t = (t + 15) / 16 * 16;
  return t ? t : 16;
}

}  // namespace drv
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_DRV_COMMON_HPP_
