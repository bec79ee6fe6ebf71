// Host-side RMA, atomics and waits on the emulated heap: what the reference
// forwards to MPI one-sided calls (src/host/host.cpp:162-249) is done here
// with copies, one-thread kernels and polling reads.
#include <mutex>

#include "drv_common.hpp"
#include "rocshmem_amd.h"

namespace rocshmem {
namespace drv {

void launch_bulk(char *dst, const char *src, size_t nbytes, hipStream_t stream);

namespace {

// Is `p` memory a kernel can dereference?  Plain host allocations are not;
// pinned host memory and device memory are.
bool device_accessible(const void *p) {
  auto &r = runtime::rt();
  const char *c = static_cast<const char *>(p);
  (void)c;
  if (r.live && r.pe_of(p) >= 0) return true;
  hipPointerAttribute_t attr;
  const hipError_t e = hipPointerGetAttributes(&attr, p);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // unregistered host memory: not an error for the caller
    return false;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeHost ||
         attr.type == hipMemoryTypeManaged;
}

// Pinned block the one-thread atomic kernel reads its operands from and writes
// its result to, the staging buffer of the polling reads, and the streams of
// the host-side operations.  Both streams are non-blocking: the null stream
// would line every host put, atomic or poll up behind whatever kernel is
// running on an ordinary stream — and that kernel may be waiting for exactly
// this operation.
struct HostSide {
  std::mutex lock;
  uint64_t *args = nullptr;  // [0] pe, [1] value, [2] cond, [3] fetched
  char *staging = nullptr;
  size_t staging_bytes = 0;
  hipStream_t poll = nullptr;  // test / wait_until reads
  hipStream_t work = nullptr;  // put / get / atomics

  void ensure() {
    std::lock_guard<std::mutex> guard(init_lock);
    if (!args) {
      DRV_CHECK_HIP(hipStreamCreateWithFlags(&poll, hipStreamNonBlocking));
      DRV_CHECK_HIP(hipStreamCreateWithFlags(&work, hipStreamNonBlocking));
      DRV_CHECK_HIP(hipHostMalloc(reinterpret_cast<void **>(&args), 64, hipHostMallocDefault));
    }
  }
  std::mutex init_lock;
  char *stage(size_t bytes) {
    if (bytes > staging_bytes) {
      if (staging) DRV_CHECK_HIP(hipHostFree(staging));
      staging_bytes = bytes < 4096 ? 4096 : bytes;
      DRV_CHECK_HIP(hipHostMalloc(reinterpret_cast<void **>(&staging), staging_bytes,
                                  hipHostMallocDefault));
    }
    return staging;
  }
};
HostSide g_host;

size_t dtype_bytes(int dtype) {
  switch (dtype) {
    case ROCSHMEM_AMD_CHAR: case ROCSHMEM_AMD_SCHAR: case ROCSHMEM_AMD_UCHAR: return 1;
    case ROCSHMEM_AMD_SHORT: case ROCSHMEM_AMD_USHORT: case ROCSHMEM_AMD_BF16: return 2;
    case ROCSHMEM_AMD_INT: case ROCSHMEM_AMD_UINT: case ROCSHMEM_AMD_FLOAT: return 4;
    case ROCSHMEM_AMD_LONG: case ROCSHMEM_AMD_LONGLONG: case ROCSHMEM_AMD_ULONG:
    case ROCSHMEM_AMD_ULONGLONG: case ROCSHMEM_AMD_DOUBLE: return 8;
    default: return 0;
  }
}

template <typename Fn>
bool for_host_wait_dtype(int dtype, Fn &&fn) {
  switch (dtype) {
    case ROCSHMEM_AMD_FLOAT: fn(static_cast<float *>(nullptr)); return true;
    case ROCSHMEM_AMD_DOUBLE: fn(static_cast<double *>(nullptr)); return true;
    case ROCSHMEM_AMD_CHAR: fn(static_cast<char *>(nullptr)); return true;
    case ROCSHMEM_AMD_SCHAR: fn(static_cast<signed char *>(nullptr)); return true;
    case ROCSHMEM_AMD_UCHAR: fn(static_cast<unsigned char *>(nullptr)); return true;
    case ROCSHMEM_AMD_SHORT: fn(static_cast<short *>(nullptr)); return true;
    case ROCSHMEM_AMD_USHORT: fn(static_cast<unsigned short *>(nullptr)); return true;
    case ROCSHMEM_AMD_INT: fn(static_cast<int *>(nullptr)); return true;
    case ROCSHMEM_AMD_UINT: fn(static_cast<unsigned int *>(nullptr)); return true;
    case ROCSHMEM_AMD_LONG: fn(static_cast<long *>(nullptr)); return true;
    case ROCSHMEM_AMD_ULONG: fn(static_cast<unsigned long *>(nullptr)); return true;
    case ROCSHMEM_AMD_LONGLONG: fn(static_cast<long long *>(nullptr)); return true;
    case ROCSHMEM_AMD_ULONGLONG: fn(static_cast<unsigned long long *>(nullptr)); return true;
    default: return false;
  }
}

}  // namespace
}  // namespace drv
}  // namespace rocshmem

using namespace rocshmem;
using namespace rocshmem::drv;

extern "C" {

int rocshmem_amd_ctx_pe(const void *ctx_opaque) {
  auto &r = runtime::rt();
  if (!r.live) return -1;
  if (!ctx_opaque) return r.me();
  const auto *c = static_cast<const detail::Context *>(ctx_opaque);
  if (c >= r.d_default_ctx && c < r.d_default_ctx + 2 * r.npes)
    return static_cast<int>((c - r.d_default_ctx) % r.npes);
  if (c >= r.d_ctx_slots && c < r.d_ctx_slots + static_cast<size_t>(r.npes) * 2 * r.max_ctxs)
    return static_cast<int>((c - r.d_ctx_slots) / (2 * r.max_ctxs));
  return -1;
}

int rocshmem_amd_host_putmem(void *dest, const void *source, size_t nbytes, int my_pe, int pe) {
  if (!valid_actor(my_pe) || !valid_pe(pe)) return -1;
  if (!nbytes) return 0;
  if (!source || !sym_ok_on(dest, nbytes, my_pe)) return -1;
  auto &r = runtime::rt();
  char *target = static_cast<char *>(r.pe_ptr(dest, pe));
  g_host.ensure();
  if (device_accessible(source)) {
    if (!local_ok(source, nbytes)) return -1;
    launch_bulk(target, static_cast<const char *>(source), nbytes, g_host.work);
  } else {
    DRV_CHECK_HIP(hipMemcpyAsync(target, source, nbytes, hipMemcpyHostToDevice, g_host.work));
  }
  DRV_CHECK_HIP(hipStreamSynchronize(g_host.work));
  return 0;
}

int rocshmem_amd_host_getmem(void *dest, const void *source, size_t nbytes, int my_pe, int pe) {
  if (!valid_actor(my_pe) || !valid_pe(pe)) return -1;
  if (!nbytes) return 0;
  if (!dest || !sym_ok_on(source, nbytes, my_pe)) return -1;
  auto &r = runtime::rt();
  const char *origin = static_cast<const char *>(r.pe_ptr(source, pe));
  g_host.ensure();
  if (device_accessible(dest)) {
    if (!local_ok(dest, nbytes)) return -1;
    launch_bulk(static_cast<char *>(dest), origin, nbytes, g_host.work);
  } else {
    DRV_CHECK_HIP(hipMemcpyAsync(dest, origin, nbytes, hipMemcpyDeviceToHost, g_host.work));
  }
  DRV_CHECK_HIP(hipStreamSynchronize(g_host.work));
  return 0;
}

int rocshmem_amd_host_amo(int amo_op, int dtype, void *dest, const void *value, const void *cond,
                          int my_pe, int pe, void *fetched) {
  if (!valid_actor(my_pe) || !valid_pe(pe) || !value) return -1;
  const size_t es = dtype_bytes(dtype);
  if (es != 4 && es != 8) return -1;
  if (amo_op == ROCSHMEM_AMD_AMO_COMPARE_SWAP && !cond) return -1;
  g_host.ensure();
  std::lock_guard<std::mutex> guard(g_host.lock);
  uint64_t *a = g_host.args;
  // One operation of the batched driver: a single "counter" per PE, so the
  // global id of the target is the PE number.
  *reinterpret_cast<uint32_t *>(&a[0]) = static_cast<uint32_t>(pe);
  a[1] = a[2] = a[3] = 0;
  memcpy(&a[1], value, es);
  if (cond) memcpy(&a[2], cond, es);
  const int rc = rocshmem_amd_amo(amo_op, dtype, dest, 1, reinterpret_cast<const uint32_t *>(&a[0]),
                                  &a[1], &a[2], &a[3], 1, my_pe, 1, 1, g_host.work);
  if (rc != 0) return rc;
  DRV_CHECK_HIP(hipStreamSynchronize(g_host.work));
  if (fetched) memcpy(fetched, &a[3], es);
  return 0;
}

int rocshmem_amd_host_peek(void *dst_host, const void *src_dev, size_t nbytes) {
  if (!runtime::rt().live || !dst_host || !src_dev) return -1;
  if (!nbytes) return 0;
  if (!local_ok(src_dev, nbytes)) return -1;
  g_host.ensure();
  std::lock_guard<std::mutex> guard(g_host.lock);
  char *stage = g_host.stage(nbytes);
  DRV_CHECK_HIP(hipMemcpyAsync(stage, src_dev, nbytes, hipMemcpyDeviceToHost, g_host.poll));
  DRV_CHECK_HIP(hipStreamSynchronize(g_host.poll));
  memcpy(dst_host, stage, nbytes);
  return 0;
}

int rocshmem_amd_host_wait_test(int wait_fn, int dtype, const void *ivars, size_t nelems,
                                const int *status, int cmp, const void *value, long timeout_ms,
                                size_t *ret_out, size_t *indices_out) {
  if (!runtime::rt().live || !ivars || !value) return -1;
  if (wait_fn < ROCSHMEM_AMD_TEST || wait_fn > ROCSHMEM_AMD_WAIT_UNTIL_SOME) return -1;
  if (wait_fn == ROCSHMEM_AMD_WAIT_UNTIL_SOME && nelems && !indices_out) return -1;
  {
    const size_t es = dtype_bytes(dtype);
    const size_t span = (wait_fn <= ROCSHMEM_AMD_WAIT_UNTIL ? 1 : nelems) * es;
    if (!es || !local_ok(ivars, span)) return -1;
  }
  int rc = 0;
  size_t ret = 0;
  const bool known = for_host_wait_dtype(dtype, [&](auto *tag) {
    using T = typename std::remove_pointer<decltype(tag)>::type;
    const T *iv = static_cast<const T *>(ivars);
    const T val = *static_cast<const T *>(value);
    bool timed_out = false;
    switch (wait_fn) {
      case ROCSHMEM_AMD_TEST:
        ret = static_cast<size_t>(detail::host_test<T>(iv, cmp, val));
        break;
      case ROCSHMEM_AMD_WAIT_UNTIL:
        timed_out = !detail::host_wait_until<T>(iv, cmp, val, timeout_ms);
        break;
      case ROCSHMEM_AMD_WAIT_UNTIL_ANY:
        ret = detail::host_wait_until_any<T>(iv, nelems, status, cmp, val, timeout_ms, &timed_out);
        break;
      case ROCSHMEM_AMD_WAIT_UNTIL_ALL:
        timed_out = !detail::host_wait_until_all<T>(iv, nelems, status, cmp, val, timeout_ms);
        break;
      default:
        ret = detail::host_wait_until_some<T>(iv, nelems, indices_out, status, cmp, val, timeout_ms,
                                              &timed_out);
        break;
    }
    rc = timed_out ? 1 : 0;
  });
  if (!known) return -1;
  if (ret_out) *ret_out = ret;
  return rc;
}

}  // extern "C"
