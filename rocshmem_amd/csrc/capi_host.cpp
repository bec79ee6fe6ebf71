// C entry points that wrap the host runtime: bring-up, symmetric allocation,
// teams, staging copies and timers.  No kernels are launched from this file.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#include "drv_common.hpp"
#include "proc_group.hpp"
#include "rocshmem_amd.h"

using rocshmem::runtime::rt;

extern "C" {

int rocshmem_amd_init(int npes, size_t heap_bytes_per_pe) {
  return rt().init(npes, heap_bytes_per_pe);
}
int rocshmem_amd_finalize(void) {
  rt().finalize();
  return 0;
}
int rocshmem_amd_n_pes(void) { return rocshmem::rocshmem_n_pes(); }
int rocshmem_amd_my_pe(void) { return rocshmem::rocshmem_my_pe(); }
int rocshmem_amd_set_pe(int pe) {
  if (!rt().live || pe < 0 || pe >= rt().npes) return -1;
  rt().set_pe(pe);
  return 0;
}
int rocshmem_amd_set_pe_rule(int rule) {
  if (!rt().live || rule < 0 || rule > 4) return -1;
  rt().set_pe_rule(rule);
  return 0;
}
size_t rocshmem_amd_procs_file_bytes(void) { return sizeof(rocshmem::runtime::ProcShared); }
int rocshmem_amd_procs_count(void) {
  return rocshmem::runtime::procs().attach_from_env() ? rocshmem::runtime::procs().nprocs() : 0;
}
int rocshmem_amd_procs_attach(const char *path, int nprocs, int rank) {
  return rocshmem::runtime::procs().attach(path, nprocs, rank);
}
int rocshmem_amd_procs_barrier(int PE_start, int PE_stride, int PE_size) {
  return rocshmem::runtime::procs().barrier(PE_start, PE_stride, PE_size);
}
int rocshmem_amd_procs_publish(const void *bytes, size_t n) {
  return rocshmem::runtime::procs().publish(bytes, n);
}
int rocshmem_amd_procs_fetch(int rank, void *bytes, size_t n) {
  return rocshmem::runtime::procs().fetch(rank, bytes, n);
}
int rocshmem_amd_procs_request_abort(int status) {
  if (!rocshmem::runtime::procs().active()) return -1;
  rocshmem::runtime::procs().request_abort(status);
  return 0;
}
int rocshmem_amd_procs_abort_requested(void) { return rocshmem::runtime::procs().abort_requested(); }
int rocshmem_amd_set_spin_limit(uint64_t polls) {
  if (!rt().live) return -1;
  rt().set_spin_limit(polls);
  return 0;
}
int64_t rocshmem_amd_waits_given_up(int clear) {
  if (!rt().live) return -1;
  return static_cast<int64_t>(rt().waits_given_up(clear != 0));
}
int rocshmem_amd_set_coalesce_puts(int on) {
  if (!rt().live) return -1;
  const int before = rt().state.coalesce_puts;
  rt().set_coalesce_puts(on);
  return before;
}
int64_t rocshmem_amd_set_ctx_options(int64_t options) {
  if (!rt().live) return -1;
  const int64_t before = rt().driver_ctx_options;
  rt().driver_ctx_options = options;
  return before;
}
int rocshmem_amd_coresident(long n_wgs, int wgs_per_cu, int n_cus) {
  return rocshmem::drv::coresident(n_wgs, wgs_per_cu, n_cus) ? 1 : 0;
}
int rocshmem_amd_hw_queues_suffice(size_t pe_streams, size_t hw_queues) {
  return rocshmem::runtime::hw_queues_suffice(pe_streams, hw_queues) ? 1 : 0;
}
int rocshmem_amd_dev_mem_info(size_t *free_bytes, size_t *total_bytes) {
  if (!free_bytes || !total_bytes) return -1;
  return hipMemGetInfo(free_bytes, total_bytes) == hipSuccess ? 0 : -1;
}
size_t rocshmem_amd_heap_alloc_bytes(void) { return rt().live ? rt().heap_alloc_bytes : 0; }
int rocshmem_amd_heap_is_uncached(void) { return rt().live ? (rt().heap_uncached ? 1 : 0) : -1; }
int rocshmem_amd_heap_held(size_t *total_bytes, size_t *idle_bytes) {
  if (!total_bytes || !idle_bytes) return -1;
  rocshmem::runtime::heap_held(total_bytes, idle_bytes);
  return 0;
}
int rocshmem_amd_pe_threads_enter(int PE_start, int PE_stride, int PE_size) {
  return rocshmem::runtime::pe_threads_enter(PE_start, PE_stride, PE_size, nullptr) ? 1 : 0;
}
void rocshmem_amd_pe_threads_leave(int PE_start, int PE_stride, int PE_size) {
  rocshmem::runtime::pe_threads_leave(PE_start, PE_stride, PE_size, 0);
}
int rocshmem_amd_team_active_set(rocshmem_amd_team_t team, int *PE_start, int *PE_stride,
                                 int *PE_size) {
  if (!rt().live || !PE_start || !PE_stride || !PE_size) return -1;
  const rocshmem::detail::Team *t =
      rt().host_team(rt().my_view(static_cast<rocshmem::rocshmem_team_t>(team)));
  if (!t) return -1;
  *PE_start = t->wrt_world.pe_start;
  *PE_stride = t->wrt_world.stride;
  *PE_size = t->wrt_world.size;
  return 0;
}
// (with one process per PE these are the collective calls: every PE makes
// them and they meet, as rocshmem_malloc / rocshmem_free do)
void *rocshmem_amd_malloc(size_t size) {
  if (rt().nprocs) return rocshmem::rocshmem_malloc(size);
  return rt().sym_malloc(size);
}
int rocshmem_amd_free(void *ptr) {
  if (rt().nprocs) {
    rocshmem::rocshmem_free(ptr);
    return 0;
  }
  rt().sym_free(ptr);
  return 0;
}
int rocshmem_amd_barrier_all(void) {
  if (!rt().live) return -1;
  rocshmem::rocshmem_barrier_all();
  return 0;
}
void *rocshmem_amd_pe_ptr(const void *ptr, int pe) {
  return rt().live ? rt().pe_ptr(ptr, pe) : nullptr;
}
size_t rocshmem_amd_heap_size(void) { return rt().allocator.size(); }
size_t rocshmem_amd_heap_used(void) { return rt().allocator.used(); }
size_t rocshmem_amd_heap_avail(void) { return rt().allocator.avail(); }
size_t rocshmem_amd_pe_stride(void) { return rt().pe_stride; }

void *rocshmem_amd_heap_model_create(uint64_t base_address, uint64_t heap_bytes) {
  return new rocshmem::runtime::Pow2Allocator(base_address, heap_bytes);
}
void rocshmem_amd_heap_model_destroy(void *model) {
  delete static_cast<rocshmem::runtime::Pow2Allocator *>(model);
}
uint64_t rocshmem_amd_heap_model_alloc(void *model, uint64_t size) {
  return static_cast<rocshmem::runtime::Pow2Allocator *>(model)->alloc(size);
}
int rocshmem_amd_heap_model_free(void *model, uint64_t offset) {
  return static_cast<rocshmem::runtime::Pow2Allocator *>(model)->free(offset) ? 0 : -1;
}
uint64_t rocshmem_amd_heap_model_used(void *model) {
  return static_cast<rocshmem::runtime::Pow2Allocator *>(model)->used();
}
uint64_t rocshmem_amd_heap_model_num_bins(void *model) {
  return static_cast<rocshmem::runtime::Pow2Allocator *>(model)->num_bins();
}
uint64_t rocshmem_amd_heap_model_bin_population(void *model, uint64_t block_bytes) {
  return static_cast<rocshmem::runtime::Pow2Allocator *>(model)->bin_population(block_bytes);
}

rocshmem_amd_team_t rocshmem_amd_team_world(void) { return rocshmem::ROCSHMEM_TEAM_WORLD; }
int rocshmem_amd_team_split_strided(rocshmem_amd_team_t parent, int start, int stride,
                                    int size, rocshmem_amd_team_t *new_team) {
  rocshmem::rocshmem_team_t t = rocshmem::ROCSHMEM_TEAM_INVALID;
  const int rc = rocshmem::rocshmem_team_split_strided(
      static_cast<rocshmem::rocshmem_team_t>(parent), start, stride, size, nullptr, 0, &t);
  *new_team = t;
  return rc;
}
void rocshmem_amd_team_destroy(rocshmem_amd_team_t team) {
  rocshmem::rocshmem_team_destroy(static_cast<rocshmem::rocshmem_team_t>(team));
}
int rocshmem_amd_team_n_pes(rocshmem_amd_team_t team) {
  return rocshmem::rocshmem_team_n_pes(static_cast<rocshmem::rocshmem_team_t>(team));
}
int rocshmem_amd_team_my_pe(rocshmem_amd_team_t team) {
  return rocshmem::rocshmem_team_my_pe(static_cast<rocshmem::rocshmem_team_t>(team));
}
int rocshmem_amd_team_translate_pe(rocshmem_amd_team_t src_team, int src_pe,
                                   rocshmem_amd_team_t dest_team) {
  return rocshmem::rocshmem_team_translate_pe(
      static_cast<rocshmem::rocshmem_team_t>(src_team), src_pe,
      static_cast<rocshmem::rocshmem_team_t>(dest_team));
}
rocshmem_amd_team_t rocshmem_amd_team_on(rocshmem_amd_team_t team, int pe) {
  return rocshmem::rocshmem_emu_team_on(static_cast<rocshmem::rocshmem_team_t>(team), pe);
}

void *rocshmem_amd_dev_alloc(size_t size) {
  void *p = nullptr;
  if (size == 0) return nullptr;
  DRV_CHECK_HIP(hipMalloc(&p, size));
  return p;
}
int rocshmem_amd_dev_free(void *ptr) {
  if (ptr) DRV_CHECK_HIP(hipFree(ptr));
  return 0;
}
int rocshmem_amd_copy_in(void *dst_dev, const void *src_host, size_t n) {
  if (n && (!dst_dev || !src_host)) return -1;
  if (n) DRV_CHECK_HIP(hipMemcpy(dst_dev, src_host, n, hipMemcpyHostToDevice));
  return 0;
}
int rocshmem_amd_copy_out(void *dst_host, const void *src_dev, size_t n) {
  if (n && (!dst_host || !src_dev)) return -1;
  if (n) DRV_CHECK_HIP(hipMemcpy(dst_host, src_dev, n, hipMemcpyDeviceToHost));
  return 0;
}
int rocshmem_amd_fill(void *dst_dev, int byte, size_t n) {
  if (n && !dst_dev) return -1;
  if (n) DRV_CHECK_HIP(hipMemset(dst_dev, byte, n));
  return 0;
}
int rocshmem_amd_copy_dev(void *dst_dev, const void *src_dev, size_t n) {
  if (n && (!dst_dev || !src_dev)) return -1;
  if (n) DRV_CHECK_HIP(hipMemcpy(dst_dev, src_dev, n, hipMemcpyDeviceToDevice));
  return 0;
}
int rocshmem_amd_stream_sync(rocshmem_amd_stream_t stream) {
  DRV_CHECK_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return 0;
}

struct DrvTimer {
  hipEvent_t start, stop;
};
void *rocshmem_amd_timer_create(void) {
  DrvTimer *t = new DrvTimer;
  DRV_CHECK_HIP(hipEventCreate(&t->start));
  DRV_CHECK_HIP(hipEventCreate(&t->stop));
  return t;
}
int rocshmem_amd_timer_start(void *timer, rocshmem_amd_stream_t stream) {
  DRV_CHECK_HIP(hipEventRecord(static_cast<DrvTimer *>(timer)->start,
                               static_cast<hipStream_t>(stream)));
  return 0;
}
int rocshmem_amd_timer_stop(void *timer, rocshmem_amd_stream_t stream) {
  DRV_CHECK_HIP(hipEventRecord(static_cast<DrvTimer *>(timer)->stop,
                               static_cast<hipStream_t>(stream)));
  return 0;
}
float rocshmem_amd_timer_elapsed_ms(void *timer) {
  DrvTimer *t = static_cast<DrvTimer *>(timer);
  DRV_CHECK_HIP(hipEventSynchronize(t->stop));
  float ms = 0.f;
  DRV_CHECK_HIP(hipEventElapsedTime(&ms, t->start, t->stop));
  return ms;
}
int rocshmem_amd_timer_destroy(void *timer) {
  DrvTimer *t = static_cast<DrvTimer *>(timer);
  DRV_CHECK_HIP(hipEventDestroy(t->start));
  DRV_CHECK_HIP(hipEventDestroy(t->stop));
  delete t;
  return 0;
}

}  // extern "C"
