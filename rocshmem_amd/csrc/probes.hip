// Measuring probes for the benchmark: what the memory system sustains in one
// direction, what an agent-scope release costs in the middle of a copy, and
// what a kernel that re-reads symmetric data gets from the caches.  Built into
// a library of their own (librocshmem_amd_probes.so): they are yardsticks the
// data path is read against, not part of it.
#include <mutex>

#include "drv_common.hpp"
#include "rocshmem_amd_probes.h"

namespace rocshmem {
namespace drv {

// What the memory system sustains in one direction only, with the copy
// kernel's instructions (one 16-byte vector per lane, non-temporal load,
// write-through streaming store): the yardstick the copy is read against.
// 128 lanes per work-group is where both directions peak (6.9 TB/s each); at
// 64 lanes a one-direction kernel is bound by work-group dispatch (4.7 TB/s).
constexpr int kProbeThreads = 128;
__global__ void probe_read_kernel(const char *src, size_t nvec, unsigned *sink) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= nvec) return;
  const detail::u32x4 a = detail::load16<true>(src + (i << 4));
  const unsigned x = a.x ^ a.y ^ a.z ^ a.w;
  if (x == 0x9e3779b9u && a.y == 0x7f4a7c15u) *sink = x;  // keeps the load alive; practically never taken
}
__global__ void probe_write_kernel(char *dst, size_t nvec) {
  const size_t first = static_cast<size_t>(blockIdx.x) * blockDim.x;
  const size_t i = first + threadIdx.x;
  const size_t left = nvec - first;
  const __amdgpu_buffer_rsrc_t w =
      detail::window_of(dst + (first << 4), (left < blockDim.x ? left : blockDim.x) << 4);
  const detail::u32x4 v = {1u, 2u, 3u, static_cast<unsigned>(i)};
  if (i < nvec) detail::store16<true>(w, static_cast<uint32_t>(threadIdx.x << 4), v);
}

// What an agent-scope release (the L2 write-back behind quiet and fence on a
// default context) costs in the middle of a copy: work-groups loop over tiles
// with the cooperative copy and release never (mode 0), once at their end
// (mode 1) or after every tile (mode 2).  The difference to mode 0, divided by
// the number of releases, is the cost of one.
template <int kMode>
__global__ void release_probe_kernel(char *dst, const char *src, size_t n, size_t tile) {
  const size_t ntiles = (n + tile - 1) / tile;
  for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const size_t off = t * tile;
    const size_t len = n - off < tile ? n - off : tile;
    detail::copy_lanes(dst + off, src + off, len, threadIdx.x, blockDim.x, 0);
    if constexpr (kMode == 2) {
      __syncthreads();
      if (threadIdx.x == 0) detail::fence_release();
    }
  }
  if constexpr (kMode == 1) {
    __syncthreads();
    if (threadIdx.x == 0) detail::fence_release();
  }
}

// A consumer that re-reads what it received: every work-group reads its tile
// of the buffer `passes` times in a row (an expert GEMM re-reads its rows
// once per output tile).  On cached memory the second and later passes hit
// the L2; on an uncached heap every pass goes back to memory.
__global__ void reuse_probe_kernel(const char *src, size_t nbytes, size_t tile, int passes,
                                   unsigned *sink) {
  const size_t ntiles = (nbytes + tile - 1) / tile;
  unsigned acc = 0;
  for (size_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const size_t off = t * tile;
    const size_t nvec = (nbytes - off < tile ? nbytes - off : tile) >> 4;
    for (int p = 0; p < passes; ++p) {
      for (size_t v = threadIdx.x; v < nvec; v += blockDim.x) {
        const detail::u32x4 a = detail::load16<false>(src + off + (v << 4));
        acc += a.x ^ a.y ^ a.z ^ a.w;
      }
      // keep the passes apart: a pass starts when the one before has been read
      __syncthreads();
    }
  }
  if (acc == 0x9e3779b9u) *sink = acc;  // keeps the loads alive; practically never taken
}

}  // namespace drv
}  // namespace rocshmem

using namespace rocshmem;
using namespace rocshmem::drv;

namespace {
unsigned *probe_sink() {
  static unsigned *sink = nullptr;  // never written in practice; allocated once
  static std::once_flag once;
  std::call_once(once, [] { DRV_CHECK_HIP(hipMalloc(&sink, sizeof(unsigned))); });
  return sink;
}
}  // namespace

extern "C" {

int rocshmem_amd_hbm_probe(int write, void *buf, size_t nbytes, rocshmem_amd_stream_t stream) {
  if (!runtime::rt().live || !buf || nbytes < (1u << 20) || (reinterpret_cast<uintptr_t>(buf) & 15u))
    return -1;
  if (!local_ok(buf, nbytes)) return -1;
  unsigned *sink = probe_sink();
  const size_t nvec = nbytes / 16;
  const unsigned grid = static_cast<unsigned>((nvec + kProbeThreads - 1) / kProbeThreads);
  if (write)
    hipLaunchKernelGGL(probe_write_kernel, dim3(grid), dim3(kProbeThreads), 0, as_stream(stream),
                       static_cast<char *>(buf), nvec);
  else
    hipLaunchKernelGGL(probe_read_kernel, dim3(grid), dim3(kProbeThreads), 0, as_stream(stream),
                       static_cast<const char *>(buf), nvec, sink);
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

int rocshmem_amd_release_probe(int mode, void *dst, const void *src, size_t nbytes,
                               size_t tile_bytes, int n_wgs, int wg_size,
                               rocshmem_amd_stream_t stream) {
  if (!runtime::rt().live || !dst || !src || !nbytes || tile_bytes < 16 || mode < 0 || mode > 2 ||
      !valid_launch(n_wgs, wg_size))
    return -1;
  if (!local_ok(dst, nbytes) || !local_ok(src, nbytes)) return -1;
  const dim3 g(n_wgs), b(wg_size);
  hipStream_t s = as_stream(stream);
  char *d = static_cast<char *>(dst);
  const char *c = static_cast<const char *>(src);
  if (mode == 0) hipLaunchKernelGGL(release_probe_kernel<0>, g, b, 0, s, d, c, nbytes, tile_bytes);
  else if (mode == 1) hipLaunchKernelGGL(release_probe_kernel<1>, g, b, 0, s, d, c, nbytes, tile_bytes);
  else hipLaunchKernelGGL(release_probe_kernel<2>, g, b, 0, s, d, c, nbytes, tile_bytes);
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

int rocshmem_amd_reuse_probe(const void *buf, size_t nbytes, size_t tile_bytes, int passes,
                             int n_wgs, int wg_size, rocshmem_amd_stream_t stream) {
  if (!runtime::rt().live || !buf || nbytes < 16 || tile_bytes < 16 || (tile_bytes & 15u) ||
      passes < 1 || (reinterpret_cast<uintptr_t>(buf) & 15u) || !valid_launch(n_wgs, wg_size))
    return -1;
  if (!local_ok(buf, nbytes)) return -1;
  hipLaunchKernelGGL(reuse_probe_kernel, dim3(n_wgs), dim3(wg_size), 0, as_stream(stream),
                     static_cast<const char *>(buf), nbytes, tile_bytes, passes, probe_sink());
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // extern "C"
