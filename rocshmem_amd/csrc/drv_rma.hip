// Drivers for the copy path: device-API put/get at thread, wavefront and
// work-group granularity, the host-initiated whole-GPU copy, and the
// wavefront coalescing utility.
#include <mutex>

#include "drv_common.hpp"
#include "rocshmem/detail/coalesce.hpp"
#include "rocshmem_amd.h"

namespace rocshmem {
namespace drv {

struct RmaArgs {
  char *dest;
  const char *source;
  size_t nbytes;
  size_t tile;
  rocshmem_ctx_t ctx;
  int pe;
  int iters;
  uint32_t scatter_mask;  // 0: tile i sits at i * tile; else at ((i * odd) & mask) * tile
};

// Where message i of a scattered run lives: an odd multiplier is a bijection
// on [0, 2^k), and neighbouring lanes land far apart.
__device__ __forceinline__ size_t tile_slot(size_t i, uint32_t scatter_mask) {
  return scatter_mask ? ((i * 0x9E3779B1ull) & scatter_mask) : i;
}

// One API call per tile; group g takes tiles g, g+G, ...
template <int kOp, int kGran, bool kScattered>
__global__ void rma_kernel(RmaArgs a) {
  size_t group, groups;
  const size_t tid = threadIdx.x, bs = blockDim.x;
  if constexpr (kGran == ROCSHMEM_AMD_WG) {
    group = blockIdx.x;
    groups = gridDim.x;
  } else if constexpr (kGran == ROCSHMEM_AMD_WAVE) {
    const size_t waves_per_wg = (bs + 63) / 64;
    group = blockIdx.x * waves_per_wg + tid / 64;
    groups = gridDim.x * waves_per_wg;
  } else {
    group = blockIdx.x * bs + tid;
    groups = gridDim.x * bs;
  }
  // No division and no multiplication on the way to a group's first load: the
  // walk is by offsets, and the scattered walk keeps the tile index beside it.
  const size_t stride = groups * a.tile;
  for (int it = 0; it < a.iters; ++it) {
    size_t i = group;
    for (size_t walk = group * a.tile; walk < a.nbytes; walk += stride) {
      size_t off = walk;
      if constexpr (kScattered) {
        off = tile_slot(i, a.scatter_mask) * a.tile;
        i += groups;
      }
      const size_t len = a.nbytes - off < a.tile ? a.nbytes - off : a.tile;
      if constexpr (kOp == ROCSHMEM_AMD_PUT) {
        if constexpr (kGran == ROCSHMEM_AMD_WG)
          rocshmem_ctx_putmem_wg(a.ctx, a.dest + off, a.source + off, len, a.pe);
        else if constexpr (kGran == ROCSHMEM_AMD_WAVE)
          rocshmem_ctx_putmem_wave(a.ctx, a.dest + off, a.source + off, len, a.pe);
        else
          rocshmem_ctx_putmem(a.ctx, a.dest + off, a.source + off, len, a.pe);
      } else if constexpr (kOp == ROCSHMEM_AMD_GET) {
        if constexpr (kGran == ROCSHMEM_AMD_WG)
          rocshmem_ctx_getmem_wg(a.ctx, a.dest + off, a.source + off, len, a.pe);
        else if constexpr (kGran == ROCSHMEM_AMD_WAVE)
          rocshmem_ctx_getmem_wave(a.ctx, a.dest + off, a.source + off, len, a.pe);
        else
          rocshmem_ctx_getmem(a.ctx, a.dest + off, a.source + off, len, a.pe);
      } else if constexpr (kOp == ROCSHMEM_AMD_PUT_NBI) {
        if constexpr (kGran == ROCSHMEM_AMD_WG)
          rocshmem_ctx_putmem_nbi_wg(a.ctx, a.dest + off, a.source + off, len, a.pe);
        else if constexpr (kGran == ROCSHMEM_AMD_WAVE)
          rocshmem_ctx_putmem_nbi_wave(a.ctx, a.dest + off, a.source + off, len, a.pe);
        else
          rocshmem_ctx_putmem_nbi(a.ctx, a.dest + off, a.source + off, len, a.pe);
      } else {
        if constexpr (kGran == ROCSHMEM_AMD_WG)
          rocshmem_ctx_getmem_nbi_wg(a.ctx, a.dest + off, a.source + off, len, a.pe);
        else if constexpr (kGran == ROCSHMEM_AMD_WAVE)
          rocshmem_ctx_getmem_nbi_wave(a.ctx, a.dest + off, a.source + off, len, a.pe);
        else
          rocshmem_ctx_getmem_nbi(a.ctx, a.dest + off, a.source + off, len, a.pe);
      }
    }
  }
  // One quiet per group, as a kernel that batches its puts would issue it.
  if (kGran != ROCSHMEM_AMD_WG || threadIdx.x == 0) rocshmem_ctx_quiet(a.ctx);
}

// A put whose source is a __shared__ array, then a get whose destination is
// one: the local side of either call may be LDS (the reference copies through
// generic pointers), which the buffer stores and global loads of the
// cooperative copy cannot reach.
struct StagedArgs {
  char *dest;
  const char *source;
  char *back;
  size_t nbytes;
  rocshmem_ctx_t ctx;
  int pe;
  int gran;
};
__global__ void staged_kernel(StagedArgs a) {
  extern __shared__ __attribute__((aligned(16))) char staged_lds[];
  char *out = staged_lds;
  char *in = staged_lds + ((a.nbytes + 15) & ~size_t{15}) + 3;  // odd offset on purpose
  for (size_t i = threadIdx.x; i < a.nbytes; i += blockDim.x) {
    out[i] = a.source[i];
    in[i] = 0;
  }
  __syncthreads();
  if (a.gran == ROCSHMEM_AMD_WG) {
    rocshmem_ctx_putmem_wg(a.ctx, a.dest, out, a.nbytes, a.pe);
    rocshmem_ctx_quiet(a.ctx);
    __syncthreads();
    rocshmem_ctx_getmem_wg(a.ctx, in, a.dest, a.nbytes, a.pe);
  } else if (a.gran == ROCSHMEM_AMD_WAVE) {
    if (threadIdx.x < 64) {
      rocshmem_ctx_putmem_wave(a.ctx, a.dest, out, a.nbytes, a.pe);
      rocshmem_ctx_quiet(a.ctx);
      rocshmem_ctx_getmem_wave(a.ctx, in, a.dest, a.nbytes, a.pe);
    }
  } else if (threadIdx.x == 0) {
    rocshmem_ctx_putmem(a.ctx, a.dest, out, a.nbytes, a.pe);
    rocshmem_ctx_quiet(a.ctx);
    rocshmem_ctx_getmem(a.ctx, in, a.dest, a.nbytes, a.pe);
  }
  __syncthreads();
  for (size_t i = threadIdx.x; i < a.nbytes; i += blockDim.x) a.back[i] = in[i];
}

// The library's own view of a thread's rank in its work-group and of the
// work-group's size, for any block shape: out[0] = size, out[1 + r] = number
// of threads that believe their rank is r (each must be 1).
__global__ void flat_ids_kernel(unsigned *out) {
  const unsigned r = detail::flat_thread_id();
  if (r == 0) out[0] = detail::flat_block_size();
  atomicAdd(&out[1 + (r < 1024 ? r : 1024)], 1u);
}

// Whole-GPU copy: every thread of the grid is one lane of a single
// cooperative copy; consecutive work-groups take consecutive 1 KiB pieces.
struct BulkArgs {
  char *dst;
  const char *src;
  size_t nbytes;
};

// One wavefront per work-group, one 16-byte vector per lane: each work-group
// moves 1 KiB and leaves.  The destination is peeled to 16-byte alignment by
// block 0 (head and tail bytes); the source may sit at any byte offset.
template <bool kNonTemporal>
__global__ void bulk_copy_kernel(BulkArgs a) {
  size_t head = (16u - (reinterpret_cast<uintptr_t>(a.dst) & 15u)) & 15u;
  if (head > a.nbytes) head = a.nbytes;
  const size_t body = a.nbytes - head;
  const size_t nvec = body >> 4;
  if (blockIdx.x == 0) {
    const size_t tail = body & 15u, done = head + (nvec << 4);
    if (threadIdx.x < head) a.dst[threadIdx.x] = a.src[threadIdx.x];
    if (threadIdx.x < tail) a.dst[done + threadIdx.x] = a.src[done + threadIdx.x];
  }
  char *d = a.dst + head;
  const char *s = a.src + head;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t first = static_cast<size_t>(blockIdx.x) * blockDim.x; first < nvec; first += stride) {
    const size_t v = first + threadIdx.x;
    const size_t left = nvec - first;
    const __amdgpu_buffer_rsrc_t w =
        detail::window_of(d + (first << 4), (left < blockDim.x ? left : blockDim.x) << 4);
    if (v < nvec)
      detail::store16<kNonTemporal>(w, static_cast<uint32_t>(threadIdx.x << 4),
                                    detail::load16<kNonTemporal>(s + (v << 4)));
  }
}

// Launch shape of the whole-GPU copy, from sweeps on MI355X with the buffers
// rotated so nothing is served from the 256 MB memory-side cache.  With
// write-through stores the smallest work-group wins: 64 lanes x one vector
// (1 KiB per work-group) sustains 6.7-6.8 TB/s of read+write traffic, 512
// lanes x two vectors 6.45, 1024 lanes 6.2 and less.  The same holds for a
// pure write stream (6.96 TB/s at one vector per lane, 6.2 at two).
constexpr int kBulkThreads = 64;
constexpr size_t kBulkMaxWgs = size_t{1} << 22;

void launch_bulk(char *dst, const char *src, size_t nbytes, hipStream_t stream) {
  if (!nbytes) return;
  BulkArgs a{dst, src, nbytes};
  const size_t wgs = (nbytes / 16 + kBulkThreads - 1) / kBulkThreads;
  const int grid = static_cast<int>(wgs < kBulkMaxWgs ? (wgs ? wgs : 1) : kBulkMaxWgs);
  if (nbytes >= runtime::rt().state.nt_bytes)
    hipLaunchKernelGGL(bulk_copy_kernel<true>, dim3(grid), dim3(kBulkThreads), 0, stream, a);
  else
    hipLaunchKernelGGL(bulk_copy_kernel<false>, dim3(grid), dim3(kBulkThreads), 0, stream, a);
  DRV_CHECK_HIP(hipGetLastError());
}

// Number of 16-byte vectors (and tail bytes) in which two device buffers differ.
__global__ void compare_kernel(const char *x, const char *y, size_t nbytes,
                               unsigned long long *differing) {
  const size_t nvec = nbytes >> 4;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  unsigned long long bad = 0;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += stride) {
    const detail::u32x4 a = detail::load16<false>(x + (i << 4)), b = detail::load16<false>(y + (i << 4));
    bad += (a.x != b.x) | (a.y != b.y) | (a.z != b.z) | (a.w != b.w);
  }
  if (blockIdx.x == 0)
    for (size_t k = (nvec << 4) + threadIdx.x; k < nbytes; k += blockDim.x) bad += x[k] != y[k];
  if (bad) atomicAdd(differing, bad);
}

// The same byte range of every PE's slice set to one value: blockIdx.y is the PE.
__global__ void fill_every_pe_kernel(char *base, uint64_t pe_stride, size_t nbytes, int byte) {
  char *p = base + static_cast<uint64_t>(blockIdx.y) * pe_stride;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nbytes; i += stride)
    p[i] = static_cast<char>(byte);
}

__global__ void coalesce_kernel(const int *pe, const uint64_t *src, const uint64_t *dst,
                                const uint64_t *size, uint64_t active_mask, int *sends,
                                uint64_t *size_out) {
  const unsigned lane = threadIdx.x;
  if (!((active_mask >> lane) & 1ull)) return;
  size_t sz = size[lane];
  const bool s = detail::wf_coalesce(pe[lane], reinterpret_cast<const void *>(src[lane]),
                                     reinterpret_cast<const void *>(dst[lane]), &sz);
  sends[lane] = s ? 1 : 0;
  size_out[lane] = sz;
}

// One wavefront whose lanes each make their own rocshmem_ctx_putmem call: lane
// i, when its bit of active_mask is set, puts size[i] bytes from source +
// src_off[i] to dest + dst_off[i] on PE pe[i].
struct LanePutArgs {
  char *dest;
  const char *source;
  const int *pe;
  const uint64_t *src_off, *dst_off, *size;
  uint64_t active_mask;
  rocshmem_ctx_t ctx;
};
__global__ void lane_puts_kernel(LanePutArgs a) {
  const unsigned lane = threadIdx.x;
  if (!((a.active_mask >> lane) & 1ull)) return;
  rocshmem_ctx_putmem(a.ctx, a.dest + a.dst_off[lane], a.source + a.src_off[lane], a.size[lane],
                      a.pe[lane]);
}

}  // namespace drv
}  // namespace rocshmem

using namespace rocshmem;
using namespace rocshmem::drv;

extern "C" {

int rocshmem_amd_rma(int rma_op, int gran, void *dest, const void *source, size_t nbytes,
                     size_t tile_bytes, int my_pe, int pe, int n_wgs, int wg_size,
                     int iters, rocshmem_amd_stream_t stream) {
  return rocshmem_amd_rma_messages(rma_op, gran, dest, source, nbytes, tile_bytes, 0, my_pe, pe,
                                   n_wgs, wg_size, iters, stream);
}

int rocshmem_amd_rma_messages(int rma_op, int gran, void *dest, const void *source, size_t nbytes,
                              size_t tile_bytes, int scattered, int my_pe, int pe, int n_wgs,
                              int wg_size, int iters, rocshmem_amd_stream_t stream) {
  if (!valid_actor(my_pe) || !valid_pe(pe) || !valid_launch(n_wgs, wg_size) || iters < 0)
    return -1;
  if (rma_op < ROCSHMEM_AMD_PUT || rma_op > ROCSHMEM_AMD_GET_NBI) return -1;
  if (gran < ROCSHMEM_AMD_THREAD || gran > ROCSHMEM_AMD_WG) return -1;
  // The remote side must be a symmetric address of my_pe; the local side may
  // be any device buffer.
  if (rma_op == ROCSHMEM_AMD_PUT || rma_op == ROCSHMEM_AMD_PUT_NBI) {
    if (!sym_ok_on(dest, nbytes, my_pe) || !local_ok(source, nbytes)) return -1;
  } else {
    if (!sym_ok_on(source, nbytes, my_pe) || !local_ok(dest, nbytes)) return -1;
  }
  size_t groups = n_wgs;
  if (gran == ROCSHMEM_AMD_WAVE) groups *= (wg_size + 63) / 64;
  if (gran == ROCSHMEM_AMD_THREAD) groups *= wg_size;
  RmaArgs a;
  a.dest = static_cast<char *>(dest);
  a.source = static_cast<const char *>(source);
  a.nbytes = nbytes;
  a.tile = tile_bytes ? tile_bytes : auto_tile(nbytes, groups);
  a.ctx = runtime::rt().driver_ctx_handle(my_pe);
  a.pe = pe;
  a.iters = iters;
  a.scatter_mask = 0;
  if (scattered) {
    // A permutation of the tiles: their number must be a power of two (up to
    // 2^32) and the last tile whole.
    const size_t ntiles = nbytes / a.tile;
    if (!ntiles || ntiles * a.tile != nbytes || (ntiles & (ntiles - 1)) || ntiles > (size_t{1} << 32))
      return -1;
    a.scatter_mask = static_cast<uint32_t>(ntiles - 1);
    if (ntiles == 1) a.scatter_mask = 0;
  }
  hipStream_t s = as_stream(stream);
  const dim3 g(n_wgs), b(wg_size);
#define RMA_CASE(OP, GR)                                                               \
  if (rma_op == OP && gran == GR) {                                                    \
    if (a.scatter_mask) hipLaunchKernelGGL((rma_kernel<OP, GR, true>), g, b, 0, s, a);  \
    else hipLaunchKernelGGL((rma_kernel<OP, GR, false>), g, b, 0, s, a);                \
  }
  RMA_CASE(ROCSHMEM_AMD_PUT, ROCSHMEM_AMD_THREAD)
  RMA_CASE(ROCSHMEM_AMD_PUT, ROCSHMEM_AMD_WAVE)
  RMA_CASE(ROCSHMEM_AMD_PUT, ROCSHMEM_AMD_WG)
  RMA_CASE(ROCSHMEM_AMD_GET, ROCSHMEM_AMD_THREAD)
  RMA_CASE(ROCSHMEM_AMD_GET, ROCSHMEM_AMD_WAVE)
  RMA_CASE(ROCSHMEM_AMD_GET, ROCSHMEM_AMD_WG)
  RMA_CASE(ROCSHMEM_AMD_PUT_NBI, ROCSHMEM_AMD_THREAD)
  RMA_CASE(ROCSHMEM_AMD_PUT_NBI, ROCSHMEM_AMD_WAVE)
  RMA_CASE(ROCSHMEM_AMD_PUT_NBI, ROCSHMEM_AMD_WG)
  RMA_CASE(ROCSHMEM_AMD_GET_NBI, ROCSHMEM_AMD_THREAD)
  RMA_CASE(ROCSHMEM_AMD_GET_NBI, ROCSHMEM_AMD_WAVE)
  RMA_CASE(ROCSHMEM_AMD_GET_NBI, ROCSHMEM_AMD_WG)
#undef RMA_CASE
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

int rocshmem_amd_rma_staged(int gran, void *dest, const void *source, void *back, size_t nbytes,
                            int my_pe, int pe, int wg_size, rocshmem_amd_stream_t stream) {
  if (!valid_actor(my_pe) || !valid_pe(pe) || !valid_launch(1, wg_size)) return -1;
  if (gran < ROCSHMEM_AMD_THREAD || gran > ROCSHMEM_AMD_WG) return -1;
  if (!nbytes || nbytes > ROCSHMEM_AMD_STAGED_MAX_BYTES) return -1;
  if (!sym_ok_on(dest, nbytes, my_pe) || !local_ok(source, nbytes) || !local_ok(back, nbytes))
    return -1;
  StagedArgs a;
  a.dest = static_cast<char *>(dest);
  a.source = static_cast<const char *>(source);
  a.back = static_cast<char *>(back);
  a.nbytes = nbytes;
  a.ctx = runtime::rt().driver_ctx_handle(my_pe);
  a.pe = pe;
  a.gran = gran;
  const size_t lds = 2 * ((nbytes + 15) & ~size_t{15}) + 16;
  hipLaunchKernelGGL(staged_kernel, dim3(1), dim3(wg_size), lds, as_stream(stream), a);
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

int rocshmem_amd_flat_ids(int bx, int by, int bz, unsigned *out_host) {
  if (!runtime::rt().live || !out_host || bx < 1 || by < 1 || bz < 1) return -1;
  if (static_cast<long>(bx) * by * bz > 1024 || bz > 64) return -1;
  unsigned *d;
  const size_t bytes = 1026 * sizeof(unsigned);
  DRV_CHECK_HIP(hipMalloc(&d, bytes));
  DRV_CHECK_HIP(hipMemset(d, 0, bytes));
  hipLaunchKernelGGL(flat_ids_kernel, dim3(1), dim3(bx, by, bz), 0, 0, d);
  DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipMemcpy(out_host, d, bytes, hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipFree(d));
  return 0;
}

int rocshmem_amd_compare(const void *x, const void *y, size_t nbytes, uint64_t *differing_out,
                         rocshmem_amd_stream_t stream) {
  if (!runtime::rt().live || !differing_out || !local_ok(x, nbytes) || !local_ok(y, nbytes)) return -1;
  *differing_out = 0;
  if (!nbytes) return 0;
  static unsigned long long *d_count = nullptr;  // allocated once
  static std::once_flag once;
  std::call_once(once, [] { DRV_CHECK_HIP(hipMalloc(&d_count, sizeof(unsigned long long))); });
  hipStream_t s = as_stream(stream);
  DRV_CHECK_HIP(hipMemsetAsync(d_count, 0, sizeof(unsigned long long), s));
  const size_t want = (nbytes / 16 + 255) / 256;
  hipLaunchKernelGGL(compare_kernel, dim3(static_cast<unsigned>(want < 8192 ? (want ? want : 1) : 8192)),
                     dim3(256), 0, s, static_cast<const char *>(x), static_cast<const char *>(y),
                     nbytes, d_count);
  DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipStreamSynchronize(s));
  unsigned long long bad = 0;
  DRV_CHECK_HIP(hipMemcpy(&bad, d_count, sizeof(bad), hipMemcpyDeviceToHost));
  *differing_out = bad;
  return 0;
}

int rocshmem_amd_fill_every_pe(void *sym, int byte, size_t nbytes, rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  auto &r = runtime::rt();
  if (!r.live || !sym_ok_on(sym, nbytes, 0)) return -1;
  if (!nbytes) return 0;
  const size_t want = (nbytes + 255) / 256;
  const dim3 grid(static_cast<unsigned>(want < 1024 ? want : 1024), r.npes);
  hipLaunchKernelGGL(fill_every_pe_kernel, grid, dim3(256), 0, as_stream(stream),
                     static_cast<char *>(sym), r.pe_stride, nbytes, byte);
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

int rocshmem_amd_putmem(void *dest, const void *source, size_t nbytes, int my_pe, int pe,
                        rocshmem_amd_stream_t stream) {
  if (!valid_actor(my_pe) || !valid_pe(pe)) return -1;
  if (!sym_ok_on(dest, nbytes, my_pe) || !local_ok(source, nbytes)) return -1;
  if (!nbytes) return 0;
  char *target = static_cast<char *>(runtime::rt().pe_ptr(dest, pe));
  launch_bulk(target, static_cast<const char *>(source), nbytes, as_stream(stream));
  return 0;
}

int rocshmem_amd_getmem(void *dest, const void *source, size_t nbytes, int my_pe, int pe,
                        rocshmem_amd_stream_t stream) {
  if (!valid_actor(my_pe) || !valid_pe(pe)) return -1;
  if (!sym_ok_on(source, nbytes, my_pe) || !local_ok(dest, nbytes)) return -1;
  if (!nbytes) return 0;
  const char *origin = static_cast<const char *>(runtime::rt().pe_ptr(source, pe));
  launch_bulk(static_cast<char *>(dest), origin, nbytes, as_stream(stream));
  return 0;
}

int rocshmem_amd_lane_puts(void *dest, const void *source, const int *pe, const uint64_t *src_off,
                           const uint64_t *dst_off, const uint64_t *size, uint64_t active_mask,
                           int my_pe, rocshmem_amd_stream_t stream) {
  if (!valid_actor(my_pe) || !pe || !src_off || !dst_off || !size) return -1;
  for (int i = 0; i < 64; ++i) {
    if (!((active_mask >> i) & 1ull)) continue;
    if (!valid_pe(pe[i])) return -1;
    if (!sym_ok_on(static_cast<char *>(dest) + dst_off[i], size[i], my_pe)) return -1;
    if (!local_ok(static_cast<const char *>(source) + src_off[i], size[i])) return -1;
  }
  // The per-lane tables live in one device block: 64 x (pe, three offsets).
  struct Tables {
    int pe[64];
    uint64_t src_off[64], dst_off[64], size[64];
  } host;
  for (int i = 0; i < 64; ++i) {
    host.pe[i] = pe[i];
    host.src_off[i] = src_off[i];
    host.dst_off[i] = dst_off[i];
    host.size[i] = size[i];
  }
  Tables *dev;
  DRV_CHECK_HIP(hipMalloc(&dev, sizeof(Tables)));
  DRV_CHECK_HIP(hipMemcpy(dev, &host, sizeof(Tables), hipMemcpyHostToDevice));
  LanePutArgs a;
  a.dest = static_cast<char *>(dest);
  a.source = static_cast<const char *>(source);
  a.pe = dev->pe;
  a.src_off = dev->src_off;
  a.dst_off = dev->dst_off;
  a.size = dev->size;
  a.active_mask = active_mask;
  a.ctx = runtime::rt().driver_ctx_handle(my_pe);
  hipStream_t s = as_stream(stream);
  hipLaunchKernelGGL(lane_puts_kernel, dim3(1), dim3(64), 0, s, a);
  DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipStreamSynchronize(s));
  DRV_CHECK_HIP(hipFree(dev));
  return 0;
}

int rocshmem_amd_wf_coalesce(const int *pe, const uint64_t *src, const uint64_t *dst,
                             const uint64_t *size, uint64_t active_mask, int *sends_out,
                             uint64_t *size_out) {
  if (!runtime::rt().live || !pe || !src || !dst || !size || !sends_out || !size_out) return -1;
  int *d_pe, *d_sends;
  uint64_t *d_src, *d_dst, *d_size, *d_size_out;
  DRV_CHECK_HIP(hipMalloc(&d_pe, 64 * sizeof(int)));
  DRV_CHECK_HIP(hipMalloc(&d_sends, 64 * sizeof(int)));
  DRV_CHECK_HIP(hipMalloc(&d_src, 64 * 8));
  DRV_CHECK_HIP(hipMalloc(&d_dst, 64 * 8));
  DRV_CHECK_HIP(hipMalloc(&d_size, 64 * 8));
  DRV_CHECK_HIP(hipMalloc(&d_size_out, 64 * 8));
  DRV_CHECK_HIP(hipMemcpy(d_pe, pe, 64 * sizeof(int), hipMemcpyHostToDevice));
  DRV_CHECK_HIP(hipMemcpy(d_src, src, 64 * 8, hipMemcpyHostToDevice));
  DRV_CHECK_HIP(hipMemcpy(d_dst, dst, 64 * 8, hipMemcpyHostToDevice));
  DRV_CHECK_HIP(hipMemcpy(d_size, size, 64 * 8, hipMemcpyHostToDevice));
  DRV_CHECK_HIP(hipMemset(d_sends, 0xff, 64 * sizeof(int)));
  DRV_CHECK_HIP(hipMemset(d_size_out, 0, 64 * 8));
  hipLaunchKernelGGL(coalesce_kernel, dim3(1), dim3(64), 0, 0, d_pe, d_src, d_dst, d_size,
                     active_mask, d_sends, d_size_out);
  DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipMemcpy(sends_out, d_sends, 64 * sizeof(int), hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipMemcpy(size_out, d_size_out, 64 * 8, hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipFree(d_pe));
  DRV_CHECK_HIP(hipFree(d_sends));
  DRV_CHECK_HIP(hipFree(d_src));
  DRV_CHECK_HIP(hipFree(d_dst));
  DRV_CHECK_HIP(hipFree(d_size));
  DRV_CHECK_HIP(hipFree(d_size_out));
  return 0;
}

}  // extern "C"
