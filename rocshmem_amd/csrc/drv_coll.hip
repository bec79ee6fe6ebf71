// Drivers for collectives: the per-work-group device API (one work-group per
// team member) and the host-called whole-GPU forms.
#include <mutex>

#include "drv_common.hpp"
#include "proc_group.hpp"
#include "rocshmem_amd.h"

namespace rocshmem {
namespace drv {

// ---------------------------------------------------------------------------
// Per-work-group device API.  Work-group j acts for team member j.
// ---------------------------------------------------------------------------
struct WgCollArgs {
  detail::Team *team_row;    // team objects of this team, indexed by world PE
  detail::Context *ctx_row;  // default contexts, indexed by world PE
  char *dest0;               // addresses of the buffers on world PE 0
  const char *src0;
  uint64_t pe_stride;
  int pe_start;
  int stride;
  int nelems;
  int root;
  int *status;
};

struct Member {
  rocshmem_ctx_t ctx;
  rocshmem_team_t team;
  char *dest;
  const char *source;
};
__device__ __forceinline__ Member member_of(const WgCollArgs &a) {
  const int pe = a.pe_start + static_cast<int>(blockIdx.x) * a.stride;
  Member m;
  m.ctx = rocshmem_ctx_t{a.ctx_row + pe, &a.team_row[pe].wrt_world};
  m.team = reinterpret_cast<rocshmem_team_t>(a.team_row + pe);
  m.dest = a.dest0 + static_cast<uint64_t>(pe) * a.pe_stride;
  m.source = a.src0 + static_cast<uint64_t>(pe) * a.pe_stride;
  return m;
}

// Public reduce entry point for (T, Op).
template <typename T, ROCSHMEM_OP Op>
struct PublicReduce;
#define DRV_PUBLIC_REDUCE(T, TN, OPN, OP)                                          \
  template <>                                                                      \
  struct PublicReduce<T, OP> {                                                     \
    using storage = T;                                                             \
    __device__ __forceinline__ static int call(rocshmem_ctx_t c, rocshmem_team_t t, T *d, \
                                              const T *s, int n) {                             \
      return rocshmem_ctx_##TN##_##OPN##_wg_reduce(c, t, d, s, n);                 \
    }                                                                              \
  };
#define DRV_PUBLIC_ARITH(T, TN)                \
  DRV_PUBLIC_REDUCE(T, TN, sum, ROCSHMEM_SUM)  \
  DRV_PUBLIC_REDUCE(T, TN, max, ROCSHMEM_MAX)  \
  DRV_PUBLIC_REDUCE(T, TN, min, ROCSHMEM_MIN)  \
  DRV_PUBLIC_REDUCE(T, TN, prod, ROCSHMEM_PROD)
#define DRV_PUBLIC_INT(T, TN)                  \
  DRV_PUBLIC_ARITH(T, TN)                      \
  DRV_PUBLIC_REDUCE(T, TN, and, ROCSHMEM_AND)  \
  DRV_PUBLIC_REDUCE(T, TN, or, ROCSHMEM_OR)    \
  DRV_PUBLIC_REDUCE(T, TN, xor, ROCSHMEM_XOR)
DRV_PUBLIC_INT(short, short)
DRV_PUBLIC_INT(int, int)
DRV_PUBLIC_INT(long, long)
DRV_PUBLIC_INT(long long, longlong)
DRV_PUBLIC_ARITH(float, float)
DRV_PUBLIC_ARITH(double, double)
template <>
struct PublicReduce<rocshmem_bf16, ROCSHMEM_SUM> {
  using storage = rocshmem_bf16;
  __device__ __forceinline__ static int call(rocshmem_ctx_t c, rocshmem_team_t t, rocshmem_bf16 *d,
                             const rocshmem_bf16 *s, int n) {
    return rocshmem_ctx_bf16_sum_wg_reduce(c, t, d, s, n);
  }
};

template <typename T, ROCSHMEM_OP Op>
__global__ void wg_reduce_kernel(WgCollArgs a) {
  const Member m = member_of(a);
  const int rc = PublicReduce<T, Op>::call(m.ctx, m.team, reinterpret_cast<T *>(m.dest),
                                           reinterpret_cast<const T *>(m.source), a.nelems);
  if (threadIdx.x == 0 && rc != ROCSHMEM_SUCCESS) atomicMax(a.status, rc);
}

// Several teams over the same PEs at once, the way the reference's testers
// scale a device collective (one team per work-group,
// tests/functional_tests/team_reduction_tester.cpp): work-group (x, y) acts
// for member x of team y and reduces the y-th slice of the arrays.
constexpr int kMaxTeamsPerLaunch = 256;
struct WgTeamsArgs {
  detail::Team *rows[kMaxTeamsPerLaunch];  // team objects of each team, indexed by world PE
  detail::Context *ctx_row;
  char *dest0;
  const char *src0;
  uint64_t pe_stride;
  int pe_start;
  int stride;
  int nelems;       // all slices together
  int slice_elems;  // per call: team y reduces slices y, y + teams, ... one call each
  int iters;        // passes over the whole range, one after the other
  int *status;      // [teams] largest return code each team saw
};

template <typename T, ROCSHMEM_OP Op>
__global__ void wg_reduce_teams_kernel(WgTeamsArgs a) {
  const int pe = a.pe_start + static_cast<int>(blockIdx.x) * a.stride;
  detail::Team *row = a.rows[blockIdx.y];
  const rocshmem_ctx_t ctx{a.ctx_row + pe, &row[pe].wrt_world};
  const rocshmem_team_t team = reinterpret_cast<rocshmem_team_t>(row + pe);
  T *dest = reinterpret_cast<T *>(a.dest0 + static_cast<uint64_t>(pe) * a.pe_stride);
  const T *source = reinterpret_cast<const T *>(a.src0 + static_cast<uint64_t>(pe) * a.pe_stride);
  const long step = static_cast<long>(gridDim.y) * a.slice_elems;
  for (int it = 0; it < a.iters; ++it) {
    for (long lo = static_cast<long>(blockIdx.y) * a.slice_elems; lo < a.nelems; lo += step) {
      const long left = a.nelems - lo;
      const int cnt = static_cast<int>(left < a.slice_elems ? left : a.slice_elems);
      const int rc = PublicReduce<T, Op>::call(ctx, team, dest + lo, source + lo, cnt);
      if (threadIdx.x == 0 && rc != ROCSHMEM_SUCCESS) atomicMax(a.status + blockIdx.y, rc);
    }
  }
}

// The members' shares of one all-reduce computed by work-groups of DIFFERENT
// sizes: block k stands for team member k and brings lanes[k] lanes (its other
// threads leave at once).  One launch has one block size, so this calls the
// fold that wg_reduce runs between its barriers directly; a member's share
// must not depend on how many lanes any member brings.
struct FoldSharesArgs {
  int *dst0;
  const int *src0;
  int64_t hop;
  int np;
  int nelems;
  int lanes[detail::SyncPad::kMaxPes];
};
__global__ void fold_shares_kernel(FoldSharesArgs a) {
  const int mine = a.lanes[blockIdx.x];
  if (static_cast<int>(threadIdx.x) >= mine) return;
  detail::fold_span_any<int, ROCSHMEM_SUM, false, detail::SHARE_BLOCKS>(a.dst0, a.src0, a.hop, a.np, 0,
                                                        static_cast<size_t>(a.nelems), threadIdx.x,
                                                        mine, blockIdx.x, a.np);
}

// Sets n words to zero from the stream (a plain kernel: safe to record in a
// HIP graph, which a memset node is not on every driver).
__global__ void clear_words_kernel(int *words, int n) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) words[i] = 0;
}

// Status words of rocshmem_amd_wg_reduce_teams_static: one per team of a
// launch.  Lives in the code object, so the entry point needs no allocation;
// every call on a GPU shares it.
constexpr int kStaticStatusWords = kMaxTeamsPerLaunch;
static __device__ __align__(256) int scratch[kStaticStatusWords];

enum WgMove { MOVE_ALLTOALL, MOVE_BROADCAST, MOVE_FCOLLECT };

template <typename T, int kMove>
__device__ __forceinline__ void wg_move_call(const Member &m, int n, int root);
#define DRV_MOVE(T, TN)                                                            \
  template <>                                                                      \
  __device__ __forceinline__ void wg_move_call<T, MOVE_ALLTOALL>(const Member &m,  \
                                                                 int n, int) {     \
    rocshmem_ctx_##TN##_wg_alltoall(m.ctx, m.team, reinterpret_cast<T *>(m.dest),  \
                                    reinterpret_cast<const T *>(m.source), n);     \
  }                                                                                \
  template <>                                                                      \
  __device__ __forceinline__ void wg_move_call<T, MOVE_BROADCAST>(const Member &m, \
                                                                  int n, int root) { \
    rocshmem_ctx_##TN##_wg_broadcast(m.ctx, m.team, reinterpret_cast<T *>(m.dest), \
                                     reinterpret_cast<const T *>(m.source), n, root); \
  }                                                                                \
  template <>                                                                      \
  __device__ __forceinline__ void wg_move_call<T, MOVE_FCOLLECT>(const Member &m,  \
                                                                 int n, int) {     \
    rocshmem_ctx_##TN##_wg_fcollect(m.ctx, m.team, reinterpret_cast<T *>(m.dest),  \
                                    reinterpret_cast<const T *>(m.source), n);     \
  }
DRV_MOVE(char, char)
DRV_MOVE(short, short)
DRV_MOVE(int, int)
DRV_MOVE(long, long)

template <typename T, int kMove>
__global__ void wg_move_kernel(WgCollArgs a) {
  wg_move_call<T, kMove>(member_of(a), a.nelems, a.root);
}

struct SyncArgs {
  detail::Team *team_row;
  detail::Context *ctx_row;
  uint64_t *scratch0;  // address on world PE 0
  uint64_t pe_stride;
  int pe_start, stride, size;
  int fn;
  int rounds;
  int *errors;
};

__global__ void wg_sync_kernel(SyncArgs a) {
  const int j = blockIdx.x;
  const int pe = a.pe_start + j * a.stride;
  const int next = (j + 1) % a.size;  // team-relative: p() translates it
  rocshmem_ctx_t ctx{a.ctx_row + pe, &a.team_row[pe].wrt_world};
  rocshmem_team_t team = reinterpret_cast<rocshmem_team_t>(a.team_row + pe);
  uint64_t *mine = reinterpret_cast<uint64_t *>(reinterpret_cast<char *>(a.scratch0) +
                                                static_cast<uint64_t>(pe) * a.pe_stride);
  for (int r = 1; r <= a.rounds; ++r) {
    if (threadIdx.x == 0) rocshmem_ctx_uint64_p(ctx, mine, static_cast<uint64_t>(r), next);
    if (a.fn == ROCSHMEM_AMD_BARRIER_ALL) rocshmem_ctx_wg_barrier_all(ctx);
    else if (a.fn == ROCSHMEM_AMD_SYNC_ALL) rocshmem_ctx_wg_sync_all(ctx);
    else rocshmem_ctx_wg_team_sync(ctx, team);
    if (threadIdx.x == 0) {
      const uint64_t seen = rocshmem_ctx_uint64_atomic_fetch(ctx, mine, pe);
      if (seen != static_cast<uint64_t>(r)) atomicAdd(a.errors, 1);
    }
    // Nobody may overwrite the word of round r before everyone has read it.
    if (a.fn == ROCSHMEM_AMD_BARRIER_ALL) rocshmem_ctx_wg_barrier_all(ctx);
    else if (a.fn == ROCSHMEM_AMD_SYNC_ALL) rocshmem_ctx_wg_sync_all(ctx);
    else rocshmem_ctx_wg_team_sync(ctx, team);
  }
}

// ---------------------------------------------------------------------------
// Host-called, whole-GPU forms.
// ---------------------------------------------------------------------------
template <typename E>
struct GridReduceArgs {
  typename detail::ElemTraits<E>::storage *dst0;        // buffers on the first member
  const typename detail::ElemTraits<E>::storage *src0;
  int64_t hop;                                          // bytes between members
  int np;
  size_t n;
  size_t span;                                          // elements per work-group span
};

// Each work-group folds contiguous spans of the index space: it reads the span
// from all P sources and writes it to all P destinations.
template <typename E, ROCSHMEM_OP Op, bool kNonTemporal>
__global__ void grid_reduce_kernel(GridReduceArgs<E> a) {
  using S = typename detail::ElemTraits<E>::storage;
  const uintptr_t mis = reinterpret_cast<uintptr_t>(a.dst0) & 15u;
  size_t head = mis ? (16u - mis) / sizeof(S) : 0;
  if (head > a.n) head = a.n;
  if (blockIdx.x == 0 && head)
    detail::fold_span_any<E, Op, false>(a.dst0, a.src0, a.hop, a.np, 0, head, threadIdx.x,
                                        blockDim.x);
  const size_t body = a.n - head;
  const size_t nspans = (body + a.span - 1) / a.span;
  for (size_t s = blockIdx.x; s < nspans; s += gridDim.x) {
    const size_t lo = head + s * a.span;
    const size_t hi = lo + a.span < a.n ? lo + a.span : a.n;
    detail::fold_span_any<E, Op, kNonTemporal>(a.dst0, a.src0, a.hop, a.np, lo, hi,
                                               threadIdx.x, blockDim.x);
  }
}

template <typename E, ROCSHMEM_OP Op>
void launch_grid_reduce(void *dst0, const void *src0, int64_t hop, int np, size_t n,
                        hipStream_t stream) {
  using S = typename detail::ElemTraits<E>::storage;
  GridReduceArgs<E> a;
  a.dst0 = static_cast<S *>(dst0);
  a.src0 = static_cast<const S *>(src0);
  a.hop = hop;
  a.np = np;
  a.n = n;
  // Shape from sweeps on MI355X (P = 8, 64 Mi elements): one wavefront per
  // work-group, one 16-byte vector per lane and source, non-temporal loads and
  // stores.  A wavefront then has P KiB of loads in flight, and the rate peaks
  // when a CU holds 48-64 KiB of them: for P = 8, 6 or 8 wavefronts per CU give
  // 6.55 TB/s (fp32, bf16 and int64 alike), 12 give 6.51, 16 or the full 32
  // 6.46-6.49, and 5 only 6.25 - so 8, the side of the optimum away from the
  // drop.  The residency is set by asking for LDS the kernel never touches.
  const int wg = 64;
  size_t lds = 0;
  if (np == 2 || np == 4 || np == 8) {
    const size_t waves_per_cu = (64 * 1024) / (static_cast<size_t>(np) * 1024);
    // An equal share of the CU's LDS per wavefront, whatever the part has
    // (160 KiB on MI355X), less the 512 bytes the allocation granule may add.
    static const size_t lds_per_cu = [] {
      int dev = 0, bytes = 0;
      if (hipGetDevice(&dev) != hipSuccess ||
          hipDeviceGetAttribute(&bytes, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev) !=
              hipSuccess || bytes <= 0) {
        (void)hipGetLastError();
        return size_t{0};
      }
      return static_cast<size_t>(bytes);
    }();
    if (waves_per_cu < 32 && lds_per_cu / waves_per_cu > 1024) lds = lds_per_cu / waves_per_cu - 512;
    if (lds > (size_t{64} << 10)) lds = size_t{64} << 10;
  }
  a.span = static_cast<size_t>(wg) * (16 / sizeof(S));
  const size_t nspans = (n + a.span - 1) / a.span;
  const size_t max_wgs = size_t{1} << 20;
  const int grid = static_cast<int>(nspans < max_wgs ? (nspans ? nspans : 1) : max_wgs);
  const bool nt = n * sizeof(S) >= runtime::rt().state.nt_bytes;
  if (nt)
    hipLaunchKernelGGL((grid_reduce_kernel<E, Op, true>), dim3(grid), dim3(wg), lds, stream, a);
  else
    hipLaunchKernelGGL((grid_reduce_kernel<E, Op, false>), dim3(grid), dim3(wg), lds, stream, a);
  DRV_CHECK_HIP(hipGetLastError());
}

// Whole-GPU alltoall / broadcast / fcollect.  One wavefront per work-group,
// 1 KiB per work-group, as in the whole-GPU copy.
struct GridMoveArgs {
  char *dest0;        // buffers on the first member
  const char *src0;
  int64_t hop;
  int np;
  int root;
  size_t nbytes;      // per block
  size_t span;
};

// alltoall: blockIdx.z is the sender, blockIdx.y the receiver, blockIdx.x
// walks the spans of their block.  Every byte is read once and written once.
template <bool kNonTemporal>
__global__ void grid_alltoall_kernel(GridMoveArgs a) {
  const int i = static_cast<int>(blockIdx.z);  // sender
  const int j = static_cast<int>(blockIdx.y);  // receiver
  char *d = a.dest0 + j * a.hop + static_cast<size_t>(i) * a.nbytes;
  const char *src = a.src0 + i * a.hop + static_cast<size_t>(j) * a.nbytes;
  for (size_t off = blockIdx.x * a.span; off < a.nbytes; off += gridDim.x * a.span) {
    const size_t len = a.nbytes - off < a.span ? a.nbytes - off : a.span;
    detail::copy_lanes_impl<1, kNonTemporal>(d + off, src + off, len, threadIdx.x, blockDim.x);
  }
}

// broadcast / fcollect: a block goes to every member, so it is read once and
// the registers are stored P (or P-1) times; the kernel is a pure write stream
// with 1/P of its traffic in reads.  blockIdx.y names the sender.  All
// receivers share the destination's alignment (the hop is a multiple of 16),
// so one peel serves them all.
template <int kMove, bool kNonTemporal>
__global__ void grid_fanout_kernel(GridMoveArgs a) {
  const int i = kMove == MOVE_BROADCAST ? a.root : static_cast<int>(blockIdx.y);
  const int skip = kMove == MOVE_BROADCAST ? a.root : -1;
  char *d = a.dest0 + (kMove == MOVE_FCOLLECT ? static_cast<size_t>(i) * a.nbytes : 0);
  const char *s = a.src0 + i * a.hop;
  size_t head = (16u - (reinterpret_cast<uintptr_t>(d) & 15u)) & 15u;
  if (head > a.nbytes) head = a.nbytes;
  const size_t body = a.nbytes - head;
  const size_t nvec = body >> 4;
  if (blockIdx.x == 0) {
    const size_t tail = body & 15u, done = head + (nvec << 4);
    for (int j = 0; j < a.np; ++j) {
      if (j == skip) continue;
      char *dj = d + j * a.hop;
      if (threadIdx.x < head) dj[threadIdx.x] = s[threadIdx.x];
      if (threadIdx.x < tail) dj[done + threadIdx.x] = s[done + threadIdx.x];
    }
  }
  d += head;
  s += head;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t first = static_cast<size_t>(blockIdx.x) * blockDim.x; first < nvec; first += stride) {
    const size_t v = first + threadIdx.x;
    const size_t left = nvec - first;
    const size_t bytes = (left < blockDim.x ? left : blockDim.x) << 4;
    detail::u32x4 val{};
    if (v < nvec) val = detail::load16<kNonTemporal>(s + (v << 4));
    for (int j = 0; j < a.np; ++j) {
      if (j == skip) continue;
      const __amdgpu_buffer_rsrc_t w = detail::window_of(d + j * a.hop + (first << 4), bytes);
      if (v < nvec)
        detail::store16<kNonTemporal>(w, static_cast<uint32_t>(threadIdx.x << 4), val);
    }
  }
}

constexpr int kMoveThreads = 64;
constexpr size_t kMoveMaxWgs = size_t{1} << 22;

template <int kMove>
void launch_grid_move(char *dest0, const char *src0, int64_t hop, int np, int root,
                      size_t nbytes, hipStream_t stream) {
  if (!nbytes) return;
  GridMoveArgs a{dest0, src0, hop, np, root, nbytes, size_t{kMoveThreads} * 16};
  const bool nt = nbytes >= runtime::rt().state.nt_bytes;
  const size_t rows = kMove == MOVE_ALLTOALL ? static_cast<size_t>(np) * np
                    : kMove == MOVE_FCOLLECT ? static_cast<size_t>(np) : 1;
  const size_t spans = (nbytes + a.span - 1) / a.span;
  const size_t max_x = kMoveMaxWgs / rows;
  const unsigned gx = static_cast<unsigned>(spans < max_x ? spans : (max_x ? max_x : 1));
  const dim3 grid = kMove == MOVE_ALLTOALL ? dim3(gx, np, np) : dim3(gx, static_cast<unsigned>(rows));
  const dim3 block(kMoveThreads);
  if constexpr (kMove == MOVE_ALLTOALL) {
    if (nt) hipLaunchKernelGGL(grid_alltoall_kernel<true>, grid, block, 0, stream, a);
    else hipLaunchKernelGGL(grid_alltoall_kernel<false>, grid, block, 0, stream, a);
  } else {
    if (nt) hipLaunchKernelGGL((grid_fanout_kernel<kMove, true>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((grid_fanout_kernel<kMove, false>), grid, block, 0, stream, a);
  }
  DRV_CHECK_HIP(hipGetLastError());
}

// ---------------------------------------------------------------------------
// One process per PE: host collectives by pulling.  Every member's process
// reads the other members' buffers through its own mappings of their slices
// (which sit at unrelated addresses, hence a table of pointers) and writes its
// own result; the processes meet before (sources final) and after (everybody
// has read them).
// ---------------------------------------------------------------------------
constexpr int kMaxTableMembers = 64;
template <typename E>
struct TableReduceArgs {
  const typename detail::ElemTraits<E>::storage *src[kMaxTableMembers];  // ascending members
  typename detail::ElemTraits<E>::storage *out;
  size_t n;
  int np;
};
template <typename E, ROCSHMEM_OP Op>
__global__ void table_reduce_kernel(TableReduceArgs<E> a) {
  using Tr = detail::ElemTraits<E>;
  using A = typename Tr::accum;
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < a.n; i += stride) {
    A acc = Tr::widen(a.src[0][i]);
    for (int p = 1; p < a.np; ++p) acc = detail::combine<A, Op>(acc, Tr::widen(a.src[p][i]));
    a.out[i] = Tr::narrow(acc);
  }
}

void launch_bulk(char *dst, const char *src, size_t nbytes, hipStream_t stream);

// Resolve a team handle (of the acting PE) to what the kernels need.
struct TeamView {
  const detail::Team *host;
  detail::Team *row;
};
inline bool view_team(rocshmem_amd_team_t team, TeamView *v) {
  auto &r = runtime::rt();
  v->host = r.host_team(r.my_view(static_cast<rocshmem_team_t>(team)));
  if (!v->host || v->host->my_pe < 0) return false;
  v->row = r.d_teams + static_cast<size_t>(v->host->pool_index) * r.npes;
  return true;
}
// Address on world PE 0 of a symmetric address given for the acting PE.
inline char *on_pe0(const void *p) {
  auto &r = runtime::rt();
  return const_cast<char *>(static_cast<const char *>(p)) -
         static_cast<size_t>(r.me()) * r.pe_stride;
}
inline bool in_heap(const void *p) {
  return runtime::rt().offset_of(p) != runtime::Pow2Allocator::kNoBlock;
}

template <typename T, ROCSHMEM_OP Op>
bool launch_wg_reduce(const WgCollArgs &a, int size, int wg_size, hipStream_t s) {
  if (!grid_fits(wg_reduce_kernel<T, Op>, size, wg_size)) return false;
  hipLaunchKernelGGL((wg_reduce_kernel<T, Op>), dim3(size), dim3(wg_size), 0, s, a);
  return true;
}

}  // namespace drv
}  // namespace rocshmem

using namespace rocshmem;
using namespace rocshmem::drv;

namespace {

template <typename Fn>
bool for_dtype_op(int dtype, int op, Fn &&fn) {
  // fn is a generic lambda taking (type tag, op tag).
  auto ops_int = [&](auto tag) -> bool {
    switch (op) {
      case ROCSHMEM_AMD_SUM: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_SUM>{}); return true;
      case ROCSHMEM_AMD_MAX: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_MAX>{}); return true;
      case ROCSHMEM_AMD_MIN: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_MIN>{}); return true;
      case ROCSHMEM_AMD_PROD: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_PROD>{}); return true;
      case ROCSHMEM_AMD_AND: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_AND>{}); return true;
      case ROCSHMEM_AMD_OR: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_OR>{}); return true;
      case ROCSHMEM_AMD_XOR: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_XOR>{}); return true;
      default: return false;
    }
  };
  auto ops_float = [&](auto tag) -> bool {
    switch (op) {
      case ROCSHMEM_AMD_SUM: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_SUM>{}); return true;
      case ROCSHMEM_AMD_MAX: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_MAX>{}); return true;
      case ROCSHMEM_AMD_MIN: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_MIN>{}); return true;
      case ROCSHMEM_AMD_PROD: fn(tag, std::integral_constant<ROCSHMEM_OP, ROCSHMEM_PROD>{}); return true;
      default: return false;
    }
  };
  switch (dtype) {
    case ROCSHMEM_AMD_SHORT: return ops_int(static_cast<short *>(nullptr));
    case ROCSHMEM_AMD_INT: return ops_int(static_cast<int *>(nullptr));
    case ROCSHMEM_AMD_LONG: return ops_int(static_cast<long *>(nullptr));
    case ROCSHMEM_AMD_LONGLONG: return ops_int(static_cast<long long *>(nullptr));
    case ROCSHMEM_AMD_FLOAT: return ops_float(static_cast<float *>(nullptr));
    case ROCSHMEM_AMD_DOUBLE: return ops_float(static_cast<double *>(nullptr));
    case ROCSHMEM_AMD_BF16:
      if (op != ROCSHMEM_AMD_SUM) return false;
      fn(static_cast<rocshmem_bf16 *>(nullptr), std::integral_constant<ROCSHMEM_OP, ROCSHMEM_SUM>{});
      return true;
    default: return false;
  }
}

// Engine element tag for a public element type.
template <typename T> struct EngineTag { using type = T; };
template <> struct EngineTag<rocshmem_bf16> { using type = detail::Bf16Tag; };

size_t dtype_size(int dtype) {
  switch (dtype) {
    case ROCSHMEM_AMD_SHORT: case ROCSHMEM_AMD_BF16: return 2;
    case ROCSHMEM_AMD_INT: case ROCSHMEM_AMD_FLOAT: case ROCSHMEM_AMD_UINT: return 4;
    default: return 8;
  }
}

int grid_reduce_common(int dtype, int op, void *dst_first, const void *src_first, int64_t hop,
                       int np, int nreduce, hipStream_t stream) {
  if (nreduce < 0) return -1;
  if (nreduce == 0) return 0;
  const bool ok = for_dtype_op(dtype, op, [&](auto *tag, auto opc) {
    using T = typename std::remove_pointer<decltype(tag)>::type;
    using E = typename EngineTag<T>::type;
    launch_grid_reduce<E, decltype(opc)::value>(dst_first, src_first, hop, np,
                                                static_cast<size_t>(nreduce), stream);
  });
  return ok ? 0 : -1;
}

WgCollArgs make_wg_args(const TeamView &v, void *dest, const void *source, int nelems, int root,
                        int *status) {
  auto &r = runtime::rt();
  WgCollArgs a;
  a.team_row = v.row;
  a.ctx_row = r.driver_ctx_row();
  a.dest0 = on_pe0(dest);
  a.src0 = on_pe0(source);
  a.pe_stride = r.pe_stride;
  a.pe_start = v.host->wrt_world.pe_start;
  a.stride = v.host->wrt_world.stride;
  a.nelems = nelems;
  a.root = root;
  a.status = status;
  return a;
}

template <int kMove>
int wg_move_common(int elem_size, rocshmem_amd_team_t team, void *dest, const void *source,
                   int nelems, int root, int wg_size, hipStream_t s) {
  TeamView v;
  if (!view_team(team, &v) || !valid_launch(1, wg_size) || nelems < 0) return -1;
  {
    const size_t blk = static_cast<size_t>(nelems) * elem_size;
    const size_t all = blk * v.host->num_pes;
    const int me = runtime::rt().me();
    if (!sym_ok_on(dest, kMove == MOVE_BROADCAST ? blk : all, me)) return -1;
    if (!sym_ok_on(source, kMove == MOVE_ALLTOALL ? all : blk, me)) return -1;
  }
  if (kMove == MOVE_BROADCAST && (root < 0 || root >= v.host->num_pes)) return -1;
  const WgCollArgs a = make_wg_args(v, dest, source, nelems, root, nullptr);
  const dim3 g(v.host->num_pes), b(wg_size);
#define DRV_MOVE_CASE(BYTES, T)                                              \
  case BYTES:                                                                \
    if (!grid_fits(wg_move_kernel<T, kMove>, g.x, wg_size)) return -1;       \
    hipLaunchKernelGGL((wg_move_kernel<T, kMove>), g, b, 0, s, a);           \
    break;
  switch (elem_size) {
    DRV_MOVE_CASE(1, char)
    DRV_MOVE_CASE(2, short)
    DRV_MOVE_CASE(4, int)
    DRV_MOVE_CASE(8, long)
    default: return -1;
  }
#undef DRV_MOVE_CASE
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

template <int kMove>
int procs_move(void *dest, const void *source, size_t nbytes, int root, int start, int stride, int size,
               hipStream_t s);

template <int kMove>
int grid_move_common(rocshmem_amd_team_t team, void *dest, const void *source, size_t nbytes,
                     int root, hipStream_t s) {
  TeamView v;
  if (!view_team(team, &v)) return -1;
  if (runtime::rt().nprocs)
    return procs_move<kMove>(dest, source, nbytes, root, v.host->wrt_world.pe_start,
                             v.host->wrt_world.stride, v.host->num_pes, s);
  {
    const size_t all = nbytes * v.host->num_pes;
    const int me = runtime::rt().me();
    if (!sym_ok_on(dest, kMove == MOVE_BROADCAST ? nbytes : all, me)) return -1;
    if (!sym_ok_on(source, kMove == MOVE_ALLTOALL ? all : nbytes, me)) return -1;
  }
  if (kMove == MOVE_BROADCAST && (root < 0 || root >= v.host->num_pes)) return -1;
  auto &r = runtime::rt();
  const int64_t first = static_cast<int64_t>(v.host->wrt_world.pe_start) * r.pe_stride;
  const int64_t hop = static_cast<int64_t>(v.host->wrt_world.stride) * r.pe_stride;
  launch_grid_move<kMove>(on_pe0(dest) + first, on_pe0(source) + first, hop, v.host->num_pes,
                          root, nbytes, s);
  return 0;
}

// ---- one process per PE -------------------------------------------------------
struct ProcSet {
  int start, stride, size, my_index;
};
// The caller's place in the strided set of world PEs, or false if it is none.
bool proc_member(int start, int stride, int size, ProcSet *out) {
  auto &r = runtime::rt();
  const int off = r.me() - start;
  if (size < 1 || size > kMaxTableMembers || stride < 1 || off < 0 || off % stride || off / stride >= size)
    return false;
  *out = ProcSet{start, stride, size, off / stride};
  return true;
}

int procs_reduce(int dtype, int op, void *dest, const void *source, int nreduce, int start, int stride,
                 int size, hipStream_t s) {
  auto &r = runtime::rt();
  ProcSet set;
  if (nreduce < 0 || !proc_member(start, stride, size, &set)) return -1;
  const size_t es = dtype_size(dtype);
  const size_t bytes = static_cast<size_t>(nreduce) * es;
  if (!sym_ok(dest, bytes) || !sym_ok(source, bytes)) return -1;
  const uint64_t dst_off = r.offset_of(dest), src_off = r.offset_of(source);
  if (nreduce == 0) return 0;
  char *temp = nullptr;
  DRV_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&temp), bytes));
  runtime::procs_meet(start, stride, size);  // every member's source is final
  const bool ok = for_dtype_op(dtype, op, [&](auto *tag, auto opc) {
    using T = typename std::remove_pointer<decltype(tag)>::type;
    using E = typename EngineTag<T>::type;
    using S = typename detail::ElemTraits<E>::storage;
    TableReduceArgs<E> a;
    for (int k = 0; k < size; ++k)
      a.src[k] = reinterpret_cast<const S *>(r.slice_base(start + k * stride) + src_off);
    a.out = reinterpret_cast<S *>(temp);
    a.n = static_cast<size_t>(nreduce);
    a.np = size;
    const size_t want = (a.n + 255) / 256;
    hipLaunchKernelGGL((table_reduce_kernel<E, decltype(opc)::value>),
                       dim3(static_cast<unsigned>(want < 4096 ? want : 4096)), dim3(256), 0, s, a);
  });
  if (ok) DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipStreamSynchronize(s));
  runtime::procs_meet(start, stride, size);  // everybody has read every source: dest may alias one
  if (ok) {
    launch_bulk(r.slice_base(r.me()) + dst_off, temp, bytes, s);
    DRV_CHECK_HIP(hipStreamSynchronize(s));
  }
  DRV_CHECK_HIP(hipFree(temp));
  return ok ? 0 : -1;
}

// kMove as in the device forms; nbytes per block; root: index in the set.
template <int kMove>
int procs_move(void *dest, const void *source, size_t nbytes, int root, int start, int stride, int size,
               hipStream_t s) {
  auto &r = runtime::rt();
  ProcSet set;
  if (!proc_member(start, stride, size, &set)) return -1;
  if (kMove == MOVE_BROADCAST && (root < 0 || root >= size)) return -1;
  const size_t all = nbytes * size;
  if (!sym_ok(dest, kMove == MOVE_BROADCAST ? nbytes : all)) return -1;
  if (!sym_ok(source, kMove == MOVE_ALLTOALL ? all : nbytes)) return -1;
  const uint64_t dst_off = r.offset_of(dest), src_off = r.offset_of(source);
  if (!nbytes) return 0;
  char *mine = r.slice_base(r.me()) + dst_off;
  runtime::procs_meet(start, stride, size);
  if (kMove == MOVE_BROADCAST) {
    if (set.my_index != root)
      launch_bulk(mine, r.slice_base(start + root * stride) + src_off, nbytes, s);
  } else {
    for (int j = 0; j < size; ++j) {
      const char *from = r.slice_base(start + j * stride) + src_off +
                         (kMove == MOVE_ALLTOALL ? static_cast<size_t>(set.my_index) * nbytes : 0);
      launch_bulk(mine + static_cast<size_t>(j) * nbytes, from, nbytes, s);
    }
  }
  DRV_CHECK_HIP(hipStreamSynchronize(s));
  runtime::procs_meet(start, stride, size);
  return 0;
}

}  // namespace

extern "C" {

int rocshmem_amd_wg_reduce(int dtype, int op, rocshmem_amd_team_t team, void *dest,
                           const void *source, int nreduce, int wg_size,
                           rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  TeamView v;
  if (!view_team(team, &v) || !valid_launch(1, wg_size) || nreduce < 0) return -1;
  {
    const size_t bytes = static_cast<size_t>(nreduce) * dtype_size(dtype);
    const int me = runtime::rt().me();
    if (!sym_ok_on(dest, bytes, me) || !sym_ok_on(source, bytes, me)) return -1;
  }
  int *d_status;
  DRV_CHECK_HIP(hipMalloc(&d_status, sizeof(int)));
  DRV_CHECK_HIP(hipMemset(d_status, 0, sizeof(int)));
  const WgCollArgs a = make_wg_args(v, dest, source, nreduce, 0, d_status);
  hipStream_t s = as_stream(stream);
  bool launched = false;
  const bool ok = for_dtype_op(dtype, op, [&](auto *tag, auto opc) {
    using T = typename std::remove_pointer<decltype(tag)>::type;
    launched = launch_wg_reduce<T, decltype(opc)::value>(a, v.host->num_pes, wg_size, s);
  });
  int status = -1;
  if (ok && launched) {
    DRV_CHECK_HIP(hipGetLastError());
    DRV_CHECK_HIP(hipStreamSynchronize(s));
    DRV_CHECK_HIP(hipMemcpy(&status, d_status, sizeof(int), hipMemcpyDeviceToHost));
  }
  DRV_CHECK_HIP(hipFree(d_status));
  return status;
}

// Validates and enqueues the many-teams reduce; d_status: n_teams device words,
// zeroed by the caller or, with clear_status, by a small kernel enqueued here
// once every argument has been accepted.  0 = enqueued, -1 = refused (nothing
// enqueued).
static int enqueue_reduce_teams(int dtype, int op, const rocshmem_amd_team_t *teams, int n_teams,
                                void *dest, const void *source, int nreduce, int chunk_elems,
                                int wg_size, int iters, int *d_status, bool clear_status,
                                hipStream_t s) {
  if (!teams || n_teams < 1 || n_teams > kMaxTeamsPerLaunch || !valid_launch(1, wg_size) ||
      nreduce < 0 || chunk_elems < 0 || iters < 1)
    return -1;
  TeamView first;
  if (!view_team(teams[0], &first)) return -1;
  WgTeamsArgs a;
  for (int t = 0; t < n_teams; ++t) {
    TeamView v;
    if (!view_team(teams[t], &v)) return -1;
    const detail::TeamInfo &x = v.host->wrt_world, &y = first.host->wrt_world;
    if (x.pe_start != y.pe_start || x.stride != y.stride || x.size != y.size) return -1;
    for (int u = 0; u < t; ++u)
      if (a.rows[u] == v.row) return -1;  // one work-group per team member
    a.rows[t] = v.row;
  }
  const size_t es = dtype_size(dtype);
  {
    const size_t bytes = static_cast<size_t>(nreduce) * es;
    const int me = runtime::rt().me();
    if (!es || !sym_ok_on(dest, bytes, me) || !sym_ok_on(source, bytes, me)) return -1;
  }
  auto &r = runtime::rt();
  a.ctx_row = r.driver_ctx_row();
  a.dest0 = on_pe0(dest);
  a.src0 = on_pe0(source);
  a.pe_stride = r.pe_stride;
  a.pe_start = first.host->wrt_world.pe_start;
  a.stride = first.host->wrt_world.stride;
  a.nelems = nreduce;
  // Equal slices, a whole number of 16-byte vectors each: one per team, or of
  // the size the caller asks for and then dealt out to the teams in turn.
  const int per_vec = static_cast<int>(16 / es);
  long slice = chunk_elems ? chunk_elems : (static_cast<long>(nreduce) + n_teams - 1) / n_teams;
  slice = (slice + per_vec - 1) / per_vec * per_vec;
  if (slice > nreduce) slice = (static_cast<long>(nreduce) + per_vec - 1) / per_vec * per_vec;
  a.slice_elems = static_cast<int>(slice > 0 ? slice : per_vec);
  a.iters = iters;
  a.status = d_status;
  const dim3 grid(first.host->num_pes, n_teams), block(wg_size);
  bool launched = false;
  const bool ok = for_dtype_op(dtype, op, [&](auto *tag, auto opc) {
    using T = typename std::remove_pointer<decltype(tag)>::type;
    if (!grid_fits(wg_reduce_teams_kernel<T, decltype(opc)::value>,
                   static_cast<long>(grid.x) * grid.y, wg_size))
      return;
    // Everything has been checked: only now is anything put on the stream.
    if (clear_status) hipLaunchKernelGGL(clear_words_kernel, dim3(1), dim3(256), 0, s, d_status, n_teams);
    hipLaunchKernelGGL((wg_reduce_teams_kernel<T, decltype(opc)::value>), grid, block, 0, s, a);
    launched = true;
  });
  if (!ok || !launched) return -1;
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

int rocshmem_amd_wg_reduce_teams(int dtype, int op, const rocshmem_amd_team_t *teams, int n_teams,
                                 void *dest, const void *source, int nreduce, int chunk_elems,
                                 int wg_size, int iters, rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  if (n_teams < 1 || n_teams > kMaxTeamsPerLaunch) return -1;
  hipStream_t s = as_stream(stream);
  int *d_status;
  DRV_CHECK_HIP(hipMalloc(&d_status, sizeof(int) * n_teams));
  DRV_CHECK_HIP(hipMemsetAsync(d_status, 0, sizeof(int) * n_teams, s));
  int status = enqueue_reduce_teams(dtype, op, teams, n_teams, dest, source, nreduce, chunk_elems,
                                    wg_size, iters, d_status, false, s);
  if (status == 0) {
    int seen[kMaxTeamsPerLaunch];
    DRV_CHECK_HIP(hipStreamSynchronize(s));
    DRV_CHECK_HIP(hipMemcpy(seen, d_status, sizeof(int) * n_teams, hipMemcpyDeviceToHost));
    for (int t = 0; t < n_teams; ++t) status = seen[t] > status ? seen[t] : status;
  }
  DRV_CHECK_HIP(hipFree(d_status));
  return status;
}

// The address of `scratch` on the current device, looked up once per device.
static int *static_status_words() {
  constexpr int kMaxDevices = 64;
  static std::mutex lock;
  static int *words[kMaxDevices] = {};
  int dev = 0;
  DRV_CHECK_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> guard(lock);
  if (!words[dev]) {
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      fprintf(stderr, "rocshmem: hipGetSymbolAddress(scratch) failed on device %d: %s\n", dev,
              hipGetErrorString(e));
      return nullptr;
    }
    words[dev] = static_cast<int *>(p);
  }
  return words[dev];
}

int rocshmem_amd_wg_reduce_teams_static(int dtype, int op, const rocshmem_amd_team_t *teams,
                                        int n_teams, void *dest, const void *source, int nreduce,
                                        int chunk_elems, int wg_size, int iters,
                                        rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  if (n_teams > kStaticStatusWords) {
    fprintf(stderr,
            "rocshmem: rocshmem_amd_wg_reduce_teams_static takes at most %d teams per call "
            "(its status words are a fixed array), %d asked for\n",
            kStaticStatusWords, n_teams);
    return -1;
  }
  if (n_teams < 1) return -1;
  int *words = static_status_words();
  if (!words) return -1;
  hipStream_t s = as_stream(stream);
  // The array keeps what the last call left: the words this call uses are
  // cleared on the stream, after the arguments have been checked.
  int status = enqueue_reduce_teams(dtype, op, teams, n_teams, dest, source, nreduce, chunk_elems,
                                    wg_size, iters, words, true, s);
  if (status == 0) {
    int seen[kStaticStatusWords];
    DRV_CHECK_HIP(hipStreamSynchronize(s));
    DRV_CHECK_HIP(hipMemcpy(seen, words, sizeof(int) * n_teams, hipMemcpyDeviceToHost));
    for (int t = 0; t < n_teams; ++t) status = seen[t] > status ? seen[t] : status;
  }
  return status;
}

int rocshmem_amd_fold_shares(void *dest, const void *source, int nreduce,
                             const int *lanes_per_member, rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  auto &r = runtime::rt();
  if (!r.live || !lanes_per_member || nreduce < 0 || r.npes > detail::SyncPad::kMaxPes) return -1;
  const size_t bytes = static_cast<size_t>(nreduce) * sizeof(int);
  if (!sym_ok_on(dest, bytes, 0) || !sym_ok_on(source, bytes, 0)) return -1;
  FoldSharesArgs a;
  a.dst0 = static_cast<int *>(dest);
  a.src0 = static_cast<const int *>(source);
  a.hop = static_cast<int64_t>(r.pe_stride);
  a.np = r.npes;
  a.nelems = nreduce;
  int widest = 0;
  for (int k = 0; k < r.npes; ++k) {
    if (lanes_per_member[k] < 1 || lanes_per_member[k] > 1024) return -1;
    a.lanes[k] = lanes_per_member[k];
    widest = lanes_per_member[k] > widest ? lanes_per_member[k] : widest;
  }
  hipLaunchKernelGGL(fold_shares_kernel, dim3(r.npes), dim3(widest), 0, as_stream(stream), a);
  DRV_CHECK_HIP(hipGetLastError());
  return 0;
}

int rocshmem_amd_wg_alltoall(int elem_size, rocshmem_amd_team_t team, void *dest,
                             const void *source, int nelems, int wg_size,
                             rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  return wg_move_common<MOVE_ALLTOALL>(elem_size, team, dest, source, nelems, 0, wg_size,
                                       as_stream(stream));
}
int rocshmem_amd_wg_broadcast(int elem_size, rocshmem_amd_team_t team, void *dest,
                              const void *source, int nelems, int pe_root, int wg_size,
                              rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  return wg_move_common<MOVE_BROADCAST>(elem_size, team, dest, source, nelems, pe_root,
                                        wg_size, as_stream(stream));
}
int rocshmem_amd_wg_fcollect(int elem_size, rocshmem_amd_team_t team, void *dest,
                             const void *source, int nelems, int wg_size,
                             rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  return wg_move_common<MOVE_FCOLLECT>(elem_size, team, dest, source, nelems, 0, wg_size,
                                       as_stream(stream));
}

int rocshmem_amd_wg_sync(int sync_fn, rocshmem_amd_team_t team, uint64_t *scratch, int rounds,
                         int wg_size, rocshmem_amd_stream_t stream) {
  DRV_ONE_PROCESS_ONLY();
  auto &r = runtime::rt();
  if (!r.live || rounds < 0 || !valid_launch(1, wg_size) || !sym_ok_on(scratch, 8, r.me())) return -1;
  if (sync_fn < ROCSHMEM_AMD_BARRIER_ALL || sync_fn > ROCSHMEM_AMD_TEAM_SYNC) return -1;
  TeamView v;
  if (sync_fn == ROCSHMEM_AMD_TEAM_SYNC) {
    if (!view_team(team, &v)) return -1;
  } else {
    if (!view_team(r.team_handle(0, r.me()), &v)) return -1;
  }
  if (!grid_fits(wg_sync_kernel, v.host->num_pes, wg_size)) return -1;
  int *d_err;
  DRV_CHECK_HIP(hipMalloc(&d_err, sizeof(int)));
  DRV_CHECK_HIP(hipMemset(d_err, 0, sizeof(int)));
  SyncArgs a;
  a.team_row = v.row;
  a.ctx_row = r.driver_ctx_row();
  a.scratch0 = reinterpret_cast<uint64_t *>(on_pe0(scratch));
  a.pe_stride = r.pe_stride;
  a.pe_start = v.host->wrt_world.pe_start;
  a.stride = v.host->wrt_world.stride;
  a.size = v.host->num_pes;
  a.fn = sync_fn;
  a.rounds = rounds;
  a.errors = d_err;
  hipStream_t s = as_stream(stream);
  hipLaunchKernelGGL(wg_sync_kernel, dim3(a.size), dim3(wg_size), 0, s, a);
  DRV_CHECK_HIP(hipGetLastError());
  DRV_CHECK_HIP(hipStreamSynchronize(s));
  int err = 0;
  DRV_CHECK_HIP(hipMemcpy(&err, d_err, sizeof(int), hipMemcpyDeviceToHost));
  DRV_CHECK_HIP(hipFree(d_err));
  return err;
}

int rocshmem_amd_to_all(int dtype, int op, void *dest, const void *source, int nreduce,
                        int PE_start, int logPE_stride, int PE_size,
                        rocshmem_amd_stream_t stream) {
  auto &r = runtime::rt();
  if (!r.live || PE_start < 0 || logPE_stride < 0 || logPE_stride > 30 || PE_size < 1) return -1;
  const int stride = 1 << logPE_stride;
  if (PE_start + static_cast<long>(stride) * (PE_size - 1) >= r.npes) return -1;
  if (nreduce < 0) return -1;
  if (r.nprocs) return procs_reduce(dtype, op, dest, source, nreduce, PE_start, stride, PE_size,
                                    as_stream(stream));
  const size_t bytes = static_cast<size_t>(nreduce) * dtype_size(dtype);
  if (!sym_ok_on(dest, bytes, PE_start) || !sym_ok_on(source, bytes, PE_start)) return -1;
  return grid_reduce_common(dtype, op, dest, source, static_cast<int64_t>(stride) * r.pe_stride,
                            PE_size, nreduce, as_stream(stream));
}

int rocshmem_amd_reduce(int dtype, int op, rocshmem_amd_team_t team, void *dest,
                        const void *source, int nreduce, rocshmem_amd_stream_t stream) {
  TeamView v;
  if (!view_team(team, &v) || nreduce < 0) return -1;
  auto &r = runtime::rt();
  if (r.nprocs)
    return procs_reduce(dtype, op, dest, source, nreduce, v.host->wrt_world.pe_start,
                        v.host->wrt_world.stride, v.host->num_pes, as_stream(stream));
  const size_t bytes = static_cast<size_t>(nreduce) * dtype_size(dtype);
  if (!sym_ok_on(dest, bytes, r.me()) || !sym_ok_on(source, bytes, r.me())) return -1;
  const int64_t first = static_cast<int64_t>(v.host->wrt_world.pe_start) * r.pe_stride;
  const int64_t hop = static_cast<int64_t>(v.host->wrt_world.stride) * r.pe_stride;
  return grid_reduce_common(dtype, op, on_pe0(dest) + first, on_pe0(source) + first, hop,
                            v.host->num_pes, nreduce, as_stream(stream));
}

int rocshmem_amd_alltoallmem(rocshmem_amd_team_t team, void *dest, const void *source,
                             size_t nbytes, rocshmem_amd_stream_t stream) {
  return grid_move_common<MOVE_ALLTOALL>(team, dest, source, nbytes, 0, as_stream(stream));
}
int rocshmem_amd_broadcastmem(rocshmem_amd_team_t team, void *dest, const void *source,
                              size_t nbytes, int pe_root, rocshmem_amd_stream_t stream) {
  return grid_move_common<MOVE_BROADCAST>(team, dest, source, nbytes, pe_root, as_stream(stream));
}
int rocshmem_amd_broadcast_active_set(void *dest, const void *source, size_t nbytes, int pe_root,
                                      int PE_start, int logPE_stride, int PE_size,
                                      rocshmem_amd_stream_t stream) {
  auto &r = runtime::rt();
  if (!r.live || PE_start < 0 || logPE_stride < 0 || logPE_stride > 30 || PE_size < 1) return -1;
  const int stride = 1 << logPE_stride;
  if (PE_start + static_cast<long>(stride) * (PE_size - 1) >= r.npes) return -1;
  if (pe_root < 0 || pe_root >= PE_size) return -1;
  if (r.nprocs)
    return procs_move<MOVE_BROADCAST>(dest, source, nbytes, pe_root, PE_start, stride, PE_size,
                                      as_stream(stream));
  if (!sym_ok_on(dest, nbytes, PE_start) || !sym_ok_on(source, nbytes, PE_start)) return -1;
  launch_grid_move<MOVE_BROADCAST>(static_cast<char *>(dest), static_cast<const char *>(source),
                                   static_cast<int64_t>(stride) * r.pe_stride, PE_size, pe_root,
                                   nbytes, as_stream(stream));
  return 0;
}
int rocshmem_amd_fcollectmem(rocshmem_amd_team_t team, void *dest, const void *source,
                             size_t nbytes, rocshmem_amd_stream_t stream) {
  return grid_move_common<MOVE_FCOLLECT>(team, dest, source, nbytes, 0, as_stream(stream));
}

}  // extern "C"
