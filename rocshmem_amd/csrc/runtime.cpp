// Host runtime: symmetric heap, PE slices, teams, context pools and the
// work/sync area, for P processing elements hosted by one process on one GPU.
//
// Plays the part of the reference's rocshmem_init -> IPCBackend bring-up
// (src/rocshmem.cpp:73-140, src/ipc/backend_ipc.cpp:56-165,274-490) without
// MPI or HIP IPC: there is one heap allocation of P slices at a fixed stride,
// so the table of peer base addresses collapses to (base, stride).
#include "runtime.hpp"
#include "proc_group.hpp"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <atomic>
#include <mutex>
#include <thread>
#include <vector>

#include "rocshmem/rocshmem.hpp"

namespace rocshmem {

rocshmem_team_t ROCSHMEM_TEAM_WORLD = ROCSHMEM_TEAM_INVALID;

namespace runtime {

thread_local int tl_pe = -1;

#define RT_CHECK_HIP(expr)                                                        \
  do {                                                                            \
    hipError_t rt_err_ = (expr);                                                  \
    if (rt_err_ != hipSuccess) {                                                  \
      fprintf(stderr, "rocshmem: HIP error %d (%s) at %s:%d\n", (int)rt_err_,     \
              hipGetErrorString(rt_err_), __FILE__, __LINE__);                    \
      exit(EXIT_FAILURE);                                                         \
    }                                                                             \
  } while (0)

namespace {

std::vector<detail::StateUploader> &uploaders() {
  static std::vector<detail::StateUploader> v;
  return v;
}
// Uploaders registered while the runtime is live (a library with device code
// loaded after rocshmem_init): their first upload waits until the next call
// into the runtime, because registration runs among the static initialisers of
// the library being loaded, possibly before HIP has registered that library's
// device code, when a copy to its symbols would fail.
std::mutex g_uploader_lock;
std::vector<detail::StateUploader> &late_uploaders() {
  static std::vector<detail::StateUploader> v;
  return v;
}
std::atomic<bool> g_late_uploaders{false};

Runtime g_rt;
int g_requested_npes = 0;
bool g_per_thread_default_stream = false;

size_t env_size(const char *name, size_t fallback) {
  const char *v = getenv(name);
  if (!v || !*v) return fallback;
  char *end = nullptr;
  unsigned long long x = strtoull(v, &end, 10);
  if (end == v) return fallback;
  return static_cast<size_t>(x);
}

size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

int ilog2(int x) {
  int l = 0;
  while ((1 << (l + 1)) <= x) ++l;
  return l;
}

}  // namespace

Runtime &rt() {
  if (g_late_uploaders.load(std::memory_order_acquire)) {
    std::vector<detail::StateUploader> todo;
    {
      std::lock_guard<std::mutex> guard(g_uploader_lock);
      todo.swap(late_uploaders());
      g_late_uploaders.store(false, std::memory_order_release);
    }
    if (g_rt.live && !todo.empty()) {
      for (auto fn : todo) fn(&g_rt.state);
      RT_CHECK_HIP(hipDeviceSynchronize());
    }
  }
  return g_rt;
}

// ---- one thread per PE -------------------------------------------------------
namespace {
struct MeetingPoint {
  std::mutex m;
  std::condition_variable cv;
  int arrived = 0;
  uint64_t round = 0;
  uint64_t result = 0;
};
struct PeThreads {
  int npes = 0;
  std::mutex m;
  std::map<uint64_t, MeetingPoint> points;  // node-based: references stay valid
  MeetingPoint &at(int start, int stride, int size) {
    const uint64_t key = (static_cast<uint64_t>(start) << 42) |
                         (static_cast<uint64_t>(stride) << 21) | static_cast<uint64_t>(size);
    std::lock_guard<std::mutex> g(m);
    return points[key];
  }
};
PeThreads g_threads;
}  // namespace

int pe_threads_count() { return g_threads.npes; }
void pe_threads_start(int npes) { g_threads.npes = npes; }

// ROCSHMEM_EMU_TRACE=1: one line on stderr per arrival at a meeting point.
bool tracing() {
  static const bool on = [] {
    const char *v = getenv("ROCSHMEM_EMU_TRACE");
    return v && atoi(v) != 0;
  }();
  return on;
}

// ---- hardware queues under PE threads ------------------------------------------
// HIP multiplexes streams onto GPU_MAX_HW_QUEUES hardware queues (4 unless the
// variable says otherwise).  Kernels of different PE threads wait for each
// other inside the GPU; two such kernels in one hardware queue run one after
// the other, so the first can wait for ever for the second.  Every stream a PE
// thread launches on therefore needs a queue of its own, and one more is kept
// for the library's own streams and the null stream.
size_t hw_queue_limit() { return env_size("GPU_MAX_HW_QUEUES", 4); }
bool hw_queues_suffice(size_t pe_streams, size_t hw_queues) {
  return pe_streams + 1 <= hw_queues;
}
[[noreturn]] void refuse_for_queues(size_t pe_streams) {
  fprintf(stderr,
          "rocshmem: %zu streams of PE threads (plus one for the library) need %zu hardware "
          "queues but GPU_MAX_HW_QUEUES=%zu: kernels of different PEs that wait for each other "
          "would share a queue and never finish.  Set GPU_MAX_HW_QUEUES to at least the number "
          "of streams in use (PEs x streams per PE + 1).  Nothing was launched.\n",
          pe_streams, pe_streams + 1, hw_queue_limit());
  fflush(nullptr);
  _Exit(EXIT_FAILURE);
}

bool pe_threads_enter(int start, int stride, int size, uint64_t *result) {
  if (tl_pe < 0 || g_threads.npes == 0 || size <= 1) return true;
  MeetingPoint &p = g_threads.at(start, stride, size);
  std::unique_lock<std::mutex> lk(p.m);
  if (tracing())
    fprintf(stderr, "rocshmem: PE %d arrives at (%d,%d,%d) round %llu as %d of %d\n", tl_pe, start,
            stride, size, static_cast<unsigned long long>(p.round), p.arrived + 1, size);
  if (++p.arrived == size) return true;  // the last to arrive does the work (lock released here)
  const uint64_t round = p.round;
  p.cv.wait(lk, [&] { return p.round != round; });
  if (result) *result = p.result;
  return false;
}

void pe_threads_leave(int start, int stride, int size, uint64_t result) {
  if (tl_pe < 0 || g_threads.npes == 0 || size <= 1) return;
  MeetingPoint &p = g_threads.at(start, stride, size);
  std::lock_guard<std::mutex> lk(p.m);
  p.arrived = 0;
  p.result = result;
  ++p.round;
  p.cv.notify_all();
}

void Runtime::push_state() {
  for (auto fn : uploaders()) fn(&state);
  RT_CHECK_HIP(hipDeviceSynchronize());
}

size_t Runtime::ws_bytes_per_pe() const {
  // [world pad][per team: SYNC_KINDS pads + pWrk]
  const size_t per_team = sizeof(detail::SyncPad) * detail::SYNC_KINDS +
                          ROCSHMEM_REDUCE_MIN_WRKDATA_SIZE * sizeof(double);
  return round_up(sizeof(detail::SyncPad) + per_team * max_teams, 4096);
}

char *Runtime::ws_of(int pe) const {
  return nprocs ? peer_base[pe] + slice_bytes : d_ws + static_cast<size_t>(pe) * ws_stride;
}

detail::SyncPad *Runtime::team_pads(int pool_index, int pe) const {
  const size_t per_team = sizeof(detail::SyncPad) * detail::SYNC_KINDS +
                          ROCSHMEM_REDUCE_MIN_WRKDATA_SIZE * sizeof(double);
  char *p = ws_of(pe) + sizeof(detail::SyncPad) + per_team * pool_index;
  return reinterpret_cast<detail::SyncPad *>(p);
}

void Runtime::write_team(int pool_index, int pe, const detail::TeamInfo &world,
                         const detail::TeamInfo &parent, int my_pe_in_team) {
  detail::Team t{};
  t.wrt_world = world;
  t.wrt_parent = parent;
  t.my_pe = my_pe_in_team;
  t.my_pe_in_world = pe;
  t.num_pes = world.size;
  t.world_size = npes;
  t.pool_index = pool_index;
  t.sync = team_pads(pool_index, pe);
  t.pWrk = reinterpret_cast<char *>(t.sync) + sizeof(detail::SyncPad) * detail::SYNC_KINDS;
  h_teams[static_cast<size_t>(pool_index) * npes + pe] = t;
  RT_CHECK_HIP(hipMemcpy(d_teams + static_cast<size_t>(pool_index) * npes + pe, &t,
                         sizeof(t), hipMemcpyHostToDevice));
}

// ---- the device allocation behind the symmetric heap ---------------------------
// The heap is UNCACHED device memory (hipDeviceMallocUncached).  That is this
// library's choice, not the reference's: built for the IPC backend with
// USE_COHERENT_HEAP, the reference takes HeapMemory<HIPAllocator>, plain
// hipMalloc (src/memory/heap_type.hpp:41-51); its uncached allocator
// (src/memory/hip_allocator.hpp:58-65) serves the other configurations.
// What the flag changes on MI355X, measured: an agent-scope release is an L2
// write-back (buffer_wbl2), which costs about 41 ns device-wide while a copy
// runs on ordinary cached memory and 4-6 ns on memory allocated uncached
// (256 MiB copied in 16 KiB tiles by 1024 work-groups of 256 with one release
// per tile: 760 us against 156 us, 87 us without releases; the copy itself runs
// at the same rate on either).  Stores to the heap never sit dirty, plain ones
// included.  Reads are cached all the same: re-reading a tile hits the L2 as
// often on either kind of heap (67 % in a probe that reads each 64 KiB tile
// four times), so a consumer of symmetric data loses nothing, and a reader
// still has to invalidate before it trusts a line (waits, barriers and thread-
// or wavefront-level gets do).  ROCSHMEM_EMU_HEAP_CACHED=1 selects plain
// hipMalloc / hipFree.
//
// Uncached memory is never given back while the process lives: on this class
// of machines memory allocated after such a release has shown wrong values.
// rocshmem_finalize marks the block idle, and a later rocshmem_init reuses
// the smallest idle block that is large enough before it allocates another.
// What the process holds that way is bounded by ROCSHMEM_EMU_HEAP_HELD_LIMIT
// (bytes; default: the device memory), reported by heap_held() and, with
// ROCSHMEM_EMU_VERBOSE=1, logged at every reuse and every new block.
namespace {
struct HeapBlock {
  char *base;
  size_t bytes;
  bool in_use;
};
std::mutex g_heap_lock;
std::vector<HeapBlock> g_heap_blocks;  // uncached blocks of this process, never freed

bool heap_cached_mode() { return env_size("ROCSHMEM_EMU_HEAP_CACHED", 0) != 0; }
bool verbose() { return env_size("ROCSHMEM_EMU_VERBOSE", 0) != 0; }

void held_unlocked(size_t *total, size_t *idle) {
  *total = *idle = 0;
  for (const HeapBlock &b : g_heap_blocks) {
    *total += b.bytes;
    if (!b.in_use) *idle += b.bytes;
  }
}

// An idle uncached block of at least `bytes`, or nullptr.
char *reuse_heap_block(size_t bytes, size_t *block_bytes) {
  std::lock_guard<std::mutex> guard(g_heap_lock);
  HeapBlock *best = nullptr;
  for (HeapBlock &b : g_heap_blocks)
    if (!b.in_use && b.bytes >= bytes && (!best || b.bytes < best->bytes)) best = &b;
  if (!best) return nullptr;
  best->in_use = true;
  *block_bytes = best->bytes;
  if (verbose())
    fprintf(stderr, "rocshmem: heap of %zu B reuses an idle uncached block of %zu B\n", bytes,
            best->bytes);
  return best->base;
}

hipError_t new_heap_block(char **base, size_t bytes) {
  if (heap_cached_mode()) return hipMalloc(reinterpret_cast<void **>(base), bytes);
  {
    std::lock_guard<std::mutex> guard(g_heap_lock);
    size_t total = 0, idle = 0, free_b = 0, device_b = 0;
    held_unlocked(&total, &idle);
    (void)hipMemGetInfo(&free_b, &device_b);
    const size_t limit = env_size("ROCSHMEM_EMU_HEAP_HELD_LIMIT", device_b);
    if (total + bytes > limit) {
      fprintf(stderr,
              "rocshmem: a new uncached heap block of %zu B is refused: this process already holds "
              "%zu B of uncached heap blocks (%zu B of them idle, none large enough; they are kept "
              "until the process ends), and the limit is %zu B (ROCSHMEM_EMU_HEAP_HELD_LIMIT)\n",
              bytes, total, idle, limit);
      return hipErrorOutOfMemory;
    }
  }
  const hipError_t e =
      hipExtMallocWithFlags(reinterpret_cast<void **>(base), bytes, hipDeviceMallocUncached);
  if (e == hipSuccess) {
    std::lock_guard<std::mutex> guard(g_heap_lock);
    g_heap_blocks.push_back(HeapBlock{*base, bytes, true});
    if (verbose()) {
      size_t total = 0, idle = 0;
      held_unlocked(&total, &idle);
      fprintf(stderr,
              "rocshmem: new uncached heap block of %zu B; the process now holds %zu B in %zu "
              "blocks (%zu B idle)\n",
              bytes, total, g_heap_blocks.size(), idle);
    }
  }
  return e;
}

void release_heap_block(char *base) {
  {
    std::lock_guard<std::mutex> guard(g_heap_lock);
    for (HeapBlock &b : g_heap_blocks)
      if (b.base == base) {
        b.in_use = false;
        return;
      }
  }
  RT_CHECK_HIP(hipFree(base));  // a cached-mode block
}
}  // namespace

void heap_held(size_t *total, size_t *idle) {
  std::lock_guard<std::mutex> guard(g_heap_lock);
  held_unlocked(total, idle);
}

// Default bound on the polls of one device wait in a process that is one PE of
// a job (a poll of a word in the heap takes 0.5-1 us on MI355X).
constexpr uint64_t kProcessSpinLimit = 400000000ull;

int Runtime::init(int want_npes, size_t want_heap) {
  if (live) return 0;
  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) {
    fprintf(stderr, "rocshmem: no GPU available\n");
    abort();
  }
  // Started as one PE of a job of processes?  Then the job says how many PEs.
  if (procs().attach_from_env()) want_npes = procs().nprocs();
  npes = want_npes > 0 ? want_npes
                       : (g_requested_npes > 0
                              ? g_requested_npes
                              : static_cast<int>(env_size("ROCSHMEM_EMU_NPES", 1)));
  if (npes < 1 || npes > detail::SyncPad::kMaxPes) {
    fprintf(stderr, "rocshmem: number of PEs must be in [1, %d]\n", detail::SyncPad::kMaxPes);
    abort();
  }
  heap_size = want_heap ? want_heap : env_size("ROCSHMEM_HEAP_SIZE", size_t{1} << 30);
  max_ctxs = static_cast<int>(env_size("ROCSHMEM_MAX_NUM_CONTEXTS", 1024));
  if (max_ctxs > detail::CtxPool::kMaxWords * 64) max_ctxs = detail::CtxPool::kMaxWords * 64;
  max_teams = static_cast<int>(env_size("ROCSHMEM_MAX_NUM_TEAMS", 40));
  if (max_teams < 1) max_teams = 1;
  size_t alloc_bytes = 0;
  bool anchored = false;
  ws_stride = ws_bytes_per_pe();
  acting_pe = 0;
  driver_ctx_options = 0;
  heap_base = nullptr;
  peer_base.clear();
  nprocs = 0;
  if (procs().active()) {
    // One process per PE: this process allocates its own slice, publishes its
    // IPC handle, and maps the slices of the others wherever HIP puts them
    // (the reference does the same with MPI_Allgather of the handles,
    // src/ipc_policy.cpp:34-118).  Allocations shared this way stay below
    // 2 GiB: opening larger ones has not returned on this class of machines.
    nprocs = procs().nprocs();
    acting_pe = procs().rank();
    const size_t two_mib = size_t{2} << 20;
    pe_stride = 0;
    slice_bytes = round_up(heap_size, two_mib);
    // The shared block: the slice, then this PE's work/sync area, so that the
    // table that finds a peer's slice also finds its barrier and reduce pads.
    const size_t block_bytes = slice_bytes + ws_stride;
    if (block_bytes >= (size_t{2} << 30)) {
      fprintf(stderr,
              "rocshmem: with one process per PE the heap of a PE must stay below 2 GiB "
              "(ROCSHMEM_HEAP_SIZE=%zu asked for)\n", heap_size);
      fflush(nullptr);
      _Exit(EXIT_FAILURE);
    }
    // The slice and the mappings of the other PEs' slices live until the
    // process ends: a later rocshmem_init of the same job finds them again
    // (same size, same handles), so nothing shared is ever unmapped or freed
    // while another process may hold it, and no uncached block is given back.
    struct Kept {
      char *own = nullptr;
      size_t bytes = 0;
      bool cached = false;
      std::vector<hipIpcMemHandle_t> handle;
      std::vector<char *> mapped;
    };
    static Kept kept;
    if (kept.own && (kept.bytes != block_bytes || kept.cached != heap_cached_mode())) {
      fprintf(stderr, "rocshmem: a process that is one PE of a job keeps the heap size and kind of "
                      "its first rocshmem_init (%zu bytes)\n", kept.bytes);
      fflush(nullptr);
      _Exit(EXIT_FAILURE);
    }
    if (!kept.own) {
      const hipError_t e = heap_cached_mode()
                               ? hipMalloc(reinterpret_cast<void **>(&kept.own), block_bytes)
                               : hipExtMallocWithFlags(reinterpret_cast<void **>(&kept.own), block_bytes,
                                                       hipDeviceMallocUncached);
      if (e != hipSuccess || !kept.own) {
        fprintf(stderr, "rocshmem: PE %d cannot allocate %zu bytes for its heap: %s\n", acting_pe,
                block_bytes, hipGetErrorString(e));
        fflush(nullptr);
        _Exit(EXIT_FAILURE);
      }
      kept.bytes = block_bytes;
      kept.cached = heap_cached_mode();
      kept.handle.resize(npes);
      kept.mapped.assign(npes, nullptr);
      RT_CHECK_HIP(hipIpcGetMemHandle(&kept.handle[acting_pe], kept.own));
    }
    char *own = kept.own;
    RT_CHECK_HIP(hipMemset(own, 0, block_bytes));
    RT_CHECK_HIP(hipDeviceSynchronize());
    // What every PE tells the others: the handle of its block and how the
    // block is laid out.  The layouts must agree — a peer's sync pads are
    // found at the same offset as one's own — so a job whose processes were
    // given different heap sizes or team counts ends here, with a message,
    // and not in a kernel that writes past a smaller peer block.
    struct Announce {
      hipIpcMemHandle_t handle;
      uint64_t slice_bytes, ws_bytes;
      uint32_t npes, cached;
    };
    static_assert(sizeof(Announce) <= kBlobBytes, "announcement larger than a publish area");
    Announce mine{};
    mine.handle = kept.handle[acting_pe];
    mine.slice_bytes = slice_bytes;
    mine.ws_bytes = ws_stride;
    mine.npes = static_cast<uint32_t>(npes);
    mine.cached = heap_cached_mode() ? 1u : 0u;
    procs().publish(&mine, sizeof(mine));
    if (procs().barrier_world() != 0) _Exit(EXIT_FAILURE);
    peer_base.assign(npes, nullptr);
    peer_base[acting_pe] = own;
    for (int p = 0; p < npes; ++p) {
      if (p == acting_pe) continue;
      Announce theirs{};
      procs().fetch(p, &theirs, sizeof(theirs));
      if (theirs.slice_bytes != mine.slice_bytes || theirs.ws_bytes != mine.ws_bytes ||
          theirs.npes != mine.npes) {
        fprintf(stderr,
                "rocshmem: PE %d and PE %d disagree about the job: %u PEs, %llu + %llu bytes per PE here, "
                "%u PEs, %llu + %llu there (every process needs the same ROCSHMEM_HEAP_SIZE and "
                "ROCSHMEM_MAX_NUM_TEAMS)\n",
                acting_pe, p, mine.npes, static_cast<unsigned long long>(mine.slice_bytes),
                static_cast<unsigned long long>(mine.ws_bytes), theirs.npes,
                static_cast<unsigned long long>(theirs.slice_bytes),
                static_cast<unsigned long long>(theirs.ws_bytes));
        fflush(nullptr);
        procs().request_abort(EXIT_FAILURE);
        _Exit(EXIT_FAILURE);
      }
      if (!kept.mapped[p] || memcmp(&theirs.handle, &kept.handle[p], sizeof(theirs.handle)) != 0) {
        RT_CHECK_HIP(hipIpcOpenMemHandle(reinterpret_cast<void **>(&kept.mapped[p]), theirs.handle,
                                         hipIpcMemLazyEnablePeerAccess));
        kept.handle[p] = theirs.handle;
      }
      peer_base[p] = kept.mapped[p];
    }
    // Everybody has read everybody's handle before anybody publishes again.
    if (procs().barrier_world() != 0) _Exit(EXIT_FAILURE);
    heap_base = own;
    alloc_bytes = block_bytes;
  } else {
    // Slice placement.  Slices start on 2 MiB boundaries and sit `pe_stride`
    // apart inside ONE device allocation.  By default the allocation holds the
    // slices and nothing else: stride = heap size rounded up to 2 MiB.
    //
    // ROCSHMEM_EMU_SPREAD=1 trades device memory for bandwidth: the slices are
    // spread over about half of the device memory on a 4 GiB grid (16 GiB apart
    // for 8 PEs) and, when the GPU is otherwise empty, the block is placed by
    // allocating half of the memory plus 1 GiB.  On MI355X a kernel that writes
    // to all P slices at once (all-reduce, alltoall) then sustains about 10 %
    // more HBM bandwidth (measured: 6.45 instead of 5.7-5.9 TB/s for the P = 8
    // fp32 all-reduce) and is steadier from run to run.  That is a property of
    // hosting P PEs inside one memory; it is off unless asked for.
    // ROCSHMEM_EMU_PE_STRIDE=<bytes> sets the stride directly;
    // ROCSHMEM_EMU_HEAP_ANCHOR=0 keeps the spread but not the placement.
    const size_t two_mib = size_t{2} << 20;
    const size_t min_stride = round_up(heap_size, two_mib);
    const bool spread = env_size("ROCSHMEM_EMU_SPREAD", 0) != 0;
    size_t want = env_size("ROCSHMEM_EMU_PE_STRIDE", 0);
    size_t free_b = 0, total_b = 0;
    RT_CHECK_HIP(hipMemGetInfo(&free_b, &total_b));
    if (!want && spread) {
      const size_t budget = total_b / 2;
      const size_t grid = size_t{4} << 30;
      want = npes <= 2 ? size_t{16} << 30 : budget / npes;
      if (want >= grid) want = want / grid * grid;
      if (want * npes > budget) want = budget / npes;
    }
    pe_stride = std::max(min_stride, want / two_mib * two_mib);

    // Three tries: the spread block placed in the upper half of the memory, the
    // spread block, the packed slices.  Each first looks for an idle block from
    // an earlier rocshmem_init of this process.
    const size_t anchor = total_b / 2 + (size_t{1} << 30);
    const bool want_anchor = spread && env_size("ROCSHMEM_EMU_HEAP_ANCHOR", 1) != 0 &&
                             pe_stride * npes >= total_b / 4 && pe_stride * npes < anchor;
    auto try_block = [&](size_t bytes) {
      size_t had = 0;
      if (!heap_cached_mode() && (heap_base = reuse_heap_block(bytes, &had))) {
        alloc_bytes = had;
        return true;
      }
      if (new_heap_block(&heap_base, bytes) == hipSuccess) {
        alloc_bytes = bytes;
        return true;
      }
      (void)hipGetLastError();
      heap_base = nullptr;
      return false;
    };
    if (want_anchor) {
      size_t had = 0;
      if (!heap_cached_mode() && (heap_base = reuse_heap_block(anchor, &had))) {
        alloc_bytes = had;
        anchored = true;
      } else if (free_b > anchor + (size_t{16} << 30)) {
        anchored = try_block(anchor);
      }
    }
    if (!heap_base && !try_block(pe_stride * npes) && pe_stride != min_stride) {
      fprintf(stderr,
              "rocshmem: no room for %d slices %zu bytes apart; packing them (stride = heap size)\n",
              npes, pe_stride);
      pe_stride = min_stride;
      try_block(pe_stride * npes);
    }
    if (!heap_base) {
      fprintf(stderr, "rocshmem: cannot allocate %zu bytes of device memory for the symmetric heap\n",
              pe_stride * npes);
      exit(EXIT_FAILURE);
    }
  }
  if (!nprocs) slice_bytes = pe_stride;
  heap_alloc_bytes = alloc_bytes;
  heap_uncached = !heap_cached_mode();
  if (verbose())
    fprintf(stderr, "rocshmem: %d PEs, heap %zu B per PE, slices %zu B apart, %zu B allocated%s%s\n",
            npes, heap_size, pe_stride, alloc_bytes, anchored ? " (placed)" : "",
            heap_cached_mode() ? " (cached)" : " (uncached)");
  // With one process per PE every process runs the allocator for itself and
  // all must arrive at the same offsets: the same model base everywhere.
  allocator.reset(nprocs ? (uint64_t{1} << 40) : reinterpret_cast<uint64_t>(heap_base), heap_size);

  // Work/sync areas: one block for all PEs, or (one process per PE) the tail
  // of every PE's shared block, cleared with it above.
  d_ws = nullptr;
  if (!nprocs) {
    RT_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&d_ws), ws_stride * npes));
    RT_CHECK_HIP(hipMemset(d_ws, 0, ws_stride * npes));
  }

  // Teams: slot 0 is the world team.
  h_teams.assign(static_cast<size_t>(max_teams) * npes, detail::Team{});
  team_slot_used.assign(max_teams, false);
  RT_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&d_teams),
                         sizeof(detail::Team) * max_teams * npes));
  RT_CHECK_HIP(hipMemset(d_teams, 0, sizeof(detail::Team) * max_teams * npes));
  team_slot_used[0] = true;
  num_user_teams = 0;
  const detail::TeamInfo world{0, 1, npes, 0};
  for (int pe = 0; pe < npes; ++pe) write_team(0, pe, world, world, pe);

  // Where every PE's slice sits relative to PE q's, for every q: row q is the
  // table of q's contexts.  With all slices in one allocation device code
  // takes the product and never reads it (the rows hold the same products, so
  // that the pointer is never a dangling one); with one process per PE only
  // this PE's row means anything (the others stay zero: the own slice).
  {
    std::vector<int64_t> delta(static_cast<size_t>(npes) * npes, 0);
    for (int q = 0; q < npes; ++q)
      for (int p = 0; p < npes; ++p) {
        if (nprocs) {
          if (q == acting_pe) delta[static_cast<size_t>(q) * npes + p] = peer_base[p] - peer_base[q];
        } else {
          delta[static_cast<size_t>(q) * npes + p] =
              static_cast<int64_t>(p - q) * static_cast<int64_t>(pe_stride);
        }
      }
    RT_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&d_peer_delta), sizeof(int64_t) * delta.size()));
    RT_CHECK_HIP(hipMemcpy(d_peer_delta, delta.data(), sizeof(int64_t) * delta.size(),
                           hipMemcpyHostToDevice));
  }
  // Contexts: one default context and one pool per PE.
  auto fill_ctx = [&](detail::Context &c, int pe, int slot) {
    c.peer_delta = d_peer_delta + static_cast<size_t>(pe) * npes;
    c.heap_base = heap_base;
    c.pe_stride = pe_stride;  // 0 with one process per PE: device code takes the table
    c.ws_stride = ws_stride;
    c.my_pe = pe;
    c.num_pes = npes;
    c.tinfo = &d_teams[pe].wrt_world;
    c.world_sync = reinterpret_cast<detail::SyncPad *>(ws_of(pe));
    c.options = 0;
    c.pool_slot = slot;
  };
  // Rows [0, npes) are the default contexts; rows [npes, 2*npes) are the same
  // with ROCSHMEM_CTX_NOSTORE set, handed out by rocshmem_ctx_create.
  std::vector<detail::Context> ctxs(2 * static_cast<size_t>(npes));
  for (int pe = 0; pe < npes; ++pe) {
    fill_ctx(ctxs[pe], pe, -1);
    fill_ctx(ctxs[npes + pe], pe, -1);
    ctxs[npes + pe].options |= static_cast<unsigned>(ROCSHMEM_CTX_NOSTORE);
  }
  RT_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&d_default_ctx),
                         sizeof(detail::Context) * ctxs.size()));
  RT_CHECK_HIP(hipMemcpy(d_default_ctx, ctxs.data(), sizeof(detail::Context) * ctxs.size(),
                         hipMemcpyHostToDevice));

  RT_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&d_ctx_slots),
                         sizeof(detail::Context) * 2 * max_ctxs * npes));
  RT_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&d_pools), sizeof(detail::CtxPool) * npes));
  // Two objects per pool slot: [0, max_ctxs) without an option, [max_ctxs,
  // 2 * max_ctxs) with ROCSHMEM_CTX_NOSTORE; kernels only read them.
  std::vector<detail::Context> slots(static_cast<size_t>(max_ctxs) * 2 * npes);
  std::vector<detail::CtxPool> pools(npes);
  for (int pe = 0; pe < npes; ++pe) {
    detail::Context *row = slots.data() + static_cast<size_t>(pe) * 2 * max_ctxs;
    for (int s = 0; s < max_ctxs; ++s) {
      fill_ctx(row[s], pe, s);
      fill_ctx(row[max_ctxs + s], pe, s);
      row[max_ctxs + s].options |= static_cast<unsigned>(ROCSHMEM_CTX_NOSTORE);
    }
    detail::CtxPool &p = pools[pe];
    memset(&p, 0, sizeof(p));
    for (int s = 0; s < max_ctxs; ++s) p.free_mask[s >> 6] |= 1ull << (s & 63);
    p.capacity = max_ctxs;
    p.slots = d_ctx_slots + static_cast<size_t>(pe) * 2 * max_ctxs;
  }
  RT_CHECK_HIP(hipMemcpy(d_ctx_slots, slots.data(), sizeof(detail::Context) * slots.size(),
                         hipMemcpyHostToDevice));
  RT_CHECK_HIP(hipMemcpy(d_pools, pools.data(), sizeof(detail::CtxPool) * npes,
                         hipMemcpyHostToDevice));

  // Queue -> PE table; no queue is bound yet (an id no queue has).
  {
    std::vector<detail::QueueBinding> none(detail::kQueueTableSize,
                                           detail::QueueBinding{~0ull, 0, 0});
    RT_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&d_queue_table),
                           sizeof(detail::QueueBinding) * none.size()));
    RT_CHECK_HIP(hipMemcpy(d_queue_table, none.data(), sizeof(detail::QueueBinding) * none.size(),
                           hipMemcpyHostToDevice));
  }
  // Pinned words the stream bindings report through, allocated here because a
  // pinned allocation or release later on may wait for the whole device, and by
  // then another PE's kernel may be running and waiting for this PE.
  RT_CHECK_HIP(hipHostMalloc(reinterpret_cast<void **>(&h_bind_problem),
                             sizeof(int) * detail::kQueueTableSize, hipHostMallocDefault));
  memset(h_bind_problem, 0, sizeof(int) * detail::kQueueTableSize);
  state.queue_table = d_queue_table;
  state.heap_base = heap_base;
  state.pe_stride = pe_stride;
  state.heap_size = heap_size;
  state.ws_stride = ws_stride;
  state.n_pes = npes;
  // With a host thread per PE, kernels learn their PE from the queue their
  // launching thread bound (rocshmem_emu_bind_stream).
  state.pe_rule = pe_threads_count() > 0 ? detail::PE_RULE_QUEUE : detail::PE_RULE_FIXED;
  state.fixed_pe = acting_pe;
  state.max_teams = max_teams;
  state.default_ctx = d_default_ctx;
  state.world_team = d_teams;
  state.ctx_pool = d_pools;
  state.ws_base = ws_of(0);
  state.nt_bytes = env_size("ROCSHMEM_NT_THRESHOLD", detail::kNonTemporalBytes);
  state.coalesce_puts = env_size("ROCSHMEM_COALESCE_PUTS", 1) != 0 ? 1 : 0;
  // Device waits spin for ever by default, as the reference's do.  Between
  // processes the peer that would end a wait may have died: there the default
  // is a limit generous enough for any live job (minutes of polling), after
  // which the wait gives up and is counted (rocshmem_amd_waits_given_up).
  state.spin_limit = env_size("ROCSHMEM_EMU_SPIN_LIMIT", nprocs ? kProcessSpinLimit : 0);
  RT_CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&d_gave_up), sizeof(unsigned long long)));
  RT_CHECK_HIP(hipMemset(d_gave_up, 0, sizeof(unsigned long long)));
  state.gave_up = d_gave_up;
  live = true;
  push_state();
  ROCSHMEM_TEAM_WORLD = team_handle(0, acting_pe);
  if (nprocs && procs().barrier_world() != 0) _Exit(EXIT_FAILURE);
  return 0;
}

void Runtime::finalize() {
  if (!live) return;
  RT_CHECK_HIP(hipDeviceSynchronize());
  if (nprocs) {
    // Nobody leaves while another PE may still be writing to its slice.  The
    // slice and the mappings stay (see rocshmem_init).
    (void)procs().barrier_world();
    heap_base = nullptr;
    peer_base.clear();
  }
  RT_CHECK_HIP(hipFree(d_peer_delta));
  d_peer_delta = nullptr;
  RT_CHECK_HIP(hipFree(d_queue_table));
  d_queue_table = nullptr;
  RT_CHECK_HIP(hipFree(d_gave_up));
  d_gave_up = nullptr;
  RT_CHECK_HIP(hipHostFree(h_bind_problem));
  h_bind_problem = nullptr;
  RT_CHECK_HIP(hipFree(d_pools));
  RT_CHECK_HIP(hipFree(d_ctx_slots));
  RT_CHECK_HIP(hipFree(d_default_ctx));
  RT_CHECK_HIP(hipFree(d_teams));
  if (d_ws) RT_CHECK_HIP(hipFree(d_ws));
  if (heap_base) release_heap_block(heap_base);
  heap_base = nullptr;
  nprocs = 0;
  d_ws = nullptr;
  d_teams = nullptr;
  h_teams.clear();
  team_slot_used.clear();
  live = false;
  memset(&state, 0, sizeof(state));
  ROCSHMEM_TEAM_WORLD = ROCSHMEM_TEAM_INVALID;
}

void Runtime::require_live(const char *what) const {
  if (!live) {
    fprintf(stderr, "rocshmem: %s called before rocshmem_init\n", what);
    abort();
  }
}

rocshmem_team_t Runtime::team_handle(int pool_index, int pe) const {
  return reinterpret_cast<rocshmem_team_t>(d_teams + static_cast<size_t>(pool_index) * npes + pe);
}

const detail::Team *Runtime::host_team(rocshmem_team_t team) const {
  std::lock_guard<std::mutex> guard(team_lock);
  return host_team_unlocked(team);
}

const detail::Team *Runtime::host_team_unlocked(rocshmem_team_t team) const {
  if (team == ROCSHMEM_TEAM_INVALID || !live) return nullptr;
  const detail::Team *p = reinterpret_cast<const detail::Team *>(team);
  if (p < d_teams || p >= d_teams + static_cast<size_t>(max_teams) * npes) return nullptr;
  const size_t idx = static_cast<size_t>(p - d_teams);
  if (!team_slot_used[idx / npes]) return nullptr;
  return &h_teams[idx];
}

void *Runtime::sym_malloc(size_t size) {
  require_live("rocshmem_malloc");
  const uint64_t off = allocator.alloc(size);
  if (off == Pow2Allocator::kNoBlock) return nullptr;
  return slice_base(me()) + off;
}

void Runtime::sym_free(void *ptr) {
  require_live("rocshmem_free");
  if (!ptr) return;
  const uint64_t off = offset_of(ptr);
  if (off == Pow2Allocator::kNoBlock || !allocator.free(off)) {
    fprintf(stderr, "rocshmem: rocshmem_free of an address that was not allocated\n");
    abort();
  }
}

uint64_t Runtime::offset_of(const void *ptr) const {
  const int pe = pe_of(ptr);
  if (pe < 0) return Pow2Allocator::kNoBlock;
  return static_cast<uint64_t>(static_cast<const char *>(ptr) - slice_base(pe));
}

int Runtime::pe_of(const void *ptr) const {
  const char *p = static_cast<const char *>(ptr);
  if (nprocs) {
    // the slices are mapped wherever HIP put them: look the address up
    for (int pe = 0; pe < npes; ++pe)
      if (p >= peer_base[pe] && p < peer_base[pe] + slice_bytes) return pe;
    return -1;
  }
  if (p < heap_base || p >= heap_base + pe_stride * npes) return -1;
  return static_cast<int>(static_cast<uint64_t>(p - heap_base) / pe_stride);
}

void *Runtime::pe_ptr(const void *ptr, int pe) const {
  const uint64_t off = offset_of(ptr);
  if (off == Pow2Allocator::kNoBlock || pe < 0 || pe >= npes) return nullptr;
  return slice_base(pe) + off;
}

// src/rocshmem.cpp:221-303.  One call creates the team object of every member.
int Runtime::team_split_strided(rocshmem_team_t parent, int start, int stride, int size,
                                rocshmem_team_t *new_team, int *slot_out) {
  require_live("rocshmem_team_split_strided");
  *new_team = ROCSHMEM_TEAM_INVALID;
  if (slot_out) *slot_out = -1;
  // The lock covers validation and the claim of a slot; the device writes
  // below touch only the claimed slot and run unlocked, so that a thread which
  // has to launch a kernel for this one to get past a device-wide wait is not
  // held up in a team lookup.
  std::unique_lock<std::mutex> guard(team_lock);
  if (num_user_teams >= max_teams - 1) return -1;
  if (parent == ROCSHMEM_TEAM_INVALID) return 0;
  const detail::Team *pt = host_team_unlocked(parent);
  if (!pt) return -1;
  if (start < 0 || start >= pt->num_pes || size < 1 || size > pt->num_pes || stride < 1)
    return -1;
  const int start_world = pt->wrt_world.pe_start + pt->wrt_world.stride * start;
  const int stride_world = stride * pt->wrt_world.stride;
  const int end_world = start_world + stride_world * (size - 1);
  // The reference compares with '>' (src/rocshmem.cpp:253-255), which lets a
  // team end one past the last PE; every member must exist here.
  if (end_world >= npes) return -1;

  int slot = -1;
  for (int i = 1; i < max_teams; ++i)
    if (!team_slot_used[i]) { slot = i; break; }
  if (slot < 0) return -1;
  team_slot_used[slot] = true;
  ++num_user_teams;
  guard.unlock();

  // Fresh sync pads for the new team on every PE.
  const size_t pad_bytes = sizeof(detail::SyncPad) * detail::SYNC_KINDS;
  // (one process per PE: each clears its own; the members meet before they use the team)
  for (int pe = 0; pe < npes; ++pe)
    if (!nprocs || pe == acting_pe) RT_CHECK_HIP(hipMemset(team_pads(slot, pe), 0, pad_bytes));

  const detail::TeamInfo world{start_world, stride_world, size, ilog2(stride_world)};
  const detail::TeamInfo wrt_parent{start, stride, size, ilog2(stride)};
  for (int pe = 0; pe < npes; ++pe) {
    const int off = pe - start_world;
    int mine = -1;
    if (off >= 0 && off % stride_world == 0 && off / stride_world < size) mine = off / stride_world;
    write_team(slot, pe, world, wrt_parent, mine);
  }
  RT_CHECK_HIP(hipDeviceSynchronize());
  if (h_teams[static_cast<size_t>(slot) * npes + me()].my_pe >= 0)
    *new_team = team_handle(slot, me());
  if (slot_out) *slot_out = slot;
  return 0;
}

void Runtime::team_destroy(rocshmem_team_t team) {
  if (team == ROCSHMEM_TEAM_INVALID || !live) return;
  std::lock_guard<std::mutex> guard(team_lock);
  const detail::Team *t = host_team_unlocked(team);
  if (!t || t->pool_index == 0) return;
  team_slot_used[t->pool_index] = false;
  --num_user_teams;
}

rocshmem_team_t Runtime::team_on(rocshmem_team_t team, int pe) const {
  std::lock_guard<std::mutex> guard(team_lock);
  const detail::Team *t = host_team_unlocked(team);
  if (!t || pe < 0 || pe >= npes) return ROCSHMEM_TEAM_INVALID;
  if (h_teams[static_cast<size_t>(t->pool_index) * npes + pe].my_pe < 0) return ROCSHMEM_TEAM_INVALID;
  return team_handle(t->pool_index, pe);
}

void Runtime::set_pe(int pe) {
  require_live("rocshmem_emu_set_pe");
  if (pe < 0 || pe >= npes) {
    fprintf(stderr, "rocshmem: PE %d out of range\n", pe);
    abort();
  }
  if (nprocs && pe != acting_pe) {
    fprintf(stderr, "rocshmem: this process is PE %d of a job of processes and cannot act as PE %d\n",
            acting_pe, pe);
    abort();
  }
  acting_pe = pe;
  ROCSHMEM_TEAM_WORLD = team_handle(0, pe);
  if (state.fixed_pe != pe) {
    state.fixed_pe = pe;
    push_state();
  }
}

void Runtime::set_spin_limit(uint64_t polls) {
  require_live("rocshmem_amd_set_spin_limit");
  if (state.spin_limit != polls) {
    state.spin_limit = polls;
    push_state();
  }
}

uint64_t Runtime::waits_given_up(bool clear) {
  require_live("rocshmem_amd_waits_given_up");
  unsigned long long n = 0;
  RT_CHECK_HIP(hipMemcpy(&n, d_gave_up, sizeof(n), hipMemcpyDeviceToHost));
  if (clear && n) RT_CHECK_HIP(hipMemset(d_gave_up, 0, sizeof(n)));
  return n;
}

void Runtime::set_coalesce_puts(int on) {
  require_live("rocshmem_amd_set_coalesce_puts");
  if (state.coalesce_puts != (on ? 1 : 0)) {
    state.coalesce_puts = on ? 1 : 0;
    push_state();
  }
}

void Runtime::set_pe_rule(int rule) {
  require_live("rocshmem_emu_set_pe_rule");
  if (rule < detail::PE_RULE_FIXED || rule > detail::PE_RULE_QUEUE) {
    fprintf(stderr, "rocshmem: unknown PE rule %d\n", rule);
    abort();
  }
  if (state.pe_rule != rule) {
    state.pe_rule = rule;
    push_state();
  }
}

}  // namespace runtime

namespace runtime {
// Meetings of the processes of a job (no-ops when all PEs live in this
// process).  A meeting that fails — a process asked the job to end, or the
// wait ran out — ends this process too.
void procs_meet(int start, int stride, int size) {
  if (!g_rt.live || !g_rt.nprocs) return;
  if (procs().barrier(start, stride, size) != 0) {
    const int asked = procs().abort_requested();
    fflush(nullptr);
    _Exit(asked >= 0 ? asked : EXIT_FAILURE);
  }
}
void procs_meet_world() { procs_meet(0, 1, g_rt.npes); }
}  // namespace runtime

namespace detail {
void register_state_uploader(StateUploader fn) {
  std::lock_guard<std::mutex> guard(runtime::g_uploader_lock);
  runtime::uploaders().push_back(fn);
  if (runtime::g_rt.live) {
    runtime::late_uploaders().push_back(fn);
    runtime::g_late_uploaders.store(true, std::memory_order_release);
  }
}
}  // namespace detail

// ============================ public host API ===============================
using runtime::rt;

// In PE threads every thread calls the collective host functions; the last
// caller of each does the work for all (pe_threads_enter / _leave).
namespace {
struct WorldMeeting {
  uint64_t result = 0;
  bool mine;
  WorldMeeting() : mine(runtime::pe_threads_enter(0, 1, runtime::pe_threads_count(), &result)) {}
  void done(uint64_t r = 0) {
    result = r;
    runtime::pe_threads_leave(0, 1, runtime::pe_threads_count(), r);
  }
};
}  // namespace

__host__ void rocshmem_init(MPI_Comm) {
  // Kernels of different PE threads wait for each other, so no two PE threads
  // may share a hardware queue: refused here, before anything is allocated or
  // enqueued, when there cannot be enough queues.
  // (A program that only uses the host API binds no stream and needs no queue
  // per PE; one built with a per-thread default stream binds one per PE right
  // below.  Streams bound later are counted as they are bound.)
  {
    const int n = runtime::pe_threads_count();
    if (n > 1 && runtime::tl_pe >= 0 && runtime::g_per_thread_default_stream &&
        !runtime::hw_queues_suffice(n, runtime::hw_queue_limit()))
      runtime::refuse_for_queues(n);
  }
  WorldMeeting w;
  if (w.mine) {
    rt().init(runtime::pe_threads_count(), 0);  // one process per PE: meets the others inside
    w.done();
  }
  // A program built with -fgpu-default-stream=per-thread launches its
  // kernel<<<grid, block>>> on this thread's own default stream: bind it now,
  // since such launches do not pass through hipLaunchKernelGGL.  (Not for
  // other programs: the stream would take a hardware queue for nothing.)
  if (runtime::tl_pe >= 0 && runtime::g_per_thread_default_stream)
    rocshmem_emu_bind_stream(hipStreamPerThread);
}
__host__ void rocshmem_init_thread(int, int *provided, MPI_Comm comm) {
  rocshmem_init(comm);
  rocshmem_query_thread(provided);
}
__host__ void rocshmem_query_thread(int *provided) { *provided = ROCSHMEM_THREAD_MULTIPLE; }
__host__ void rocshmem_dump_stats() {}
__host__ void rocshmem_reset_stats() {}
__host__ void rocshmem_finalize() {
  WorldMeeting w;  // (one process per PE: Runtime::finalize meets the others itself)
  if (w.mine) {
    rt().finalize();
    w.done();
  }
}
// Collective (include/rocshmem/rocshmem.hpp:115-123): one allocation serves
// every PE; each caller gets the address in its own slice.
__host__ void *rocshmem_malloc(size_t size) {
  WorldMeeting w;
  if (w.mine) {
    void *mine = rt().sym_malloc(size);
    w.done(mine ? rt().offset_of(mine) + 1 : 0);
  }
  // One process per PE: every process has run its own allocator to the same
  // offset; the call is also a meeting, as in the reference
  // (src/rocshmem.cpp: a barrier ends rocshmem_malloc).
  runtime::procs_meet_world();
  if (!w.result) return nullptr;
  return rt().slice_base(rt().me()) + (w.result - 1);
}
__host__ void rocshmem_free(void *ptr) {
  runtime::procs_meet_world();  // nobody frees what another PE may still be using
  WorldMeeting w;
  if (w.mine) {
    rt().sym_free(ptr);
    w.done();
  }
}
// Usable before rocshmem_init, as in the reference (src/rocshmem.cpp:113-121).
__host__ int rocshmem_n_pes() {
  if (rt().live) return rt().npes;
  if (runtime::procs().attach_from_env()) return runtime::procs().nprocs();
  if (runtime::pe_threads_count() > 0) return runtime::pe_threads_count();
  if (runtime::g_requested_npes > 0) return runtime::g_requested_npes;
  return static_cast<int>(runtime::env_size("ROCSHMEM_EMU_NPES", 1));
}
__host__ int rocshmem_my_pe() {
  if (runtime::tl_pe >= 0) return runtime::tl_pe;
  if (!rt().live && runtime::procs().attach_from_env()) return runtime::procs().rank();
  return rt().live ? rt().acting_pe : 0;
}
__host__ int rocshmem_ctx_create(int64_t options, rocshmem_ctx_t *ctx) {
  rt().require_live("rocshmem_ctx_create");
  *ctx = rt().ctx_handle(rt().me(), options);
  return 0;
}
__host__ void rocshmem_ctx_destroy(rocshmem_ctx_t) {}

// src/team.cpp:51-111
__host__ int rocshmem_team_translate_pe(rocshmem_team_t src_team, int src_pe,
                                        rocshmem_team_t dest_team) {
  const detail::Team *s = rt().host_team(rt().my_view(src_team));
  const detail::Team *d = rt().host_team(rt().my_view(dest_team));
  if (!s || !d) return -1;
  const int world = s->wrt_world.pe_start + s->wrt_world.stride * src_pe;
  const int off = world - d->wrt_world.pe_start;
  if (off < 0 || off % d->wrt_world.stride) return -1;
  const int rel = off / d->wrt_world.stride;
  return rel >= d->num_pes ? -1 : rel;
}
__host__ int rocshmem_team_n_pes(rocshmem_team_t team) {
  const detail::Team *t = rt().host_team(rt().my_view(team));
  return t ? t->num_pes : -1;
}
__host__ int rocshmem_team_my_pe(rocshmem_team_t team) {
  const detail::Team *t = rt().host_team(rt().my_view(team));
  return t ? t->my_pe : -1;
}
// Collective over the parent team (src/rocshmem.cpp:221-303).  In PE threads
// the last member to arrive creates the team objects of all PEs; every caller
// then takes the handle of its own PE.
__host__ int rocshmem_team_split_strided(rocshmem_team_t parent_team, int start, int stride,
                                         int size, const rocshmem_team_config_t *, long,
                                         rocshmem_team_t *new_team) {
  parent_team = rt().my_view(parent_team);
  const detail::Team *pt = rt().host_team(parent_team);
  if (!pt || runtime::tl_pe < 0) {
    // (one process per PE: each member makes its own objects, then they meet)
    const int rc = rt().team_split_strided(parent_team, start, stride, size, new_team);
    if (pt) runtime::procs_meet(pt->wrt_world.pe_start, pt->wrt_world.stride, pt->wrt_world.size);
    return rc;
  }
  const detail::TeamInfo w = pt->wrt_world;
  uint64_t packed = 0;  // (return code + 1) << 32 | (slot + 1)
  if (runtime::pe_threads_enter(w.pe_start, w.stride, w.size, &packed)) {
    rocshmem_team_t unused;
    int created = -1;
    const int rc = rt().team_split_strided(parent_team, start, stride, size, &unused, &created);
    packed = (static_cast<uint64_t>(rc + 1) << 32) | static_cast<uint64_t>(created + 1);
    runtime::pe_threads_leave(w.pe_start, w.stride, w.size, packed);
  }
  const int rc = static_cast<int>(packed >> 32) - 1;
  const int slot = static_cast<int>(packed & 0xffffffffu) - 1;
  // Every member receives the same handle (the first member's object), so a
  // program that keeps it in a variable its PE threads share still works; the
  // host calls and, under the queue rule, the device calls resolve it to the
  // caller's own object.  That variable is written once, with the final value:
  // another member may already be reading it (all members store the same
  // handle), and a transient ROCSHMEM_TEAM_INVALID there would reach its kernel.
  rocshmem_team_t result = ROCSHMEM_TEAM_INVALID;
  if (rc == 0 && slot >= 0) {
    const rocshmem_team_t mine = rt().team_on(rt().team_handle(slot, w.pe_start), rt().me());
    if (mine != ROCSHMEM_TEAM_INVALID) {
      const detail::Team *t = rt().host_team(mine);
      result = rt().team_handle(slot, t->wrt_world.pe_start);
    }
  }
  *new_team = result;
  return rc;
}
__host__ void rocshmem_team_destroy(rocshmem_team_t team) {
  if (team == ROCSHMEM_TEAM_WORLD || team == ROCSHMEM_TEAM_INVALID) return;
  team = rt().my_view(team);
  const detail::Team *t = rt().host_team(team);
  if (!t || t->pool_index == 0) return;
  const detail::TeamInfo w = t->wrt_world;
  if (runtime::pe_threads_enter(w.pe_start, w.stride, w.size, nullptr)) {
    rt().team_destroy(team);
    runtime::pe_threads_leave(w.pe_start, w.stride, w.size, 0);
  }
}
// With every PE in this process, host-side ordering and barriers reduce to
// draining the device.
__host__ void rocshmem_ctx_fence(rocshmem_ctx_t) { RT_CHECK_HIP(hipDeviceSynchronize()); }
__host__ void rocshmem_fence() { RT_CHECK_HIP(hipDeviceSynchronize()); }
__host__ void rocshmem_ctx_quiet(rocshmem_ctx_t) { RT_CHECK_HIP(hipDeviceSynchronize()); }
__host__ void rocshmem_quiet() { RT_CHECK_HIP(hipDeviceSynchronize()); }
__host__ void rocshmem_barrier_all() {
  // A PE thread drains its own streams and then meets the others; draining the
  // whole device from here could wait on a kernel of another PE that in turn
  // waits for work this PE launches after the barrier.
  if (runtime::tl_pe >= 0) RT_CHECK_HIP(rocshmem_emu_device_synchronize());
  WorldMeeting w;
  if (w.mine) {
    if (runtime::tl_pe < 0) RT_CHECK_HIP(hipDeviceSynchronize());
    w.done();
  }
  runtime::procs_meet_world();
}
__host__ void rocshmem_sync_all() { rocshmem_barrier_all(); }
// Ends the whole job at once, as the reference's MPI_Abort does
// (src/rocshmem.cpp): other PE threads may be asleep inside a collective, so
// no destructors run.
__host__ void rocshmem_global_exit(int status) {
  fflush(nullptr);
  runtime::procs().request_abort(status);  // the other processes of the job leave at their next meeting
  _Exit(status);
}

namespace {
// Records "this hardware queue belongs to PE `pe`".  A slot that already names
// another PE for the same queue means two PE threads share the queue; a slot
// that names another queue is a collision in the table.  Either is reported
// through *problem (1 / 2) and leaves the table as it was.
__global__ void bind_queue_kernel(detail::QueueBinding *table, int pe, int *problem) {
  const unsigned long long id = detail::dispatch_queue_id();
  detail::QueueBinding &slot = table[id % detail::kQueueTableSize];
  if (slot.queue_id == id && slot.pe != pe) {
    *problem = 1;
  } else if (slot.queue_id != ~0ull && slot.queue_id != id) {
    *problem = 2;
  } else {
    slot = detail::QueueBinding{id, pe, 0};
  }
}

// Streams the calling PE thread has bound since the runtime came up.
std::vector<hipStream_t> &bound_streams() {
  static thread_local std::vector<hipStream_t> bound;
  static thread_local const void *bound_for = nullptr;
  if (bound_for != rt().d_queue_table) {
    bound.clear();
    bound_for = rt().d_queue_table;
  }
  return bound;
}

// Streams bound by all PE threads of the current runtime.
std::mutex g_bind_lock;
size_t g_bound_total = 0;
const void *g_bound_total_for = nullptr;
}  // namespace

void rocshmem_emu_bind_stream(hipStream_t stream) {
  if (runtime::tl_pe < 0 || !rt().live) return;
  std::vector<hipStream_t> &bound = bound_streams();
  if (std::find(bound.begin(), bound.end(), stream) != bound.end()) return;
  std::lock_guard<std::mutex> guard(g_bind_lock);
  if (g_bound_total_for != rt().d_queue_table) {
    g_bound_total_for = rt().d_queue_table;
    g_bound_total = 0;
  }
  // One more stream than there are hardware queues left would alias an
  // earlier one: refuse before its first kernel is enqueued.
  if (!runtime::hw_queues_suffice(g_bound_total + 1, runtime::hw_queue_limit()) ||
      g_bound_total >= static_cast<size_t>(detail::kQueueTableSize))
    runtime::refuse_for_queues(g_bound_total + 1);
  int *problem = rt().h_bind_problem + g_bound_total;  // pinned word the kernel reports through
  *problem = 0;
  hipLaunchKernelGGL(bind_queue_kernel, dim3(1), dim3(1), 0, stream, rt().d_queue_table,
                     runtime::tl_pe, problem);
  RT_CHECK_HIP(hipGetLastError());
  RT_CHECK_HIP(hipStreamSynchronize(stream));
  const int seen = *problem;
  if (seen) {
    fprintf(stderr,
            seen == 1 ? "rocshmem: the stream PE %d launches on shares its hardware queue with a "
                        "stream of another PE thread; raise GPU_MAX_HW_QUEUES (now %zu)\n"
                      : "rocshmem: PE %d: no room in the queue table for another hardware queue "
                        "(GPU_MAX_HW_QUEUES=%zu)\n",
            runtime::tl_pe, runtime::hw_queue_limit());
    fflush(nullptr);
    _Exit(EXIT_FAILURE);
  }
  ++g_bound_total;
  bound.push_back(stream);
}

// What hipDeviceSynchronize means to a process that is one PE: wait for this
// PE's own work.  The device-wide call would also wait for the kernels of the
// other PE threads, which may be waiting for a kernel this thread has yet to
// launch.
hipError_t rocshmem_emu_device_synchronize() {
  if (runtime::tl_pe < 0 || !rt().live) return hipDeviceSynchronize();
  for (hipStream_t s : bound_streams()) {
    const hipError_t e = hipStreamSynchronize(s);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

int rocshmem_emu_run_pes(int npes, int (*pe_main)(int, char **), int argc, char **argv) {
  // Started as one PE of a job of processes: this process is that PE, no threads.
  if (runtime::procs().attach_from_env()) return pe_main(argc, argv);
  if (npes <= 0) npes = rocshmem_n_pes();
  if (runtime::pe_threads_count() != 0 || rt().live) {
    fprintf(stderr, "rocshmem: rocshmem_emu_run_pes needs a runtime that is not yet up\n");
    abort();
  }
  runtime::pe_threads_start(npes);
  std::vector<int> rc(npes, 0);
  std::vector<std::thread> threads;
  for (int pe = 0; pe < npes; ++pe)
    threads.emplace_back([&rc, pe, pe_main, argc, argv] {
      runtime::tl_pe = pe;
      rc[pe] = pe_main(argc, argv);
    });
  for (auto &t : threads) t.join();
  runtime::pe_threads_start(0);
  for (int r : rc)
    if (r) return r;
  return 0;
}

void rocshmem_emu_set_npes(int npes) { runtime::g_requested_npes = npes; }
void rocshmem_emu_per_thread_default_stream() { runtime::g_per_thread_default_stream = true; }
void rocshmem_emu_set_pe(int pe) { rt().set_pe(pe); }
void rocshmem_emu_set_pe_rule(int rule) { rt().set_pe_rule(rule); }
void *rocshmem_emu_pe_ptr(const void *ptr, int pe) { return rt().pe_ptr(ptr, pe); }
rocshmem_team_t rocshmem_emu_team_on(rocshmem_team_t team, int pe) { return rt().team_on(team, pe); }
size_t rocshmem_emu_pe_stride() { return rt().pe_stride; }

}  // namespace rocshmem
