// Host-side runtime object shared by the C++ host API, the C entry points and
// the kernel launchers.
#ifndef ROCSHMEM_AMD_RUNTIME_HPP_
#define ROCSHMEM_AMD_RUNTIME_HPP_

#include <cstddef>
#include <cstdint>
#include <mutex>
#include <vector>

#include "pow2_allocator.hpp"
#include "rocshmem/detail/state.hpp"

namespace rocshmem {
namespace runtime {

// PE this thread runs as while rocshmem_emu_run_pes hosts one thread per PE;
// -1 for every other thread.
extern thread_local int tl_pe;

struct Runtime {
  bool live = false;
  int npes = 0;
  int acting_pe = 0;  // PE the host acts as outside PE threads (rocshmem_emu_set_pe)
  // PE the calling thread acts as.
  int me() const { return tl_pe >= 0 ? tl_pe : acting_pe; }
  int max_ctxs = 0;
  int max_teams = 0;
  int num_user_teams = 0;
  size_t heap_size = 0;
  // Bytes between the slices of consecutive PEs.  With one process per PE the
  // slices are separate mappings and no such distance exists: the stride is 0
  // there (host or device arithmetic that still used it would stay inside the
  // caller's own slice) and slice_bytes is what a slice spans.
  size_t pe_stride = 0;
  size_t slice_bytes = 0;
  size_t ws_stride = 0;
  size_t heap_alloc_bytes = 0;  // size of the device allocation that holds the slices
  bool heap_uncached = true;    // false under ROCSHMEM_EMU_HEAP_CACHED=1
  char *heap_base = nullptr;
  // One process per PE (proc_group.hpp): this process holds its own slice and
  // has the others' mapped through HIP IPC wherever HIP put them.
  int nprocs = 0;                   // 0: all PEs live in this process
  std::vector<char *> peer_base;    // [npes] in process mode: where each PE's slice is mapped here
  int64_t *d_peer_delta = nullptr;  // device, [npes][npes]: (slice of p) - (slice of q) at [q][p]
  char *slice_base(int pe) const {
    return nprocs ? peer_base[pe] : heap_base + static_cast<size_t>(pe) * pe_stride;
  }
  char *d_ws = nullptr;
  detail::Team *d_teams = nullptr;         // [max_teams][npes]
  detail::Context *d_default_ctx = nullptr;  // [2*npes]: default, then NOSTORE
  detail::Context *d_ctx_slots = nullptr;  // [npes][2 * max_ctxs]: per slot one object per ordering option
  detail::CtxPool *d_pools = nullptr;      // [npes]
  detail::QueueBinding *d_queue_table = nullptr;  // [kQueueTableSize]
  unsigned long long *d_gave_up = nullptr;  // waits and barriers that ran into the spin limit
  int *h_bind_problem = nullptr;  // pinned, [kQueueTableSize]: what each stream binding reported
  std::vector<detail::Team> h_teams;       // host mirror of d_teams
  std::vector<bool> team_slot_used;
  Pow2Allocator allocator;
  detail::DeviceState state{};

  int init(int want_npes, size_t want_heap);
  void finalize();
  void require_live(const char *what) const;
  void push_state();

  void *sym_malloc(size_t size);
  void sym_free(void *ptr);
  uint64_t offset_of(const void *ptr) const;
  int pe_of(const void *ptr) const;
  void *pe_ptr(const void *ptr, int pe) const;

  // Team creation, destruction and lookup may come from several host threads
  // at once (PE threads whose sub-teams are disjoint meet at different
  // rendezvous points): team_lock serialises them.  slot_out, when given,
  // receives the team's slot (-1 on failure).
  int team_split_strided(rocshmem_team_t parent, int start, int stride, int size,
                         rocshmem_team_t *new_team, int *slot_out = nullptr);
  void team_destroy(rocshmem_team_t team);
  rocshmem_team_t team_handle(int pool_index, int pe) const;
  rocshmem_team_t team_on(rocshmem_team_t team, int pe) const;
  // The handle a PE thread should use for `team`: its own PE's view of it
  // (ROCSHMEM_TEAM_WORLD is one global and names PE 0's view).  Unchanged
  // outside PE threads.
  rocshmem_team_t my_view(rocshmem_team_t team) const {
    return tl_pe < 0 ? team : team_on(team, tl_pe);
  }
  const detail::Team *host_team(rocshmem_team_t team) const;
  mutable std::mutex team_lock;

  void set_pe(int pe);
  void set_pe_rule(int rule);
  void set_coalesce_puts(int on);
  void set_spin_limit(uint64_t polls);
  uint64_t waits_given_up(bool clear);

  // Context handle of PE `pe` bound to its member object of team slot `slot`.
  rocshmem_ctx_t default_ctx_handle(int pe, int slot = 0) const {
    return rocshmem_ctx_t{d_default_ctx + pe,
                          &d_teams[static_cast<size_t>(slot) * npes + pe].wrt_world};
  }

  // Options of the contexts the benchmark/test drivers act through.
  int64_t driver_ctx_options = 0;
  detail::Context *driver_ctx_row() const {
    return d_default_ctx + ((driver_ctx_options & ROCSHMEM_CTX_NOSTORE) ? npes : 0);
  }
  rocshmem_ctx_t driver_ctx_handle(int pe) const { return ctx_handle(pe, driver_ctx_options); }

  // Host-created context of PE `pe` on the world team with `options`
  // (ROCSHMEM_CTX_* bits).  Contexts hold no per-context state here, so all
  // contexts of one PE with the same ordering option share one object.
  rocshmem_ctx_t ctx_handle(int pe, int64_t options) const {
    const bool nostore = (options & ROCSHMEM_CTX_NOSTORE) != 0;
    return rocshmem_ctx_t{d_default_ctx + (nostore ? npes : 0) + pe, &d_teams[pe].wrt_world};
  }

 private:
  const detail::Team *host_team_unlocked(rocshmem_team_t team) const;
  size_t ws_bytes_per_pe() const;
  char *ws_of(int pe) const;  // work/sync area of a PE
  detail::SyncPad *team_pads(int pool_index, int pe) const;
  void write_team(int pool_index, int pe, const detail::TeamInfo &world,
                  const detail::TeamInfo &parent, int my_pe_in_team);
};

Runtime &rt();

// One process per PE: meet the other processes of the strided PE set / of the
// world (nothing to do when all PEs live in this process).
void procs_meet(int start, int stride, int size);
void procs_meet_world();

// Uncached heap blocks this process holds (they are kept until it ends): all
// of them, and those no live runtime uses.
void heap_held(size_t *total, size_t *idle);

// ---- one thread per PE (rocshmem_emu_run_pes) --------------------------------
// Collective host calls made by PE threads meet here.  The callers are the
// members of the strided set (start, stride, size) of world PEs.  enter()
// returns true in exactly one of them, the last to arrive, which performs the
// operation for the whole set and then calls leave(result); the others sleep
// in enter() until then and return false with *result filled in.  Outside PE
// threads enter() returns true at once and leave() does nothing.
bool pe_threads_enter(int start, int stride, int size, uint64_t *result);
void pe_threads_leave(int start, int stride, int size, uint64_t result);
int pe_threads_count();  // P while PE threads run, else 0
// Hardware queues HIP will use (GPU_MAX_HW_QUEUES, default 4); whether
// `pe_streams` streams of PE threads plus one for the library fit; and the
// fatal refusal (message, exit status 1, nothing launched) when they do not.
size_t hw_queue_limit();
bool hw_queues_suffice(size_t pe_streams, size_t hw_queues);
[[noreturn]] void refuse_for_queues(size_t pe_streams);
void pe_threads_start(int npes);

}  // namespace runtime
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_RUNTIME_HPP_
