// Device-visible runtime state: the symmetric-heap geometry, the per-PE
// contexts and teams, and the work/sync area collectives use.
//
// One process hosts all P processing elements: PE p's share of the symmetric
// heap is the slice [heap_base + p*pe_stride, +heap_size).  A symmetric
// address handed to the API is always "my slice" address, and the matching
// address on PE q is   addr + (q - my_pe) * pe_stride   — the closed form of
// the reference's  ipc_bases[pe] + (dest - ipc_bases[my_pe])  translation
// (src/ipc/context_ipc_device.cpp:62-69,109-125) for slices at a fixed stride.
// When every PE is a process of its own (rocshmem_amd/launch.py), a process
// holds its own slice and has the others' mapped through HIP IPC at whatever
// addresses it was given; the distance then comes from a table (remote_addr).
//
// Every translation unit that includes the public header owns a private
// __constant__ copy of DeviceState; the host runtime refreshes all registered
// copies whenever the state changes, so no relocatable device code is needed
// to link user kernels against the library.
#ifndef ROCSHMEM_AMD_DETAIL_STATE_HPP_
#define ROCSHMEM_AMD_DETAIL_STATE_HPP_

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

#include "../rocshmem_common.hpp"

namespace rocshmem {
namespace detail {

// How a work-group that asks for "the" context (default context, or
// rocshmem_wg_ctx_create with no team) learns which PE it is acting as.
enum PeRule : int {
  PE_RULE_FIXED = 0,    // DeviceState::fixed_pe
  PE_RULE_BLOCK_X = 1,  // blockIdx.x % n_pes
  PE_RULE_BLOCK_Y = 2,  // blockIdx.y % n_pes
  PE_RULE_BLOCK_Z = 3,  // blockIdx.z % n_pes
  PE_RULE_QUEUE = 4     // the PE whose host thread bound the hardware queue the
                        // kernel was dispatched on (DeviceState::queue_table)
};

// One entry of the queue -> PE table used when every PE is a host thread: the
// thread binds each stream it launches on by running a one-thread kernel on
// it, which records the id of the hardware queue it finds itself on.
struct QueueBinding {
  unsigned long long queue_id;
  int pe;
  int pad_;
};
constexpr int kQueueTableSize = 64;

// (pe_start, stride, size) of a team with respect to the world team; the
// object rocshmem_ctx_t::team_opaque points at.  Mirrors what the reference
// keeps in TeamInfo (src/team.hpp, used by src/rocshmem_gpu.cpp:267-274).
struct TeamInfo {
  int pe_start;
  int stride;
  int size;
  int log_stride;
};

// Epoch-based flag array one collective kind of one team synchronises on.
// slots[j] holds the highest epoch team member j has announced to this PE;
// epoch is this PE's own count of completed rounds.  Nothing is ever reset,
// so a round costs one store per peer and one polling sweep.
struct SyncPad {
  static constexpr int kMaxPes = 256;
  unsigned long long slots[kMaxPes];
  unsigned long long epoch;
  // On the first member of a team: the counter from which the members'
  // wavefronts draw blocks of a large all-reduce (detail/reduce_engine.hpp).
  unsigned long long tickets;
  unsigned long long pad_[6];
};

enum SyncKind : int {
  SYNC_BARRIER = 0,
  SYNC_REDUCE = 1,
  SYNC_BCAST = 2,
  SYNC_ALLTOALL = 3,
  SYNC_KINDS = 4
};

// Per-PE, per-team object a rocshmem_team_t points at.
struct Team {
  TeamInfo wrt_world;
  TeamInfo wrt_parent;
  int my_pe;           // my index inside this team
  int my_pe_in_world;
  int num_pes;
  int world_size;
  int pool_index;      // which slice of the work/sync area this team owns
  int pad_;
  SyncPad *sync;       // [SYNC_KINDS] pads of this PE for this team
  void *pWrk;          // ROCSHMEM_REDUCE_MIN_WRKDATA_SIZE * 8 bytes
};

// Per-PE communication context (device memory, pooled).  Kernels never write
// a context: the host fills them all in at initialisation, so device code
// reads them through the scalar data path (see ctx_view).
struct alignas(16) Context {
  // What every put, get and atomic reads, side by side: one 16-byte scalar
  // load brings all three.
  uint64_t pe_stride;   // bytes between consecutive slices; 0: the slices are found through peer_delta
  int my_pe;
  unsigned options;     // ROCSHMEM_CTX_* bits, fixed per object
  // With one process per PE the other PEs' slices are mapped wherever HIP put
  // them: peer_delta[pe] = (where PE pe's slice is mapped here) - (my slice).
  // Read only when pe_stride is 0, valid always.
  const int64_t *peer_delta;
  char *heap_base;      // base of PE 0's slice (of this PE's own slice with one process per PE)
  uint64_t ws_stride;   // bytes between consecutive PEs' work/sync areas
  int num_pes;
  int pool_slot;        // index in the context pool, -1 for default contexts
  TeamInfo *tinfo;      // world team of this PE
  SyncPad *world_sync;  // this PE's pad for barrier_all / sync_all
};

// Pool of pre-built contexts for one PE.  A set bit in free_mask marks a free
// slot; claiming is a fetch-and that clears the bit, releasing a fetch-or, so
// work-groups never hold a lock (the reference guards a free list with a
// ticket mutex, src/containers/free_list_impl.hpp:76-137).
// Slot s stands for two prebuilt objects, slots[s] with no option and
// slots[capacity + s] with ROCSHMEM_CTX_NOSTORE, so that claiming a context
// with either option writes nothing into it.
struct CtxPool {
  static constexpr int kMaxWords = 64;  // up to 4096 contexts per PE
  unsigned long long free_mask[kMaxWords];
  int capacity;
  int pad_;
  Context *slots;       // [2 * capacity]
};

struct DeviceState {
  char *heap_base;
  uint64_t pe_stride;
  uint64_t heap_size;
  uint64_t ws_stride;
  int n_pes;
  int pe_rule;
  int fixed_pe;
  int max_teams;
  Context *default_ctx;   // [n_pes]
  Team *world_team;       // [n_pes]
  CtxPool *ctx_pool;      // [n_pes] one pool per PE
  char *ws_base;          // work/sync area of PE 0
  uint64_t nt_bytes;      // copies at least this large use non-temporal accesses
  QueueBinding *queue_table;  // [kQueueTableSize], indexed by queue id modulo the size
  int coalesce_puts;      // thread-level puts first look for one run across the wavefront
  int pad_;
  // Polls after which a wait or barrier gives up, counts itself in *gave_up and
  // returns as if satisfied; 0 = wait for ever, as the reference does.
  uint64_t spin_limit;
  unsigned long long *gave_up;
};

#if defined(__HIPCC__)

// This translation unit's copy of the runtime state.
__attribute__((used)) static __constant__ DeviceState g_state;

// Id of the hardware (HSA) queue this kernel was dispatched on: the `id`
// field of hsa_queue_t, 32 bytes into the structure the queue pointer names.
__device__ __forceinline__ unsigned long long dispatch_queue_id() {
  typedef __attribute__((address_space(4))) unsigned long long constant_u64;
  const constant_u64 *q = (const constant_u64 *)__builtin_amdgcn_queue_ptr();  // NOLINT
  return q[4];
}

__device__ __forceinline__ int acting_pe() {
  const int rule = g_state.pe_rule;
  if (rule == PE_RULE_FIXED) return g_state.fixed_pe;
  if (rule == PE_RULE_QUEUE) {
    const unsigned long long id = dispatch_queue_id();
    const QueueBinding b = g_state.queue_table[id % kQueueTableSize];
    return b.queue_id == id ? b.pe : g_state.fixed_pe;
  }
  const unsigned block = rule == PE_RULE_BLOCK_X ? blockIdx.x
                         : rule == PE_RULE_BLOCK_Y ? blockIdx.y : blockIdx.z;
  return static_cast<int>(block % static_cast<unsigned>(g_state.n_pes));
}

// A null ctx_opaque denotes the default context of the acting PE.
__device__ __forceinline__ Context *ctx_of(rocshmem_ctx_t ctx) {
  Context *c = reinterpret_cast<Context *>(ctx.ctx_opaque);
  return c ? c : g_state.default_ctx + acting_pe();
}

// A team handle names one PE's object of the team.  When kernels take their PE
// from the queue they were dispatched on (one host thread per PE), a handle
// may come from a variable that the PE threads share, so it is re-read as
// "this team" and resolved to the acting PE's object: the objects of one team
// are consecutive, indexed by world PE.  Returns nullptr for
// ROCSHMEM_TEAM_INVALID and for the object of a PE that is not a member;
// callers treat that as an error instead of dereferencing it.
__device__ __forceinline__ Team *team_of(rocshmem_team_t team) {
  Team *t = reinterpret_cast<Team *>(team);
  if (!t) return nullptr;
  if (g_state.pe_rule == PE_RULE_QUEUE) t = t - t->my_pe_in_world + acting_pe();
  return t->my_pe < 0 ? nullptr : t;
}

// A context as read-only data in the constant address space.  The address of a
// context is the same in every lane of a wavefront, and nothing writes a
// context while kernels run, so its fields can come through the scalar data
// cache (one s_load shared by the wavefront, a fraction of the latency of a
// vector load that queues behind the wavefront's bulk traffic).  The compiler
// only chooses that path for memory it knows to be constant.
typedef const __attribute__((address_space(4))) Context ContextView;
__device__ __forceinline__ ContextView *ctx_view(const Context *c) {
  return (ContextView *)c;  // NOLINT: address-space cast
}

// The context's first 16 bytes — stride, PE, options — as the one scalar load
// they share: asked for as a unit, none of the three can be fetched on its
// own later, behind a branch.
static_assert(offsetof(Context, pe_stride) == 0 && offsetof(Context, my_pe) == 8 &&
                  offsetof(Context, options) == 12 && alignof(Context) >= 16,
              "the context's hot fields are read as one 16-byte word");
typedef unsigned HotWords __attribute__((ext_vector_type(4)));
__device__ __forceinline__ HotWords hot_words(const Context *c) {
  return *reinterpret_cast<const __attribute__((address_space(4))) HotWords *>(ctx_view(c));
}
__device__ __forceinline__ unsigned ctx_options(const Context *c) { return hot_words(c).w; }

// One entry of the context's table of mapped slices.  The host writes the
// table once, before any kernel runs, so it is read like the context itself:
// as constant memory, through the scalar data path.  (Read as ordinary global
// memory the entry lands in a vector register, and every address derived from
// it — on the table-free path too, after the two paths merge — is then formed
// and used lane by lane: measured +0.16 us per ping-pong hop.)
__device__ __forceinline__ int64_t peer_hop(const Context *c, int pe) {
  typedef const __attribute__((address_space(4))) int64_t ConstDelta;
  return ((ConstDelta *)ctx_view(c)->peer_delta)[pe];  // NOLINT: address-space cast
}

// Address of the same symmetric object on PE `pe`: my address plus the distance
// between the two slices — the reference's ipc_bases[pe] + (dest - ipc_bases[my_pe])
// (src/ipc/context_ipc_device.cpp:62-69).  With all slices in one allocation
// the distance is a product; with one process per PE (and, by the same code,
// with one GPU per PE) it comes from the context's table of mapped slices.
template <typename T>
__device__ __forceinline__ T *remote_addr(const Context *c, T *local, int pe) {
  // A stride of zero marks a context whose peers are found through the table.
  // The test is on a word that the product needs anyway: the common path
  // stays one scalar load and a multiply.
  const HotWords hot = hot_words(c);
  const uint64_t stride = static_cast<uint64_t>(hot.x) | (static_cast<uint64_t>(hot.y) << 32);
  const int my_pe = static_cast<int>(hot.z);
  int64_t hop = static_cast<int64_t>(pe - my_pe) * static_cast<int64_t>(stride);
  if (__builtin_expect(stride == 0, 0)) hop = peer_hop(c, pe);
  return reinterpret_cast<T *>(
      reinterpret_cast<char *>(const_cast<typename std::remove_const<T>::type *>(local)) + hop);
}

// True when this context finds its peers through the table (one process per PE).
__device__ __forceinline__ bool peers_by_table(const Context *c) {
  const HotWords hot = hot_words(c);
  return (hot.x | hot.y) == 0;
}

// Address of the same work/sync object on PE `pe`.
template <typename T>
__device__ __forceinline__ T *remote_ws(const Context *c, T *local, int pe) {
  // (with one process per PE the area follows the slice in the mapped block)
  int64_t hop;
  if (__builtin_expect(peers_by_table(c), 0))
    hop = peer_hop(c, pe);
  else
    hop = static_cast<int64_t>(pe - ctx_view(c)->my_pe) * static_cast<int64_t>(ctx_view(c)->ws_stride);
  return reinterpret_cast<T *>(reinterpret_cast<char *>(local) + hop);
}

// Work-group extents.  From code object version 5 on (hipcc's default is
// later still) the three 16-bit sizes sit at bytes 12, 14 and 16 of the
// implicit kernel arguments; read as the two aligned words that hold them they
// come through scalar loads, where blockDim.y and .z read one by one get
// merged into a misaligned word that only the vector memory path can fetch.
// A translation unit built for an older code object version
// (-mcode-object-version=4) has another layout there and takes blockDim: the
// version is a constant of the device libraries, so the test folds away.
struct BlockExtent {
  unsigned x, y, z;
};
#if defined(__HIP_DEVICE_COMPILE__)
extern "C" __device__ const int __oclc_ABI_version;
#endif
__device__ __forceinline__ BlockExtent block_extent() {
#if defined(__HIP_DEVICE_COMPILE__)
  if (__oclc_ABI_version < 500) return BlockExtent{blockDim.x, blockDim.y, blockDim.z};
#endif
  typedef const __attribute__((address_space(4))) uint32_t const_u32;
  const_u32 *ia = (const_u32 *)__builtin_amdgcn_implicitarg_ptr();  // NOLINT
  const uint32_t xy = ia[3], z = ia[4];
  return BlockExtent{xy & 0xffffu, xy >> 16, z & 0xffffu};
}
__device__ __forceinline__ unsigned flat_thread_id() {
  const BlockExtent b = block_extent();
  return threadIdx.x + (threadIdx.y + threadIdx.z * b.y) * b.x;
}
__device__ __forceinline__ unsigned flat_block_size() {
  const BlockExtent b = block_extent();
  return b.x * b.y * b.z;
}
__device__ __forceinline__ bool is_block_leader() { return flat_thread_id() == 0; }
__device__ __forceinline__ bool is_wave_leader() {
  return (flat_thread_id() & 63u) == 0;
}

#endif  // __HIPCC__

// ---- host side: keeping every translation unit's g_state current ----------
using StateUploader = void (*)(const DeviceState *);
// Implemented by the runtime library.  Registers `fn` and, when the runtime is
// already initialised, calls it immediately.
void register_state_uploader(StateUploader fn);

#if defined(__HIPCC__)
static void upload_state_to_this_tu(const DeviceState *s) {
  // The address form of the symbol: the only one every HIP build mode offers
  // (a per-thread default stream leaves out the reference-taking overload).
  hipError_t e = hipMemcpyToSymbol(static_cast<const void *>(&g_state), s, sizeof(DeviceState), 0,
                                   hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    fprintf(stderr, "rocshmem: state upload failed: %s\n", hipGetErrorString(e));
    abort();
  }
}
__attribute__((used)) static const int state_uploader_registered_ =
    (register_state_uploader(&upload_state_to_this_tu), 0);
#endif

}  // namespace detail
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_DETAIL_STATE_HPP_
