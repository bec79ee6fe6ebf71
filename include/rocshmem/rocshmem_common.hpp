// Enumerations, ABI constants and handle types shared by the host and device
// halves of the symmetric-heap data-movement API.
//
// Values and layouts are ABI: they match the reference's
// include/rocshmem/rocshmem_common.hpp:35-126 (enum orders, sync-array sizes,
// context option bits, the two-pointer rocshmem_ctx_t, rocshmem_team_t as a
// uint64_t pointer, ROCSHMEM_TEAM_INVALID == nullptr).
#ifndef ROCSHMEM_AMD_COMMON_HPP_
#define ROCSHMEM_AMD_COMMON_HPP_

#include <cstddef>
#include <cstdint>

// The device API is defined in these headers.  A call that stays a call costs
// a GPU kernel the callee's worst-case register budget, a stack frame in
// scratch memory and spilled scalar registers around it (the many-teams
// all-reduce driver: 120 vector registers and 88 bytes of scratch per lane
// with the public function called, against 40 and none with it inlined), so
// by default every public device function is inlined into its caller.
// USE_FUNC_CALL keeps the reference's meaning: real calls.
#ifdef USE_FUNC_CALL
#define ATTR_NO_INLINE __attribute__((noinline))
#else
#define ATTR_NO_INLINE __attribute__((always_inline))
#endif

namespace rocshmem {

enum ROCSHMEM_STATUS { ROCSHMEM_SUCCESS = 0, ROCSHMEM_ERROR = 1 };

enum ROCSHMEM_OP {
  ROCSHMEM_SUM = 0,
  ROCSHMEM_MAX = 1,
  ROCSHMEM_MIN = 2,
  ROCSHMEM_PROD = 3,
  ROCSHMEM_AND = 4,
  ROCSHMEM_OR = 5,
  ROCSHMEM_XOR = 6,
  ROCSHMEM_REPLACE = 7
};

enum ROCSHMEM_SIGNAL_OPS { ROCSHMEM_SIGNAL_SET = 0, ROCSHMEM_SIGNAL_ADD = 1 };

enum rocshmem_cmps {
  ROCSHMEM_CMP_EQ = 0,
  ROCSHMEM_CMP_NE = 1,
  ROCSHMEM_CMP_GT = 2,
  ROCSHMEM_CMP_GE = 3,
  ROCSHMEM_CMP_LT = 4,
  ROCSHMEM_CMP_LE = 5
};

enum rocshmem_thread_ops {
  ROCSHMEM_THREAD_SINGLE = 0,
  ROCSHMEM_THREAD_FUNNELED = 1,
  ROCSHMEM_THREAD_WG_FUNNELED = 2,
  ROCSHMEM_THREAD_SERIALIZED = 3,
  ROCSHMEM_THREAD_MULTIPLE = 4
};

enum rocshmem_team_configs {
  ROCSHMEM_TEAM_DEFAULT_CONFIGS = 0,
  ROCSHMEM_TEAM_NUM_CONTEXTS = 1
};

typedef struct {
  int num_contexts;
} rocshmem_team_config_t;

constexpr size_t ROCSHMEM_REDUCE_MIN_WRKDATA_SIZE = 1024;
constexpr size_t ROCSHMEM_ATA_MAX_WRKDATA_SIZE = 4u * 1024u * 1024u;
constexpr size_t ROCSHMEM_BARRIER_SYNC_SIZE = 256;
constexpr size_t ROCSHMEM_REDUCE_SYNC_SIZE = 256;
constexpr size_t ROCSHMEM_BCAST_SYNC_SIZE = ROCSHMEM_BARRIER_SYNC_SIZE;
constexpr size_t ROCSHMEM_ALLTOALL_SYNC_SIZE = ROCSHMEM_BARRIER_SYNC_SIZE + 1;
constexpr size_t ROCSHMEM_FCOLLECT_SYNC_SIZE = ROCSHMEM_ALLTOALL_SYNC_SIZE;
constexpr size_t ROCSHMEM_SYNC_VALUE = 0;

const int ROCSHMEM_CTX_ZERO = 0;
const int ROCSHMEM_CTX_NOSTORE = 1;
const int ROCSHMEM_CTX_SERIALIZED = 2;
const int ROCSHMEM_CTX_WG_PRIVATE = 4;
const int ROCSHMEM_CTX_SHARED = 8;

// Context handle.  ctx_opaque points at a detail::Context in device memory,
// team_opaque at the detail::TeamInfo (pe_start, stride, size) the context
// translates team-relative PE numbers with.
typedef struct {
  void *ctx_opaque;
  void *team_opaque;
} rocshmem_ctx_t;

// Team handle: address of a detail::Team object in device memory.
typedef uint64_t *rocshmem_team_t;
const rocshmem_team_t ROCSHMEM_TEAM_INVALID = nullptr;

// Host-side handle of the world team of the acting PE (set by rocshmem_init).
extern rocshmem_team_t ROCSHMEM_TEAM_WORLD;

}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_COMMON_HPP_
