/* C entry points of the MI355X symmetric-heap data-movement library.
 *
 * The reference library has no C or FFI layer: its interface is the C++ API of
 * include/rocshmem/rocshmem.hpp, with the data path living in __device__
 * functions that user kernels call.  This header is that interface flattened
 * for callers that cannot compile HIP C++ (ctypes, cgo, JNI ...):
 *
 *   - the host API (init / malloc / teams) one to one, and
 *   - for every device-side operation a "driver": a kernel launch in which
 *     work-groups call the public device function exactly as a user kernel
 *     would, with the PE each work-group acts for given by the caller.
 *
 * Conventions
 *   - All P processing elements live in this process on one GPU, unless the
 *     process was started as one PE of a job of processes (see "One process
 *     per PE" below): then it acts for that PE only (`my_pe` must be it) and
 *     the drivers that host several PEs in one launch return -1.  A symmetric
 *     address is always passed as the address on PE `my_pe` (what
 *     rocshmem_amd_malloc returned while that PE was acting, or
 *     rocshmem_amd_pe_ptr of it).
 *   - `stream` is a hipStream_t (NULL = the null stream).  Drivers only
 *     enqueue; call rocshmem_amd_stream_sync to wait.
 *   - Return value 0 = success, negative = argument error (nothing launched).
 *     HIP failures are fatal (message on stderr, exit), as in the reference
 *     (src/util.hpp:41-49).
 */
#ifndef ROCSHMEM_AMD_H_
#define ROCSHMEM_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *rocshmem_amd_stream_t;
typedef void *rocshmem_amd_team_t;

/* Element types (reductions, atomics, waits). */
enum rocshmem_amd_dtype {
  ROCSHMEM_AMD_SHORT = 0,
  ROCSHMEM_AMD_INT = 1,
  ROCSHMEM_AMD_LONG = 2,
  ROCSHMEM_AMD_LONGLONG = 3,
  ROCSHMEM_AMD_FLOAT = 4,
  ROCSHMEM_AMD_DOUBLE = 5,
  ROCSHMEM_AMD_BF16 = 6,
  ROCSHMEM_AMD_UINT = 7,
  ROCSHMEM_AMD_ULONG = 8,
  ROCSHMEM_AMD_ULONGLONG = 9,
  /* host-side waits only */
  ROCSHMEM_AMD_CHAR = 10,
  ROCSHMEM_AMD_SCHAR = 11,
  ROCSHMEM_AMD_UCHAR = 12,
  ROCSHMEM_AMD_USHORT = 13
};

/* Reduction operators: values of ROCSHMEM_OP (rocshmem_common.hpp:40-49). */
enum rocshmem_amd_op {
  ROCSHMEM_AMD_SUM = 0,
  ROCSHMEM_AMD_MAX = 1,
  ROCSHMEM_AMD_MIN = 2,
  ROCSHMEM_AMD_PROD = 3,
  ROCSHMEM_AMD_AND = 4,
  ROCSHMEM_AMD_OR = 5,
  ROCSHMEM_AMD_XOR = 6
};

enum rocshmem_amd_granularity {
  ROCSHMEM_AMD_THREAD = 0, /* rocshmem_putmem / getmem            */
  ROCSHMEM_AMD_WAVE = 1,   /* rocshmem_putmem_wave / getmem_wave  */
  ROCSHMEM_AMD_WG = 2      /* rocshmem_putmem_wg / getmem_wg      */
};

enum rocshmem_amd_rma_op {
  ROCSHMEM_AMD_PUT = 0,
  ROCSHMEM_AMD_GET = 1,
  ROCSHMEM_AMD_PUT_NBI = 2, /* rocshmem_putmem_nbi[_wave|_wg]: completes at the closing quiet */
  ROCSHMEM_AMD_GET_NBI = 3
};

enum rocshmem_amd_amo_op {
  ROCSHMEM_AMD_AMO_FETCH_ADD = 0,
  ROCSHMEM_AMD_AMO_ADD = 1,
  ROCSHMEM_AMD_AMO_FETCH_INC = 2,
  ROCSHMEM_AMD_AMO_INC = 3,
  ROCSHMEM_AMD_AMO_COMPARE_SWAP = 4,
  ROCSHMEM_AMD_AMO_FETCH = 5,
  ROCSHMEM_AMD_AMO_SET = 6,
  ROCSHMEM_AMD_AMO_SWAP = 7,
  ROCSHMEM_AMD_AMO_FETCH_AND = 8,
  ROCSHMEM_AMD_AMO_FETCH_OR = 9,
  ROCSHMEM_AMD_AMO_FETCH_XOR = 10
};

enum rocshmem_amd_wait_fn {
  ROCSHMEM_AMD_TEST = 0,
  ROCSHMEM_AMD_WAIT_UNTIL = 1,
  ROCSHMEM_AMD_WAIT_UNTIL_ANY = 2,
  ROCSHMEM_AMD_WAIT_UNTIL_ALL = 3,
  ROCSHMEM_AMD_WAIT_UNTIL_SOME = 4
};

enum rocshmem_amd_sync_fn {
  ROCSHMEM_AMD_BARRIER_ALL = 0, /* rocshmem_ctx_wg_barrier_all */
  ROCSHMEM_AMD_SYNC_ALL = 1,    /* rocshmem_ctx_wg_sync_all    */
  ROCSHMEM_AMD_TEAM_SYNC = 2    /* rocshmem_ctx_wg_team_sync   */
};

/* ===================== host API (runtime, heap, teams) ===================== */

/* rocshmem_init (include/rocshmem/rocshmem.hpp:62, src/rocshmem.cpp:73-105).
 * npes <= 0: take ROCSHMEM_EMU_NPES (default 1); heap_bytes_per_pe == 0: take
 * ROCSHMEM_HEAP_SIZE (default 1 GiB, src/memory/heap_memory.hpp:114). */
int rocshmem_amd_init(int npes, size_t heap_bytes_per_pe);
/* rocshmem_finalize (rocshmem.hpp:103). */
int rocshmem_amd_finalize(void);
/* rocshmem_n_pes / rocshmem_my_pe (rocshmem.hpp:130-137). */
int rocshmem_amd_n_pes(void);
int rocshmem_amd_my_pe(void);
/* Emulation controls (no reference counterpart): which PE the host acts as,
 * and how default-context work-groups find their PE (0 fixed, 1/2/3 =
 * blockIdx.x/y/z mod P). */
int rocshmem_amd_set_pe(int pe);
int rocshmem_amd_set_pe_rule(int rule);
/* Options (ROCSHMEM_CTX_* bits, include/rocshmem/rocshmem_common.hpp:98-102)
 * of the contexts the RMA, AMO, put_signal, ping-pong and dispatch drivers
 * below act through, as if each PE had called
 * rocshmem_ctx_create(options, &ctx) (rocshmem.hpp:144) and used that ctx.
 * 0 (the start value) is the default context.  With ROCSHMEM_CTX_NOSTORE (1)
 * quiet / fence, the close of every _wave / _wg put and the signal of
 * put_signal wait on the wavefront's own write-through stores instead of
 * writing the L2 back, and AMOs are relaxed (src/fence_policy.hpp:45-63 turns
 * the reference's flush off for that option).  Returns the previous options,
 * -1 before init. */
int64_t rocshmem_amd_set_ctx_options(int64_t options);
/* One process per PE.  The reference runs one process per PE under an MPI
 * launcher and exchanges the heaps' IPC handles with MPI_Allgather
 * (src/ipc_policy.cpp:34-118, src/ipc/backend_ipc.cpp:274-357).  Here
 * `python -m rocshmem_amd.launch -n P prog args...` starts P processes of an
 * unchanged program with ROCSHMEM_EMU_PROCS / _RANK / _RDV set; rocshmem_init
 * then allocates this PE's heap (below 2 GiB), publishes its HIP IPC handle
 * through the rendezvous file, maps the other PEs' heaps, and device code
 * finds a peer's slice through a table (detail/state.hpp::remote_addr).  The
 * host API works between the processes (put / get / atomics / waits on mapped
 * memory, barriers and collective malloc / free through the rendezvous file,
 * to_all / reduce / broadcast / alltoall / fcollect by pulling); device-side
 * collectives and barriers between processes are not supported, and the test
 * drivers of this header are for the one-process harness.
 *
 * The rendezvous on its own (no GPU needed, for tests and other launchers):
 * a zero-filled file of rocshmem_amd_procs_file_bytes() bytes shared by the
 * processes; attach maps it for rank `rank` of `nprocs`; barrier meets the
 * other members of the strided PE set (0, or -1 after ROCSHMEM_EMU_RDV_TIMEOUT_S
 * seconds, default 120, or once a process has asked the job to end); publish
 * stores up to 192 bytes in this rank's area and fetch reads a rank's area
 * (meet in between); request_abort asks every process to leave at its next
 * meeting, abort_requested returns the status asked for or -1; count is the
 * number of processes of the job this process was started as one PE of (it
 * attaches from the environment when that has not happened yet), 0 when it
 * was not. */
size_t rocshmem_amd_procs_file_bytes(void);
int rocshmem_amd_procs_count(void);
int rocshmem_amd_procs_attach(const char *path, int nprocs, int rank);
int rocshmem_amd_procs_barrier(int PE_start, int PE_stride, int PE_size);
int rocshmem_amd_procs_publish(const void *bytes, size_t n);
int rocshmem_amd_procs_fetch(int rank, void *bytes, size_t n);
int rocshmem_amd_procs_request_abort(int status);
int rocshmem_amd_procs_abort_requested(void);
/* The reference's device-side waits and barriers spin without bound
 * (src/context_tmpl_device.hpp:201-218, src/ipc/context_ipc_device_coll.cpp:31-99),
 * and by default so do these.  With a limit (polls per wait; initial value
 * ROCSHMEM_EMU_SPIN_LIMIT, 0 = none) a wait_until* or barrier that has polled
 * that often counts itself, stops waiting and returns, so that a kernel whose
 * partner never arrives ends instead of holding the GPU; what it returns with
 * is then not to be trusted.  rocshmem_amd_waits_given_up returns how many
 * waits have ended that way since the count was last cleared (clear != 0
 * clears it); call it after waiting for the kernels.  -1 before rocshmem_init. */
int rocshmem_amd_set_spin_limit(uint64_t polls);
int64_t rocshmem_amd_waits_given_up(int clear);
/* Whether thread-level puts (rocshmem_putmem / rocshmem_<T>_put) first look
 * for one run across the active lanes of the wavefront — messages to the same
 * PE that continue one another, what the reference's coalescing policy merges
 * (src/wf_coal_policy.cpp:57-172) — and move such a run with the whole
 * wavefront.  Initial value: ROCSHMEM_COALESCE_PUTS (default 1: on).  Returns the
 * previous setting, -1 before rocshmem_init. */
int rocshmem_amd_set_coalesce_puts(int on);
/* rocshmem_malloc / rocshmem_free (rocshmem.hpp:115-123): NULL on size 0 or
 * exhaustion; the object exists at the same offset on every PE. */
void *rocshmem_amd_malloc(size_t size);
int rocshmem_amd_free(void *ptr);
/* Host rocshmem_barrier_all (rocshmem.hpp; src/rocshmem.cpp): waits for the
 * device work of this process and, with one process per PE, for every other
 * PE to arrive.  -1 before rocshmem_init. */
int rocshmem_amd_barrier_all(void);
/* Address of a symmetric object on another PE; NULL if ptr is not in the heap. */
void *rocshmem_amd_pe_ptr(const void *ptr, int pe);
/* Allocator accounting: SingleHeap::get_size/get_used/get_avail
 * (src/memory/single_heap.cpp:56-62), per PE. */
size_t rocshmem_amd_heap_size(void);
size_t rocshmem_amd_heap_used(void);
size_t rocshmem_amd_heap_avail(void);
/* Bytes between the slices of consecutive PEs (0 with one process per PE,
 * where the slices are separate mappings: use rocshmem_amd_pe_ptr). */
size_t rocshmem_amd_pe_stride(void);
/* Bytes of the one device allocation that holds the P slices (no reference
 * counterpart: there every PE allocates its own heap, src/memory/heap_memory.hpp).
 * pe_stride x P by default (stride = heap size rounded up to 2 MiB);
 * ROCSHMEM_EMU_SPREAD=1 spreads the slices over half of the device memory. */
size_t rocshmem_amd_heap_alloc_bytes(void);
/* 1 when the heap of the live runtime is uncached device memory (the default),
 * 0 under ROCSHMEM_EMU_HEAP_CACHED=1 (plain hipMalloc, what the reference's
 * IPC build uses: src/memory/heap_type.hpp:41-51), -1 before rocshmem_init. */
int rocshmem_amd_heap_is_uncached(void);
/* Uncached heap blocks are kept until the process ends (rocshmem_finalize
 * marks them idle, a later rocshmem_init reuses the smallest idle block that
 * is large enough).  total_bytes: all such blocks of this process; idle_bytes:
 * those no live runtime uses.  A new block that would take the total beyond
 * ROCSHMEM_EMU_HEAP_HELD_LIMIT (bytes, default: the device memory) is refused
 * with a message.  No reference counterpart. */
int rocshmem_amd_heap_held(size_t *total_bytes, size_t *idle_bytes);

/* The allocator on its own, usable without a GPU (planning and host-side
 * tests): a model heap of heap_bytes whose base has the alignment of
 * base_address.  Same algorithm as rocshmem_amd_malloc: SingleHeap / Pow2Bins
 * (src/memory/single_heap.cpp:29-64, pow2_bins.hpp:90-152).  alloc returns the
 * block's offset from the base, or UINT64_MAX for "nullptr". */
void *rocshmem_amd_heap_model_create(uint64_t base_address, uint64_t heap_bytes);
void rocshmem_amd_heap_model_destroy(void *model);
uint64_t rocshmem_amd_heap_model_alloc(void *model, uint64_t size);
int rocshmem_amd_heap_model_free(void *model, uint64_t offset);
uint64_t rocshmem_amd_heap_model_used(void *model);
uint64_t rocshmem_amd_heap_model_num_bins(void *model);
uint64_t rocshmem_amd_heap_model_bin_population(void *model, uint64_t block_bytes);

/* Teams (rocshmem.hpp:165-236; src/rocshmem.cpp:193-319, src/team.cpp:51-111). */
rocshmem_amd_team_t rocshmem_amd_team_world(void);
int rocshmem_amd_team_split_strided(rocshmem_amd_team_t parent, int start, int stride,
                                    int size, rocshmem_amd_team_t *new_team);
void rocshmem_amd_team_destroy(rocshmem_amd_team_t team);
int rocshmem_amd_team_n_pes(rocshmem_amd_team_t team);
int rocshmem_amd_team_my_pe(rocshmem_amd_team_t team);
int rocshmem_amd_team_translate_pe(rocshmem_amd_team_t src_team, int src_pe,
                                   rocshmem_amd_team_t dest_team);
/* The same team as seen by another PE (NULL if that PE is not a member). */
rocshmem_amd_team_t rocshmem_amd_team_on(rocshmem_amd_team_t team, int pe);

/* World PEs of a team: PE_start, PE_start + PE_stride, ... (PE_size of them). */
int rocshmem_amd_team_active_set(rocshmem_amd_team_t team, int *PE_start, int *PE_stride,
                                 int *PE_size);
/* Launch rules of the drivers whose work-groups wait for each other (wg_reduce,
 * wg_reduce_teams, wg_alltoall / broadcast / fcollect, wg_sync, pingpong,
 * put_flag_check, wait_test_woken).  No reference counterpart: the reference
 * leaves co-residency to the caller (its barriers spin without bound,
 * src/ipc/context_ipc_device_coll.cpp:31-99).  Such a grid is launched only if
 * all of it can be resident at once, n_wgs <= wgs_per_cu x n_cus with
 * wgs_per_cu from hipOccupancyMaxActiveBlocksPerMultiprocessor for the kernel
 * and work-group size; otherwise the driver returns -1 and launches nothing.
 * This is that arithmetic (1 = fits). */
int rocshmem_amd_coresident(long n_wgs, int wgs_per_cu, int n_cus);
/* With one host thread per PE (rocshmem_emu_run_pes) every stream a PE thread
 * launches on needs a hardware queue of its own, plus one for the library:
 * 1 if pe_streams + 1 <= hw_queues (GPU_MAX_HW_QUEUES, HIP's default 4).
 * rocshmem_init and the stream binding end the process with a message,
 * before enqueueing anything, when this is 0. */
int rocshmem_amd_hw_queues_suffice(size_t pe_streams, size_t hw_queues);
/* Meeting point of the host collectives when every PE is a thread of this
 * process (rocshmem_emu_run_pes, include/rocshmem/rocshmem_emu.hpp; the
 * reference's PEs are processes that meet inside MPI).  Each member of the
 * strided set calls enter: it returns 1 in the last one to arrive, which then
 * performs the operation for the whole set and calls leave; in the others it
 * returns 0 once that has happened.  Outside PE threads enter returns 1 at
 * once and leave does nothing. */
int rocshmem_amd_pe_threads_enter(int PE_start, int PE_stride, int PE_size);
void rocshmem_amd_pe_threads_leave(int PE_start, int PE_stride, int PE_size);

/* Plain device memory and staging for callers without a HIP binding. */
int rocshmem_amd_dev_mem_info(size_t *free_bytes, size_t *total_bytes); /* hipMemGetInfo */
void *rocshmem_amd_dev_alloc(size_t size);
int rocshmem_amd_dev_free(void *ptr);
int rocshmem_amd_copy_in(void *dst_dev, const void *src_host, size_t n);
int rocshmem_amd_copy_out(void *dst_host, const void *src_dev, size_t n);
int rocshmem_amd_fill(void *dst_dev, int byte, size_t n);
/* Compares two device buffers on the device (after waiting for the stream):
 * differing_out = the number of 16-byte vectors, plus tail bytes, in which they
 * differ.  How the benchmark verifies what its timed loops moved without
 * bringing 256 MiB back to the host.  No reference counterpart. */
int rocshmem_amd_compare(const void *x, const void *y, size_t nbytes, uint64_t *differing_out,
                         rocshmem_amd_stream_t stream);
/* The symmetric object `sym` (address on PE 0) set to `byte` on every PE with
 * one launch on `stream` — e.g. signal words cleared between dispatches. */
int rocshmem_amd_fill_every_pe(void *sym, int byte, size_t n, rocshmem_amd_stream_t stream);
/* hipMemcpy device-to-device by the HIP runtime's own copy kernel: a plain copy
 * of known size to calibrate hardware byte counters against. */
int rocshmem_amd_copy_dev(void *dst_dev, const void *src_dev, size_t n);
int rocshmem_amd_stream_sync(rocshmem_amd_stream_t stream);
/* hipEvent pair on `stream`; elapsed time in milliseconds. */
void *rocshmem_amd_timer_create(void);
int rocshmem_amd_timer_start(void *timer, rocshmem_amd_stream_t stream);
int rocshmem_amd_timer_stop(void *timer, rocshmem_amd_stream_t stream);
float rocshmem_amd_timer_elapsed_ms(void *timer);
int rocshmem_amd_timer_destroy(void *timer);

/* ============================ RMA drivers ================================== */

/* rocshmem_ctx_putmem[_wave|_wg] / rocshmem_ctx_getmem[_wave|_wg]
 * (rocshmem_RMA.hpp, rocshmem_RMA_X.hpp:243-274,744-775;
 *  src/ipc/context_ipc_device.cpp:62-164).
 * n_wgs work-groups of wg_size threads act for PE my_pe.  The message of
 * nbytes is cut into tiles of tile_bytes (0 = one equal share per group,
 * rounded up to 16 bytes); group g — a work-group, a wavefront or a thread,
 * per `gran` — moves tiles g, g+G, g+2G ... with one API call each.  The whole
 * transfer is repeated `iters` times inside the kernel, which ends with one
 * rocshmem_ctx_quiet per group.  The _NBI operations issue
 * rocshmem_ctx_putmem_nbi[_wave|_wg] / getmem_nbi[_wave|_wg]
 * (rocshmem_RMA.hpp:259-264,640-645) instead, which that quiet completes. */
int rocshmem_amd_rma(int rma_op, int gran, void *dest, const void *source, size_t nbytes,
                     size_t tile_bytes, int my_pe, int pe, int n_wgs, int wg_size,
                     int iters, rocshmem_amd_stream_t stream);
/* The same with the tiles visited through a permutation when `scattered` is
 * nonzero: group g's i-th call moves the tile at slot ((i * odd) mod n_tiles)
 * of both buffers instead of slot i, so that the messages of neighbouring
 * lanes (or wavefronts) are far apart — the access pattern of the reference's
 * per-thread testers with random targets, as opposed to lanes that continue
 * one another (scripts/functional_tests/driver.sh:142-218 runs both
 * granularities over sizes from 1 B up).  Needs a power-of-two number of whole
 * tiles, else -1. */
int rocshmem_amd_rma_messages(int rma_op, int gran, void *dest, const void *source, size_t nbytes,
                              size_t tile_bytes, int scattered, int my_pe, int pe, int n_wgs,
                              int wg_size, int iters, rocshmem_amd_stream_t stream);

/* The same calls with the local buffer in LDS: one work-group stages `nbytes`
 * of `source` (a device buffer) in a __shared__ array, puts from there to
 * `dest` on `pe` (rocshmem_ctx_putmem[_wave|_wg] + quiet), gets the bytes back
 * from `pe` into a second __shared__ array at an odd offset, and copies that
 * array to `back` (a device buffer).  The reference copies through generic
 * pointers, so it accepts __shared__ and stack buffers on the local side
 * (src/util.hpp:170-262); nbytes <= ROCSHMEM_AMD_STAGED_MAX_BYTES. */
#define ROCSHMEM_AMD_STAGED_MAX_BYTES 24576
int rocshmem_amd_rma_staged(int gran, void *dest, const void *source, void *back, size_t nbytes,
                            int my_pe, int pe, int wg_size, rocshmem_amd_stream_t stream);

/* Work-group rank and size as the _wg calls compute them (the flat thread id
 * of the reference's get_flat_block_id / get_flat_block_size, src/util.hpp:100-118),
 * for a block of bx x by x bz threads: out_host[0] = the size seen by rank 0,
 * out_host[1 + r] = how many threads computed rank r, for r < 1024
 * (out_host holds 1026 words). */
int rocshmem_amd_flat_ids(int bx, int by, int bz, unsigned *out_host);
/* Host-initiated bulk copy between PEs over the whole GPU: the host-side
 * rocshmem_putmem / rocshmem_getmem (rocshmem_RMA.hpp; reference forwards them
 * to MPI_Put / MPI_Get, src/host/host_helpers.hpp:52-88). */
int rocshmem_amd_putmem(void *dest, const void *source, size_t nbytes, int my_pe, int pe,
                        rocshmem_amd_stream_t stream);
int rocshmem_amd_getmem(void *dest, const void *source, size_t nbytes, int my_pe, int pe,
                        rocshmem_amd_stream_t stream);

/* One wavefront whose lanes each make their own rocshmem_ctx_putmem call
 * (src/ipc/context_ipc_device.cpp:62-69 behind the coalescing front end,
 * src/wf_coal_policy.cpp:57-172): lane i, when bit i of active_mask is set,
 * puts size[i] bytes from source + src_off[i] to dest + dst_off[i] (a symmetric
 * address on my_pe) on PE pe[i].  Host arrays of 64 entries.  Waits for the
 * kernel. */
int rocshmem_amd_lane_puts(void *dest, const void *source, const int *pe, const uint64_t *src_off,
                           const uint64_t *dst_off, const uint64_t *size, uint64_t active_mask,
                           int my_pe, rocshmem_amd_stream_t stream);
/* wf_coal_policy coalesce (src/wf_coal_policy.cpp:57-172) on one wavefront:
 * lane i of the 64 is active iff bit i of active_mask; inputs are 64-entry
 * host arrays; outputs say whether the lane must send and its message size. */
int rocshmem_amd_wf_coalesce(const int *pe, const uint64_t *src, const uint64_t *dst,
                             const uint64_t *size, uint64_t active_mask, int *sends_out,
                             uint64_t *size_out);

/* ========================= collective drivers ============================== */

/* rocshmem_ctx_<T>_<op>_wg_reduce (rocshmem_COLL.hpp:348-598;
 * src/ipc/context_ipc_tmpl_device.hpp:361-418): one work-group per team member.
 * dest/source are the addresses on the member the host currently acts as
 * (which must belong to the team).  Returns the device status
 * (ROCSHMEM_SUCCESS 0 / ROCSHMEM_ERROR 1), after waiting for the kernel. */
int rocshmem_amd_wg_reduce(int dtype, int op, rocshmem_amd_team_t team, void *dest,
                           const void *source, int nreduce, int wg_size,
                           rocshmem_amd_stream_t stream);
/* The same call made by n_teams (<= 256) work-groups per PE at once, each with a
 * team of its own over the same PEs — how the reference's testers spread a
 * device collective over the GPU (one team per work-group,
 * tests/functional_tests/team_reduction_tester.cpp:60-110).  The arrays are
 * cut into equal slices of whole 16-byte vectors: with chunk_elems == 0 one
 * slice per team (team t reduces the t-th), otherwise slices of chunk_elems
 * elements dealt out in turn (team t reduces slices t, t + n_teams, ..., one
 * call each, so that at any moment the teams work side by side in one narrow
 * window of the arrays).  teams: host array of handles of distinct teams with
 * the same members.  Every work-group makes its calls `iters` (>= 1) times in
 * a row inside the kernel, as the reference's testers loop inside theirs.
 * Returns the largest device status any team saw, after waiting for the
 * kernel; -1 if nothing was launched (bad argument, or the grid n_teams x P
 * cannot be resident at once). */
int rocshmem_amd_wg_reduce_teams(int dtype, int op, const rocshmem_amd_team_t *teams, int n_teams,
                                 void *dest, const void *source, int nreduce, int chunk_elems,
                                 int wg_size, int iters, rocshmem_amd_stream_t stream);
/* rocshmem_amd_wg_reduce_teams for callers that cannot allocate device memory
 * (tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, same results; the per-team
 * status words, which rocshmem_amd_wg_reduce_teams allocates and frees on
 * every call, live in a fixed array inside the library's code object instead:
 * 256 words (1 KiB) per GPU, held until the process ends.  The call makes no
 * hipMalloc / hipFree; like its sibling it waits for the kernel and copies the
 * status words back, so it is not for code under stream capture.  n_teams
 * beyond 256 is refused with a message on stderr.  All calls on one GPU share
 * the array: once the arguments have been accepted it is cleared on the stream
 * before the launch, and two calls that overlap in time on one GPU race on it
 * (run them one after the other). */
int rocshmem_amd_wg_reduce_teams_static(int dtype, int op, const rocshmem_amd_team_t *teams,
                                        int n_teams, void *dest, const void *source, int nreduce,
                                        int chunk_elems, int wg_size, int iters,
                                        rocshmem_amd_stream_t stream);
/* The members' shares of one int32 sum all-reduce over the world team computed
 * by work-groups of different sizes in one launch: block k stands for member k
 * and works with lanes_per_member[k] (1..1024) lanes.  Runs the fold that
 * rocshmem_ctx_<T>_<op>_wg_reduce performs between its two barriers
 * (include/rocshmem/detail/reduce_engine.hpp); a test aid for the rule that a
 * member's share of the index range does not depend on work-group sizes.
 * dest / source: symmetric addresses on PE 0. */
int rocshmem_amd_fold_shares(void *dest, const void *source, int nreduce,
                             const int *lanes_per_member, rocshmem_amd_stream_t stream);
/* rocshmem_ctx_<T>_wg_alltoall / _wg_broadcast / _wg_fcollect
 * (rocshmem_COLL.hpp:44-258; context_ipc_tmpl_device.hpp:420-531).
 * elem_size in {1,2,4,8} selects the typed entry point (char/short/int/long). */
int rocshmem_amd_wg_alltoall(int elem_size, rocshmem_amd_team_t team, void *dest,
                             const void *source, int nelems, int wg_size,
                             rocshmem_amd_stream_t stream);
int rocshmem_amd_wg_broadcast(int elem_size, rocshmem_amd_team_t team, void *dest,
                              const void *source, int nelems, int pe_root, int wg_size,
                              rocshmem_amd_stream_t stream);
int rocshmem_amd_wg_fcollect(int elem_size, rocshmem_amd_team_t team, void *dest,
                             const void *source, int nelems, int wg_size,
                             rocshmem_amd_stream_t stream);
/* rocshmem_ctx_wg_barrier_all / _wg_sync_all / _wg_team_sync
 * (rocshmem.hpp:440-493; src/ipc/context_ipc_device_coll.cpp:31-123).
 * One work-group per PE runs `rounds` rounds of: put the round number into
 * the next member's `scratch` word, synchronise, check the word it received.
 * scratch: symmetric uint64.  Returns the number of wrong observations. */
int rocshmem_amd_wg_sync(int sync_fn, rocshmem_amd_team_t team, uint64_t *scratch,
                         int rounds, int wg_size, rocshmem_amd_stream_t stream);

/* Host-called all-reduce over an active set, all CUs:
 * rocshmem_ctx_<T>_<op>_to_all(ctx, dest, source, nreduce, PE_start,
 * logPE_stride, PE_size, pWrk, pSync) (src/rocshmem.cpp:724-735,974-980;
 * src/host/host_templates.hpp:333-376, in place when dest == source).
 * dest/source: addresses on PE PE_start. */
int rocshmem_amd_to_all(int dtype, int op, void *dest, const void *source, int nreduce,
                        int PE_start, int logPE_stride, int PE_size,
                        rocshmem_amd_stream_t stream);
/* Team form: host rocshmem_ctx_<T>_<op>_reduce (src/rocshmem.cpp:737-747). */
int rocshmem_amd_reduce(int dtype, int op, rocshmem_amd_team_t team, void *dest,
                        const void *source, int nreduce, rocshmem_amd_stream_t stream);
/* Host-called alltoall / broadcast / fcollect over a team, all CUs (byte
 * counts per team member).  broadcast: host rocshmem_ctx_<T>_broadcast
 * (rocshmem_COLL.hpp; src/host/host_templates.hpp:160-200). */
int rocshmem_amd_alltoallmem(rocshmem_amd_team_t team, void *dest, const void *source,
                             size_t nbytes, rocshmem_amd_stream_t stream);
int rocshmem_amd_broadcastmem(rocshmem_amd_team_t team, void *dest, const void *source,
                              size_t nbytes, int pe_root, rocshmem_amd_stream_t stream);
int rocshmem_amd_fcollectmem(rocshmem_amd_team_t team, void *dest, const void *source,
                             size_t nbytes, rocshmem_amd_stream_t stream);

/* ========================= host-side operations =========================== */

/* The __host__ halves of rocshmem_RMA.hpp / rocshmem_AMO.hpp /
 * rocshmem_P2P_SYNC.hpp, which the reference forwards to MPI one-sided calls
 * on a window over the heap (src/host/host.cpp:162-249).  The typed C++ names
 * (include/rocshmem/rocshmem_HOST.hpp) are inline wrappers over these.  All of
 * them are complete when they return.  They run on streams of the library's
 * own and are ordered with each other only — not with work the caller has
 * queued on HIP streams, which a host call therefore neither waits for nor
 * holds up (the reference's MPI traffic has no ordering with HIP streams
 * either): a kernel that is running may be waiting for just this put. */

/* PE a context handle belongs to (rocshmem_ctx_t::ctx_opaque, as filled in by
 * rocshmem_ctx_create or a driver); the acting PE for NULL; -1 if the pointer
 * is not a context of this runtime. */
int rocshmem_amd_ctx_pe(const void *ctx_opaque);
/* rocshmem_ctx_putmem / rocshmem_ctx_getmem called from the host
 * (rocshmem_RMA.hpp:237-242,618-623; src/host/host_helpers.hpp:52-88:
 * MPI_Put / MPI_Get + flush).  The symmetric side is given as my_pe's address
 * and resolved on `pe`; the local side may be host memory (pageable or pinned)
 * or device memory. */
int rocshmem_amd_host_putmem(void *dest, const void *source, size_t nbytes, int my_pe, int pe);
int rocshmem_amd_host_getmem(void *dest, const void *source, size_t nbytes, int my_pe, int pe);
/* One rocshmem_ctx_<T>_atomic_<op> called from the host (rocshmem_AMO.hpp;
 * src/host/host_templates.hpp:254-330: MPI_Fetch_and_op /
 * MPI_Compare_and_swap).  value / cond / fetched point at one element of
 * `dtype` in host memory (cond is read for compare_swap only; fetched may be
 * NULL). */
int rocshmem_amd_host_amo(int amo_op, int dtype, void *dest, const void *value, const void *cond,
                          int my_pe, int pe, void *fetched);
/* nbytes of device memory as they are now, read on a stream of the library's
 * own so that a kernel running on another stream does not hold the read back
 * (the reference reads its own window with MPI_Fetch_and_op(MPI_NO_OP),
 * src/host/host_templates.hpp:426-446). */
int rocshmem_amd_host_peek(void *dst_host, const void *src_dev, size_t nbytes);
/* rocshmem_<T>_test / _wait_until / _wait_until_any / _all / _some called from
 * the host (rocshmem_P2P_SYNC.hpp; src/host/host_templates.hpp:448-641).
 * ivars: device memory; status (may be NULL), value, indices_out, ret_out:
 * host memory.  ret_out: test -> 0/1, any -> index or SIZE_MAX, some -> count,
 * others -> 0.  timeout_ms < 0 waits for ever; otherwise the call gives up
 * after that long and returns 1. */
int rocshmem_amd_host_wait_test(int wait_fn, int dtype, const void *ivars, size_t nelems,
                                const int *status, int cmp, const void *value, long timeout_ms,
                                size_t *ret_out, size_t *indices_out);
/* Host rocshmem_ctx_<T>_broadcast over an active set (rocshmem_COLL.hpp:122-125;
 * src/host/host_templates.hpp:160-175): nbytes from the root's source to the
 * dest of every other member.  pe_root counts within the set.  dest/source:
 * addresses on PE_start. */
int rocshmem_amd_broadcast_active_set(void *dest, const void *source, size_t nbytes, int pe_root,
                                      int PE_start, int logPE_stride, int PE_size,
                                      rocshmem_amd_stream_t stream);

/* ====================== atomics, signals, waits ============================ */

/* rocshmem_<T>_atomic_<op> (rocshmem_AMO.hpp; src/ipc_policy.hpp:69-99).
 * `counters` is a symmetric array of n_slots elements (address on my_pe).
 * Operation i targets global counter ids[i] in [0, P*n_slots): PE
 * ids[i] / n_slots, element ids[i] % n_slots, with operand values[i]
 * (values == NULL: operand 1) and, for compare_swap, conds[i].  Fetching
 * operations store their result in fetched[i] (may be NULL).  ids, values,
 * conds, fetched are device arrays.  Thread t of the grid performs operations
 * t, t+T, t+2T ... */
int rocshmem_amd_amo(int amo_op, int dtype, void *counters, uint32_t n_slots,
                     const uint32_t *ids, const void *values, const void *conds,
                     void *fetched, size_t n_ops, int my_pe, int n_wgs, int wg_size,
                     rocshmem_amd_stream_t stream);

/* rocshmem_putmem_signal[_wave|_wg] (rocshmem_SIG_OP.hpp:27-228;
 * src/ipc/context_ipc_device.cpp:221-298).  Every group (thread / wavefront /
 * work-group per `gran`) of the grid acting for my_pe sends its tile of the
 * message (tiling as in rocshmem_amd_rma, one tile per group) and updates the
 * signal word on `pe`, `calls` times. */
int rocshmem_amd_put_signal(int gran, void *dest, const void *source, size_t nbytes,
                            uint64_t *sig_addr, uint64_t signal, int sig_op, int my_pe,
                            int pe, int n_wgs, int wg_size, int calls,
                            rocshmem_amd_stream_t stream);
/* rocshmem_signal_fetch[_wave|_wg] (rocshmem_SIG_OP.hpp:616-618): value read
 * by PE my_pe from its own word. */
int rocshmem_amd_signal_fetch(int gran, const uint64_t *sig_addr, int my_pe,
                              uint64_t *value_out);

/* A loop that polls with gets, and nothing else, must come to see a value that
 * another PE has put (OpenSHMEM forward progress; the reference's gets end in a
 * fence, src/ipc/context_ipc_device.cpp:71-78,146-154).  `pairs` (<= 128)
 * work-groups act for pe_a, each with a poller acting for pe_b.  Per round the
 * poller reads its own eight words once (so the old value is in its caches),
 * tells its partner, and then polls with rocshmem_ctx_uint64_g (kind 0),
 * rocshmem_ctx_getmem of the 64 bytes (1) or rocshmem_ctx_getmem_wave (2)
 * until the last word holds the round's number,
 * which the partner writes with rocshmem_ctx_uint64_p.  No wait_until, no
 * fence.  words: 8*pairs symmetric uint64, ready: pairs symmetric uint64
 * (addresses on pe_a).  Every wait is bounded: timed_out_out = 1 if one ran out
 * (all work-groups then leave). */
int rocshmem_amd_poll_with_gets(uint64_t *words, uint64_t *ready, int pairs, int rounds, int pe_a,
                                int pe_b, int kind, int wg_size, int *timed_out_out,
                                rocshmem_amd_stream_t stream);
/* Put, quiet, then raise a flag — the pattern quiet exists for (OpenSHMEM
 * message passing; rocshmem_ctx_quiet, include/rocshmem/rocshmem.hpp:408;
 * src/ipc/context_ipc_device.cpp:100-102) — with the receiver checking the
 * payload inside the same kernel.  `pairs` (<= 128) producer work-groups act
 * for pe_a, each with a receiver work-group acting for pe_b.  Per round a
 * producer fills a fresh pattern, calls rocshmem_ctx_putmem_wg of nbytes
 * (multiple of 4) into its slot of `data` on pe_b, calls rocshmem_ctx_quiet and
 * then sets its flag on pe_b with a relaxed store — or, with_signal == 1, does
 * all three with one rocshmem_ctx_putmem_signal_wg (rocshmem_SIG_OP.hpp:128-131);
 * with_signal == 2 / 3: the message goes out as several
 * rocshmem_ctx_putmem_nbi_wave calls per wavefront / rocshmem_ctx_putmem_nbi
 * calls of 12 bytes per thread, every thread calls rocshmem_ctx_quiet, and
 * thread 0 sets the flag after a work-group barrier; with_signal == 4 / 5: as
 * 0 / 1 with the pattern staged in the producer's LDS (nbytes <= 64 KiB), so
 * the put's local side is a __shared__ buffer;
 * the receiver waits for the flag, compares every word, and acknowledges.  data: pairs*nbytes symmetric bytes,
 * flags: 2*pairs symmetric uint64 (addresses on pe_a).  mismatches_out = words
 * that differed; timed_out_out = 1 if a bounded wait ran out (all work-groups
 * then leave). */
int rocshmem_amd_put_flag_check(void *data, uint64_t *flags, size_t nbytes, int pairs, int rounds,
                                int pe_a, int pe_b, int wg_size, int with_signal,
                                uint64_t *mismatches_out, int *timed_out_out,
                                rocshmem_amd_stream_t stream);

/* Ping-pong (tests/functional_tests/ping_pong_tester.cpp:43-61,
 * examples/rocshmem_put_signal_test.cc:31-47; the reference runs it with 1, 8
 * and 32 work-groups, scripts/functional_tests/driver.sh:313-315): `pairs`
 * (<= 128) pairs of work-groups at once, the even one of a pair acting for
 * pe_a, the odd one for pe_b; `iters` round trips of putmem_signal_wg (payload
 * nbytes from the pair's slot of `buf` to the same slot on the peer, the
 * pair's word of `sig` set to the round number) answered after
 * rocshmem_ulong_wait_until.  Slots are nbytes rounded up to 256 bytes apart;
 * sig holds `pairs` words.  buf/sig: addresses on pe_a.  ticks_out (host,
 * optional) receives the wall_clock64 ticks the slowest pair's pe_a side
 * spent; tick_hz_out the tick rate. */
int rocshmem_amd_pingpong(void *buf, uint64_t *sig, size_t nbytes, int iters, int pairs,
                          int pe_a, int pe_b, int wg_size, uint64_t *ticks_out,
                          double *tick_hz_out, rocshmem_amd_stream_t stream);

/* MoE-style dispatch with put_signal.  For every ordered pair (s, d) of the P
 * world PEs, rows [send_row[s*P+d], +count[s*P+d]) of s's `send` buffer go to
 * rows starting at recv_row[s*P+d] of d's `recv` buffer, rows_per_call rows per
 * rocshmem_putmem_signal_wg call, each call adding the number of rows it sent
 * to d's sig[s]; work-groups acting for the sources share out the list of all
 * calls, and one more work-group per PE d waits with
 * rocshmem_ulong_wait_until(sig[s], GE, count[s*P+d]) for every s.
 * count/send_row/recv_row: host arrays of P*P uint32 (a device copy is kept
 * and reused while consecutive calls pass the same tables).  send/recv/sig:
 * addresses on PE 0.
 * expect == NULL: sig must be zero when the kernel starts.  Otherwise expect is
 * P*P uint64 of device memory that the caller zeroes once together with sig:
 * the receivers keep in expect[d*P+s] the total they have waited for on d's
 * word s and wait for that total plus this dispatch's count, so the signal
 * words just keep growing and one dispatch follows the other with nothing to
 * clear in between (how an application that dispatches every step uses
 * ROCSHMEM_SIGNAL_ADD with rocshmem_wait_until(..., GE, running total),
 * examples/rocshmem_put_signal_test.cc:31-47). */
int rocshmem_amd_dispatch_put_signal(void *recv, const void *send, uint64_t *sig,
                                     const uint32_t *count, const uint32_t *send_row,
                                     const uint32_t *recv_row, size_t row_bytes,
                                     int rows_per_call, int wg_size, uint64_t *expect,
                                     rocshmem_amd_stream_t stream);

/* rocshmem_<T>_test / _wait_until / _wait_until_any / _all / _some
 * (rocshmem_P2P_SYNC.hpp:44-556; src/context_tmpl_device.hpp:201-377) called
 * by one thread on the device array ivars (nelems elements of dtype); `value`
 * points at one host element of dtype.  ret_out: the function's return value
 * (test: 0/1; any: index or SIZE_MAX; some: count; others 0); indices_out
 * (host, nelems entries, optional) receives wait_until_some's indices.
 * A blocking form whose condition does not hold yet would spin for ever (there
 * is nobody to change ivars): it is refused with -2 and nothing is launched;
 * use the waker below for those. */
int rocshmem_amd_wait_test(int wait_fn, int dtype, void *ivars, size_t nelems,
                           const int *status, int cmp, const void *value,
                           size_t *ret_out, size_t *indices_out);
/* Same call made by work-group 0 while work-group 1 stores `wake_value` into
 * ivars[wake_index] after roughly delay_ticks wall-clock ticks. */
int rocshmem_amd_wait_test_woken(int wait_fn, int dtype, void *ivars, size_t nelems,
                                 const int *status, int cmp, const void *value,
                                 size_t wake_index, const void *wake_value,
                                 uint64_t delay_ticks, size_t *ret_out,
                                 size_t *indices_out);

/* A device-side wait with an end, for checking that something the HOST does
 * while a kernel runs reaches that kernel: one thread polls
 * rocshmem_<T>_test(ivar, cmp, value) (rocshmem_P2P_SYNC.hpp) up to max_polls
 * times.  Only enqueues.  result_dev (device memory, 2 x uint64): [0] = 1 if
 * the condition was seen, 0 if the polls ran out; [1] = polls made. */
int rocshmem_amd_poll_until(int dtype, void *ivar, int cmp, const void *value, uint64_t max_polls,
                            uint64_t *result_dev, rocshmem_amd_stream_t stream);

/* Context lifecycle (rocshmem.hpp:334-370; src/rocshmem_gpu.cpp:286-325): each
 * of n_wgs work-groups creates per_wg contexts (rocshmem_wg_ctx_create, or
 * rocshmem_wg_team_create_ctx when team != NULL), records each return code in
 * status_out[wg*per_wg + k] and the context's rocshmem_ctx_my_pe / n_pes in
 * pe_out / npes_out (host arrays), then destroys them all. */
int rocshmem_amd_ctx_cycle(rocshmem_amd_team_t team, int n_wgs, int wg_size, int per_wg,
                           int *status_out, int *pe_out, int *npes_out);

#ifdef __cplusplus
}
#endif

#endif /* ROCSHMEM_AMD_H_ */
