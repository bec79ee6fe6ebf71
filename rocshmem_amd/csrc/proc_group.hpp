// One process per PE: how the processes of a job find each other and meet.
//
// The reference starts one process per PE under an MPI launcher and uses MPI
// for its bootstrap and its host-side barriers (src/ipc_policy.cpp:34-118,
// src/ipc/backend_ipc.cpp:274-357 exchange the heaps' IPC handles with
// MPI_Allgather).  Here the launcher (rocshmem_amd/launch.py) creates one
// zero-filled file in shared memory and hands every process its path, the
// number of processes and its rank through the environment; the file holds a
// publish area per rank (IPC handles travel through it) and a table of
// barriers keyed by PE set.  Nothing in this file touches the GPU, so the
// logic is tested on the CPU.
#ifndef ROCSHMEM_AMD_PROC_GROUP_HPP_
#define ROCSHMEM_AMD_PROC_GROUP_HPP_

#include <atomic>
#include <cstddef>
#include <cstdint>

namespace rocshmem {
namespace runtime {

constexpr int kMaxProcs = 64;
constexpr size_t kBlobBytes = 192;
constexpr int kBarrierSlots = 128;

// What the shared file holds.  All-zero is its valid initial state.
struct ProcShared {
  std::atomic<uint32_t> attached;  // processes that have mapped the file
  std::atomic<int32_t> abort_status_plus_one;  // nonzero once a process asked the whole job to end
  uint32_t pad_[14];
  struct Barrier {
    std::atomic<uint64_t> key;    // 0 = free; else the PE set (start, stride, size)
    std::atomic<uint32_t> count;  // arrivals of the current round
    std::atomic<uint32_t> round;  // completed rounds
  } barriers[kBarrierSlots];
  struct Blob {
    std::atomic<uint64_t> version;  // bumped after every publish
    unsigned char bytes[kBlobBytes];
  } blobs[kMaxProcs];
};

class ProcGroup {
 public:
  // Reads ROCSHMEM_EMU_PROCS / _RANK / _RDV and maps the file; false when the
  // process was not started as one PE of a job (no variables).  Problems with
  // the variables or the file end the process with a message.
  bool attach_from_env();
  // The same with explicit arguments; 0 on success, -1 on a bad argument or file.
  int attach(const char *path, int nprocs, int rank);
  void detach();

  bool active() const { return shared_ != nullptr; }
  int nprocs() const { return nprocs_; }
  int rank() const { return rank_; }

  // Meets the other members of the strided PE set; every member must call with
  // the same set.  Returns 0, or -1 when the wait ran out (timeout_s) or
  // another process has asked the job to end (callers then leave).
  int barrier(int start, int stride, int size);
  int barrier_world() { return barrier(0, 1, nprocs_); }

  // A rank's publish area: write own, read anybody's (after a barrier).
  int publish(const void *bytes, size_t n);
  int fetch(int rank, void *bytes, size_t n) const;

  // Asks every process of the job to end with `status` at its next meeting.
  void request_abort(int status);
  // Status another process asked the job to end with, or -1.
  int abort_requested() const;

  double timeout_s = 120.0;

 private:
  ProcShared *shared_ = nullptr;
  int nprocs_ = 0;
  int rank_ = -1;
};

ProcGroup &procs();

}  // namespace runtime
}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_PROC_GROUP_HPP_
