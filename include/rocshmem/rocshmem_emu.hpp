// Controls for hosting all P processing elements in one process on one GPU.
// These have no counterpart in the reference, where P comes from the MPI
// launcher and each process is one PE.
//
//   * P is rocshmem_emu_set_npes(P) before rocshmem_init(), else the
//     ROCSHMEM_EMU_NPES environment variable, else 1.
//   * The host thread acts as one PE at a time (rocshmem_emu_set_pe);
//     rocshmem_my_pe(), rocshmem_malloc() and team handles are reported for
//     that PE.  rocshmem_malloc() allocates the object on every PE at once
//     and returns the acting PE's address.
//   * Or every PE gets a host thread of its own: rocshmem_emu_run_pes(P, fn,
//     argc, argv) runs fn once per PE, each in its own thread, and inside them
//     the host API behaves as it does in the reference's one-process-per-PE
//     programs: rocshmem_my_pe() is the thread's PE, rocshmem_init / malloc /
//     free / barrier_all / team_split_strided / broadcast / reduce are
//     collective calls that every member makes.  A program written for the
//     reference runs that way unchanged when it is compiled with
//     -DROCSHMEM_EMU_PE_THREADS_MAIN: its main() becomes the per-PE function
//     (single translation unit; P from ROCSHMEM_EMU_NPES).  File-scope
//     variables of such a program are shared by all PEs.
//   * A work-group learns its PE from its context.  Contexts made by
//     rocshmem_wg_team_create_ctx take the PE of the team object; the default
//     context and rocshmem_wg_ctx_create use the rule chosen with
//     rocshmem_emu_set_pe_rule (fixed acting PE, or blockIdx.{x,y,z} mod P).
#ifndef ROCSHMEM_AMD_EMU_HPP_
#define ROCSHMEM_AMD_EMU_HPP_

#include <hip/hip_runtime.h>

#include <cstddef>

#include "rocshmem_common.hpp"

namespace rocshmem {

enum rocshmem_emu_pe_rule {
  ROCSHMEM_EMU_PE_FIXED = 0,
  ROCSHMEM_EMU_PE_BLOCK_X = 1,
  ROCSHMEM_EMU_PE_BLOCK_Y = 2,
  ROCSHMEM_EMU_PE_BLOCK_Z = 3,
  ROCSHMEM_EMU_PE_QUEUE = 4  // the PE thread that bound the kernel's queue (the rule in PE threads)
};

// Runs pe_main(argc, argv) in npes threads (npes <= 0: ROCSHMEM_EMU_NPES), one
// per PE, before the runtime is up; returns the first non-zero result.
int rocshmem_emu_run_pes(int npes, int (*pe_main)(int, char **), int argc, char **argv);
// In a PE thread: makes kernels launched on `stream` from now on act as this
// thread's PE when they use the default context or rocshmem_wg_ctx_create
// (a one-thread kernel on the stream records the hardware queue it runs on).
// Each PE thread needs streams, and hardware queues, of its own
// (GPU_MAX_HW_QUEUES at least the number of streams in use).  Compiling with
// -DROCSHMEM_EMU_PE_THREADS makes hipLaunchKernelGGL call this by itself.
void rocshmem_emu_bind_stream(hipStream_t stream);
// In a PE thread: waits for the streams this thread has bound, i.e. for this
// PE's own device work, as hipDeviceSynchronize does in a process that is one
// PE.  -DROCSHMEM_EMU_PE_THREADS makes hipDeviceSynchronize() mean this.
hipError_t rocshmem_emu_device_synchronize();
// Tells the library that the program was built with
// -fgpu-default-stream=per-thread, so that rocshmem_init binds each PE
// thread's own default stream.  Called by itself in such builds (below).
void rocshmem_emu_per_thread_default_stream();
void rocshmem_emu_set_npes(int npes);
void rocshmem_emu_set_pe(int pe);
void rocshmem_emu_set_pe_rule(int rule);
// Address of the symmetric object `ptr` (any PE's address of it) on PE `pe`.
void *rocshmem_emu_pe_ptr(const void *ptr, int pe);
// Handle of the same team as seen by PE `pe` (ROCSHMEM_TEAM_INVALID when that
// PE is not a member).
rocshmem_team_t rocshmem_emu_team_on(rocshmem_team_t team, int pe);
// Bytes between the slices of consecutive PEs; 0 in a process that is one PE of
// a job of processes (the slices are separate mappings: use rocshmem_emu_pe_ptr).
size_t rocshmem_emu_pe_stride();

}  // namespace rocshmem

#if (defined(ROCSHMEM_EMU_PE_THREADS) || defined(ROCSHMEM_EMU_PE_THREADS_MAIN)) && \
    defined(HIP_API_PER_THREAD_DEFAULT_STREAM)
namespace rocshmem {
namespace detail {
__attribute__((used)) static const int per_thread_default_stream_announced_ =
    (rocshmem_emu_per_thread_default_stream(), 0);
}  // namespace detail
}  // namespace rocshmem
#endif

#if defined(ROCSHMEM_EMU_PE_THREADS) || defined(ROCSHMEM_EMU_PE_THREADS_MAIN)
// hipDeviceSynchronize() covers the calling PE's work only (the other PEs'
// kernels may be waiting for one this thread has yet to launch), and every
// hipLaunchKernelGGL first binds its stream to the launching PE thread.
#define hipDeviceSynchronize() ::rocshmem::rocshmem_emu_device_synchronize()
#undef hipLaunchKernelGGLInternal
#define hipLaunchKernelGGLInternal(kernelName, numBlocks, numThreads, memPerBlock, streamId, ...) \
  do {                                                                                            \
    ::rocshmem::rocshmem_emu_bind_stream(streamId);                                               \
    kernelName<<<(numBlocks), (numThreads), (memPerBlock), (streamId)>>>(__VA_ARGS__);            \
  } while (0)
#endif

#if defined(ROCSHMEM_EMU_PE_THREADS_MAIN)
// The program's own main, under another name, in whichever of the usual
// forms it was written.
int rocshmem_emu_pe_main(int argc, char **argv, char **envp) __attribute__((weak));
int rocshmem_emu_pe_main(int argc, char **argv) __attribute__((weak));
int rocshmem_emu_pe_main() __attribute__((weak));
extern char **environ;
int main(int argc, char **argv) {
  return rocshmem::rocshmem_emu_run_pes(
      0,
      [](int c, char **v) -> int {
        int (*with_env)(int, char **, char **) = rocshmem_emu_pe_main;
        int (*with_args)(int, char **) = rocshmem_emu_pe_main;
        int (*without_args)() = rocshmem_emu_pe_main;
        if (with_env) return with_env(c, v, environ);
        return with_args ? with_args(c, v) : without_args();
      },
      argc, argv);
}
#define main rocshmem_emu_pe_main
#endif

#endif  // ROCSHMEM_AMD_EMU_HPP_
