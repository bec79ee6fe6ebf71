/* The few MPI names that programs written for the reference use around the
 * rocSHMEM calls (its launcher is mpirun: rocshmem_init takes an MPI_Comm,
 * tests call MPI_Barrier and MPI_Abort), for builds without an MPI
 * installation.  No message passing happens here: the "communicator" is the
 * set of all PEs, whether they are threads of this process or the processes
 * of a job started by rocshmem_amd.launch, and a barrier is the library's own
 * host meeting.  Put this directory on the include path to
 * satisfy `#include <mpi.h>`; rocshmem.hpp pulls it in by itself when no real
 * mpi.h is found. */
#ifndef ROCSHMEM_AMD_COMPAT_MPI_H_
#define ROCSHMEM_AMD_COMPAT_MPI_H_

#include <stdio.h>
#include <stdlib.h>

#include "../../rocshmem_amd.h"

typedef int MPI_Comm;
#ifndef MPI_COMM_WORLD
#define MPI_COMM_WORLD 0
#endif
#ifndef MPI_COMM_NULL
#define MPI_COMM_NULL (-1)
#endif
#ifndef MPI_SUCCESS
#define MPI_SUCCESS 0
#endif
#define MPI_THREAD_SINGLE 0
#define MPI_THREAD_FUNNELED 1
#define MPI_THREAD_SERIALIZED 2
#define MPI_THREAD_MULTIPLE 3

static inline int MPI_Init(int *, char ***) { return MPI_SUCCESS; }
static inline int MPI_Init_thread(int *, char ***, int, int *provided) {
  if (provided) *provided = MPI_THREAD_MULTIPLE;
  return MPI_SUCCESS;
}
static inline int MPI_Initialized(int *flag) {
  *flag = 1;
  return MPI_SUCCESS;
}
static inline int MPI_Finalize(void) { return MPI_SUCCESS; }
static inline int MPI_Comm_rank(MPI_Comm, int *rank) {
  *rank = rocshmem_amd_my_pe();
  return MPI_SUCCESS;
}
static inline int MPI_Comm_size(MPI_Comm, int *size) {
  *size = rocshmem_amd_n_pes();
  return MPI_SUCCESS;
}
/* Every PE thread, or every process of the job, arrives; otherwise there is
 * nobody to wait for. */
static inline int MPI_Barrier(MPI_Comm) {
  const int n = rocshmem_amd_n_pes();
  if (rocshmem_amd_procs_count() > 0) {
    if (rocshmem_amd_procs_barrier(0, 1, n) != 0) {
      const int asked = rocshmem_amd_procs_abort_requested();
      fflush(NULL);
      _Exit(asked >= 0 ? asked : EXIT_FAILURE);
    }
    return MPI_SUCCESS;
  }
  if (rocshmem_amd_pe_threads_enter(0, 1, n)) rocshmem_amd_pe_threads_leave(0, 1, n);
  return MPI_SUCCESS;
}
/* Programs written for the reference end a failed run with MPI_Abort; the
 * other processes of a job leave at their next meeting. */
static inline int MPI_Abort(MPI_Comm, int errorcode) {
  fflush(NULL);
  if (rocshmem_amd_procs_count() > 0) rocshmem_amd_procs_request_abort(errorcode);
  _Exit(errorcode);
  return MPI_SUCCESS;
}

#endif /* ROCSHMEM_AMD_COMPAT_MPI_H_ */
