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
//   * A work-group learns its PE from its context.  Contexts made by
//     rocshmem_wg_team_create_ctx take the PE of the team object; the default
//     context and rocshmem_wg_ctx_create use the rule chosen with
//     rocshmem_emu_set_pe_rule (fixed acting PE, or blockIdx.{x,y,z} mod P).
#ifndef ROCSHMEM_AMD_EMU_HPP_
#define ROCSHMEM_AMD_EMU_HPP_

#include <cstddef>

#include "rocshmem_common.hpp"

namespace rocshmem {

enum rocshmem_emu_pe_rule {
  ROCSHMEM_EMU_PE_FIXED = 0,
  ROCSHMEM_EMU_PE_BLOCK_X = 1,
  ROCSHMEM_EMU_PE_BLOCK_Y = 2,
  ROCSHMEM_EMU_PE_BLOCK_Z = 3
};

void rocshmem_emu_set_npes(int npes);
void rocshmem_emu_set_pe(int pe);
void rocshmem_emu_set_pe_rule(int rule);
// Address of the symmetric object `ptr` (any PE's address of it) on PE `pe`.
void *rocshmem_emu_pe_ptr(const void *ptr, int pe);
// Handle of the same team as seen by PE `pe` (ROCSHMEM_TEAM_INVALID when that
// PE is not a member).
rocshmem_team_t rocshmem_emu_team_on(rocshmem_team_t team, int pe);
// Bytes between the slices of consecutive PEs.
size_t rocshmem_emu_pe_stride();

}  // namespace rocshmem

#endif  // ROCSHMEM_AMD_EMU_HPP_
