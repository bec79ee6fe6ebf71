/* Build configuration of this library: the intra-node load/store ("IPC")
 * data path over a coherent, single-node symmetric heap — the one
 * configuration the reference supports (scripts/build_configs/ipc_single). */
#ifndef ROCSHMEM_AMD_CONFIG_H_
#define ROCSHMEM_AMD_CONFIG_H_
#define USE_IPC 1
#define USE_COHERENT_HEAP 1
#define USE_SINGLE_NODE 1
#define ROCSHMEM_AMD_EMULATED_PES 1
#endif
