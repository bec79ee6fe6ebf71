/* Measuring probes of the MI355X symmetric-heap library's benchmark
 * (librocshmem_amd_probes.so): yardsticks that the data path of
 * librocshmem_amd.so is read against.  They are not part of that library's
 * interface and have no counterpart in the reference; the runtime must have
 * been brought up through rocshmem_amd_init.  Return value 0 = launched,
 * negative = argument error (nothing launched). */
#ifndef ROCSHMEM_AMD_PROBES_H_
#define ROCSHMEM_AMD_PROBES_H_

#include "rocshmem_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Reads (write == 0) or overwrites
 * (write != 0) nbytes (>= 1 MiB, 16-byte aligned) of device memory with the
 * whole GPU, with the load and store instructions of the bulk copy, and nothing
 * else — the one-directional rate of the memory system that a copy is judged
 * against. */
int rocshmem_amd_hbm_probe(int write, void *buf, size_t nbytes, rocshmem_amd_stream_t stream);
/* What one agent-scope release —
 * the L2 write-back that rocshmem_ctx_quiet / fence and every barrier perform
 * on a default context — costs while a copy is running.  n_wgs work-groups of
 * wg_size threads copy nbytes from src to dst in tiles of tile_bytes (tile t
 * to work-group t mod n_wgs) with the cooperative copy of putmem_wg and issue a
 * release never (mode 0), once per work-group at its end (mode 1) or after
 * every tile (mode 2).  Time modes 1 / 2 against mode 0 and divide by the
 * number of releases. */
int rocshmem_amd_release_probe(int mode, void *dst, const void *src, size_t nbytes,
                               size_t tile_bytes, int n_wgs, int wg_size,
                               rocshmem_amd_stream_t stream);
/* What a consumer that re-reads received data gets from the caches: n_wgs
 * work-groups of wg_size threads read nbytes (16-byte aligned) in tiles of
 * tile_bytes (multiple of 16; tile t to work-group t mod n_wgs), each tile
 * `passes` times in a row.  On cached memory the later passes hit the L2; on
 * an uncached symmetric heap every pass goes to memory.  Time it and divide
 * passes * nbytes by the time. */
int rocshmem_amd_reuse_probe(const void *buf, size_t nbytes, size_t tile_bytes, int passes,
                             int n_wgs, int wg_size, rocshmem_amd_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* ROCSHMEM_AMD_PROBES_H_ */
