"""ctypes binding of ``librocshmem_amd.so`` (declarations: include/rocshmem_amd.h)."""

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librocshmem_amd.so")

# Enumerations of include/rocshmem_amd.h.
(SHORT, INT, LONG, LONGLONG, FLOAT, DOUBLE, BF16, UINT, ULONG, ULONGLONG, CHAR, SCHAR, UCHAR,
 USHORT) = range(14)
SUM, MAX, MIN, PROD, AND, OR, XOR = range(7)
THREAD, WAVE, WG = range(3)
PUT, GET, PUT_NBI, GET_NBI = range(4)
(AMO_FETCH_ADD, AMO_ADD, AMO_FETCH_INC, AMO_INC, AMO_COMPARE_SWAP, AMO_FETCH, AMO_SET,
 AMO_SWAP, AMO_FETCH_AND, AMO_FETCH_OR, AMO_FETCH_XOR) = range(11)
CTX_NOSTORE = 1  # ROCSHMEM_CTX_NOSTORE
TEST, WAIT_UNTIL, WAIT_UNTIL_ANY, WAIT_UNTIL_ALL, WAIT_UNTIL_SOME = range(5)
BARRIER_ALL, SYNC_ALL, TEAM_SYNC = range(3)
CMP_EQ, CMP_NE, CMP_GT, CMP_GE, CMP_LT, CMP_LE = range(6)
SIGNAL_SET, SIGNAL_ADD = range(2)
SIZE_MAX = (1 << 64) - 1

_vp, _sz, _i, _u32, _u64 = C.c_void_p, C.c_size_t, C.c_int, C.c_uint32, C.c_uint64

# name -> (restype, argtypes); every symbol the header declares.
SIGNATURES = {
    "rocshmem_amd_init": (_i, [_i, _sz]),
    "rocshmem_amd_finalize": (_i, []),
    "rocshmem_amd_n_pes": (_i, []),
    "rocshmem_amd_my_pe": (_i, []),
    "rocshmem_amd_set_pe": (_i, [_i]),
    "rocshmem_amd_set_pe_rule": (_i, [_i]),
    "rocshmem_amd_set_ctx_options": (C.c_int64, [C.c_int64]),
    "rocshmem_amd_set_coalesce_puts": (_i, [_i]),
    "rocshmem_amd_procs_file_bytes": (_sz, []),
    "rocshmem_amd_procs_count": (_i, []),
    "rocshmem_amd_procs_attach": (_i, [C.c_char_p, _i, _i]),
    "rocshmem_amd_procs_barrier": (_i, [_i, _i, _i]),
    "rocshmem_amd_procs_publish": (_i, [_vp, _sz]),
    "rocshmem_amd_procs_fetch": (_i, [_i, _vp, _sz]),
    "rocshmem_amd_procs_request_abort": (_i, [_i]),
    "rocshmem_amd_procs_abort_requested": (_i, []),
    "rocshmem_amd_set_spin_limit": (_i, [_u64]),
    "rocshmem_amd_waits_given_up": (C.c_int64, [_i]),
    "rocshmem_amd_malloc": (_vp, [_sz]),
    "rocshmem_amd_free": (_i, [_vp]),
    "rocshmem_amd_barrier_all": (_i, []),
    "rocshmem_amd_pe_ptr": (_vp, [_vp, _i]),
    "rocshmem_amd_heap_size": (_sz, []),
    "rocshmem_amd_heap_used": (_sz, []),
    "rocshmem_amd_heap_avail": (_sz, []),
    "rocshmem_amd_pe_stride": (_sz, []),
    "rocshmem_amd_heap_alloc_bytes": (_sz, []),
    "rocshmem_amd_heap_is_uncached": (_i, []),
    "rocshmem_amd_heap_held": (_i, [C.POINTER(_sz), C.POINTER(_sz)]),
    "rocshmem_amd_coresident": (_i, [C.c_long, _i, _i]),
    "rocshmem_amd_hw_queues_suffice": (_i, [_sz, _sz]),
    "rocshmem_amd_heap_model_create": (_vp, [_u64, _u64]),
    "rocshmem_amd_heap_model_destroy": (None, [_vp]),
    "rocshmem_amd_heap_model_alloc": (_u64, [_vp, _u64]),
    "rocshmem_amd_heap_model_free": (_i, [_vp, _u64]),
    "rocshmem_amd_heap_model_used": (_u64, [_vp]),
    "rocshmem_amd_heap_model_num_bins": (_u64, [_vp]),
    "rocshmem_amd_heap_model_bin_population": (_u64, [_vp, _u64]),
    "rocshmem_amd_team_world": (_vp, []),
    "rocshmem_amd_team_split_strided": (_i, [_vp, _i, _i, _i, C.POINTER(_vp)]),
    "rocshmem_amd_team_destroy": (None, [_vp]),
    "rocshmem_amd_team_n_pes": (_i, [_vp]),
    "rocshmem_amd_team_my_pe": (_i, [_vp]),
    "rocshmem_amd_team_translate_pe": (_i, [_vp, _i, _vp]),
    "rocshmem_amd_team_on": (_vp, [_vp, _i]),
    "rocshmem_amd_team_active_set": (_i, [_vp, C.POINTER(_i), C.POINTER(_i), C.POINTER(_i)]),
    "rocshmem_amd_pe_threads_enter": (_i, [_i, _i, _i]),
    "rocshmem_amd_pe_threads_leave": (None, [_i, _i, _i]),
    "rocshmem_amd_dev_mem_info": (_i, [C.POINTER(_sz), C.POINTER(_sz)]),
    "rocshmem_amd_dev_alloc": (_vp, [_sz]),
    "rocshmem_amd_dev_free": (_i, [_vp]),
    "rocshmem_amd_copy_in": (_i, [_vp, _vp, _sz]),
    "rocshmem_amd_copy_out": (_i, [_vp, _vp, _sz]),
    "rocshmem_amd_fill": (_i, [_vp, _i, _sz]),
    "rocshmem_amd_compare": (_i, [_vp, _vp, _sz, C.POINTER(_u64), _vp]),
    "rocshmem_amd_fill_every_pe": (_i, [_vp, _i, _sz, _vp]),
    "rocshmem_amd_copy_dev": (_i, [_vp, _vp, _sz]),
    "rocshmem_amd_stream_sync": (_i, [_vp]),
    "rocshmem_amd_timer_create": (_vp, []),
    "rocshmem_amd_timer_start": (_i, [_vp, _vp]),
    "rocshmem_amd_timer_stop": (_i, [_vp, _vp]),
    "rocshmem_amd_timer_elapsed_ms": (C.c_float, [_vp]),
    "rocshmem_amd_timer_destroy": (_i, [_vp]),
    "rocshmem_amd_rma": (_i, [_i, _i, _vp, _vp, _sz, _sz, _i, _i, _i, _i, _i, _vp]),
    "rocshmem_amd_rma_messages": (_i, [_i, _i, _vp, _vp, _sz, _sz, _i, _i, _i, _i, _i, _i, _vp]),
    "rocshmem_amd_rma_staged": (_i, [_i, _vp, _vp, _vp, _sz, _i, _i, _i, _vp]),
    "rocshmem_amd_flat_ids": (_i, [_i, _i, _i, _vp]),
    "rocshmem_amd_ctx_pe": (_i, [_vp]),
    "rocshmem_amd_host_putmem": (_i, [_vp, _vp, _sz, _i, _i]),
    "rocshmem_amd_host_getmem": (_i, [_vp, _vp, _sz, _i, _i]),
    "rocshmem_amd_host_amo": (_i, [_i, _i, _vp, _vp, _vp, _i, _i, _vp]),
    "rocshmem_amd_host_peek": (_i, [_vp, _vp, _sz]),
    "rocshmem_amd_host_wait_test": (_i, [_i, _i, _vp, _sz, _vp, _i, _vp, C.c_long,
                                         C.POINTER(_sz), _vp]),
    "rocshmem_amd_broadcast_active_set": (_i, [_vp, _vp, _sz, _i, _i, _i, _i, _vp]),
    "rocshmem_amd_poll_with_gets": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, C.POINTER(_i), _vp]),
    "rocshmem_amd_put_flag_check": (_i, [_vp, _vp, _sz, _i, _i, _i, _i, _i, _i,
                                         C.POINTER(_u64), C.POINTER(_i), _vp]),
    "rocshmem_amd_putmem": (_i, [_vp, _vp, _sz, _i, _i, _vp]),
    "rocshmem_amd_getmem": (_i, [_vp, _vp, _sz, _i, _i, _vp]),
    "rocshmem_amd_lane_puts": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _u64, _i, _vp]),
    "rocshmem_amd_wf_coalesce": (_i, [_vp, _vp, _vp, _vp, _u64, _vp, _vp]),
    "rocshmem_amd_wg_reduce": (_i, [_i, _i, _vp, _vp, _vp, _i, _i, _vp]),
    "rocshmem_amd_wg_reduce_teams": (_i, [_i, _i, C.POINTER(_vp), _i, _vp, _vp, _i, _i, _i, _i, _vp]),
    "rocshmem_amd_wg_reduce_teams_static": (_i, [_i, _i, C.POINTER(_vp), _i, _vp, _vp, _i, _i, _i,
                                                 _i, _vp]),
    "rocshmem_amd_fold_shares": (_i, [_vp, _vp, _i, C.POINTER(_i), _vp]),
    "rocshmem_amd_wg_alltoall": (_i, [_i, _vp, _vp, _vp, _i, _i, _vp]),
    "rocshmem_amd_wg_broadcast": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "rocshmem_amd_wg_fcollect": (_i, [_i, _vp, _vp, _vp, _i, _i, _vp]),
    "rocshmem_amd_wg_sync": (_i, [_i, _vp, _vp, _i, _i, _vp]),
    "rocshmem_amd_to_all": (_i, [_i, _i, _vp, _vp, _i, _i, _i, _i, _vp]),
    "rocshmem_amd_reduce": (_i, [_i, _i, _vp, _vp, _vp, _i, _vp]),
    "rocshmem_amd_alltoallmem": (_i, [_vp, _vp, _vp, _sz, _vp]),
    "rocshmem_amd_broadcastmem": (_i, [_vp, _vp, _vp, _sz, _i, _vp]),
    "rocshmem_amd_fcollectmem": (_i, [_vp, _vp, _vp, _sz, _vp]),
    "rocshmem_amd_amo": (_i, [_i, _i, _vp, _u32, _vp, _vp, _vp, _vp, _sz, _i, _i, _i, _vp]),
    "rocshmem_amd_put_signal": (_i, [_i, _vp, _vp, _sz, _vp, _u64, _i, _i, _i, _i, _i, _i, _vp]),
    "rocshmem_amd_signal_fetch": (_i, [_i, _vp, _i, C.POINTER(_u64)]),
    "rocshmem_amd_pingpong": (_i, [_vp, _vp, _sz, _i, _i, _i, _i, _i, C.POINTER(_u64),
                                   C.POINTER(C.c_double), _vp]),
    "rocshmem_amd_dispatch_put_signal": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _i, _i, _vp, _vp]),
    "rocshmem_amd_wait_test": (_i, [_i, _i, _vp, _sz, _vp, _i, _vp, C.POINTER(_sz), _vp]),
    "rocshmem_amd_wait_test_woken": (_i, [_i, _i, _vp, _sz, _vp, _i, _vp, _sz, _vp, _u64,
                                          C.POINTER(_sz), _vp]),
    "rocshmem_amd_poll_until": (_i, [_i, _vp, _i, _vp, _u64, _vp, _vp]),
    "rocshmem_amd_ctx_cycle": (_i, [_vp, _i, _i, _i, _vp, _vp, _vp]),
}


# The benchmark's measuring probes (include/rocshmem_amd_probes.h), a library of
# their own next to the product.
PROBES_PATH = os.path.join(_HERE, "lib", "librocshmem_amd_probes.so")
PROBE_SIGNATURES = {
    "rocshmem_amd_hbm_probe": (_i, [_i, _vp, _sz, _vp]),
    "rocshmem_amd_release_probe": (_i, [_i, _vp, _vp, _sz, _sz, _i, _i, _vp]),
    "rocshmem_amd_reuse_probe": (_i, [_vp, _sz, _sz, _i, _i, _i, _vp]),
}


class Library:
    """The loaded shared library with typed entry points as attributes
    (``lib.malloc`` is ``rocshmem_amd_malloc`` and so on)."""

    def __init__(self, path=LIB_PATH, signatures=None):
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is not built; run `make -C rocshmem_amd/csrc` "
                "(or __graft_entry__.build()). There is no CPU fallback.")
        self.path = path
        self.cdll = C.CDLL(path, mode=C.RTLD_GLOBAL)
        for name, (res, args) in (SIGNATURES if signatures is None else signatures).items():
            fn = getattr(self.cdll, name)
            fn.restype = res
            fn.argtypes = args
            setattr(self, name[len("rocshmem_amd_"):], fn)


_LIB = None


def load():
    global _LIB
    if _LIB is None:
        _LIB = Library()
    return _LIB


_PROBES = None


def load_probes():
    """The measuring probes; loads the product library first (they run on its
    runtime)."""
    global _PROBES
    load()
    if _PROBES is None:
        _PROBES = Library(PROBES_PATH, PROBE_SIGNATURES)
    return _PROBES
